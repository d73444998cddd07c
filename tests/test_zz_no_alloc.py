"""The entry point that allocates nothing, `mdattn_bwd_bf16_static` (backward with its lse / delta scratch in a static
device array of the library), called through the C ABI and held bit for bit to `mdattn_bwd_bf16` with a
caller-provided workspace: two calls in a row on the shared array, the second on a smaller input."""
import ctypes

import pytest
import torch

from maxdiffusion_amd import _lib, ops

pytestmark = pytest.mark.gpu


def _case(dev, lib, B, H, sq, skv, seed, layout="bshd"):
  gen = torch.Generator(device=dev).manual_seed(seed)

  def mk(S):
    x = torch.randn((B, S, H, 128), generator=gen, device=dev, dtype=torch.float32).to(torch.bfloat16)
    return x.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3) if layout == "bhsd" else x

  q, k, v, dout = mk(sq), mk(skv), mk(skv), mk(sq)
  out, lse = ops.flash_attention(q, k, v, return_lse=True, out_layout=layout)
  want = ops.flash_attention_backward(q, k, v, out, dout, lse)  # mdattn_bwd_bf16, workspace from torch
  # everything the static entry point touches exists before the call: it must not allocate
  got = tuple(torch.full_like(t, float("nan")) for t in (q, k, v))
  assert lib.mdattn_bwd_static_max_floats() == 8 * 1024 * 1024  # the documented warm-up: resolves the array's address
  torch.cuda.synchronize()
  before = torch.cuda.memory_allocated(dev)
  free_before = torch.cuda.mem_get_info(dev)[0]  # the driver's own count: sees a hipMalloc that torch's allocator would not
  P, S = ctypes.c_void_p, _lib.Strides
  st = lambda t: ctypes.byref(S(t.stride(0), t.stride(1), t.stride(2)))
  rc = lib.mdattn_bwd_bf16_static(
      P(torch.cuda.current_stream().cuda_stream), P(q.data_ptr()), P(k.data_ptr()), P(v.data_ptr()), P(out.data_ptr()),
      P(dout.data_ptr()), P(lse.data_ptr()), P(got[0].data_ptr()), P(got[1].data_ptr()), P(got[2].data_ptr()),
      B, H, sq, skv, 128, st(q), st(k), st(v), st(out), 128**-0.5)
  assert rc == _lib.E_OK, _lib.strerror(rc)
  torch.cuda.synchronize()
  assert torch.cuda.memory_allocated(dev) == before
  assert torch.cuda.mem_get_info(dev)[0] == free_before
  for name, g, w in zip(("dq", "dk", "dv"), got, want):
    assert bool(torch.isfinite(g.float()).all()), f"{name} B={B} H={H} Sq={sq} Skv={skv}"
    assert torch.equal(g, w), f"{name} differs from mdattn_bwd_bf16: B={B} H={H} Sq={sq} Skv={skv} {layout}"


def test_static_backward_equals_workspace_backward_on_two_calls_in_a_row(dev, lib):
  print("mdattn_bwd_bf16_static: B=2 H=3 Sq=300 Skv=333, then B=1 H=2 Sq=65 Skv=31 (bhsd)", flush=True)
  _case(dev, lib, 2, 3, 300, 333, seed=21)
  _case(dev, lib, 1, 2, 65, 31, seed=22, layout="bhsd")  # smaller: the array still holds the first call's values
  _case(dev, lib, 2, 3, 300, 333, seed=21)               # and back, through the ops wrapper's twin below


def test_ops_wrapper_and_size_limit(dev, lib):
  gen = torch.Generator(device=dev).manual_seed(5)
  q, k, v, dout = (torch.randn((1, s, 2, 128), generator=gen, device=dev).to(torch.bfloat16) for s in (130, 70, 70, 130))
  out, lse = ops.flash_attention(q, k, v, return_lse=True)
  want = ops.flash_attention_backward(q, k, v, out, dout, lse)
  got = ops.flash_attention_backward_static(q, k, v, out, dout, lse, *(torch.empty_like(t) for t in (q, k, v)))
  for g, w in zip(got, want):
    assert torch.equal(g, w)
  # beyond the static array: rejected on the host, nothing is launched (the pointers are never dereferenced)
  assert lib.mdattn_bwd_static_max_floats() == 8 * 1024 * 1024
  fake = ctypes.c_void_p(0x1000)
  s = ctypes.byref(_lib.Strides(0, 64 * 128, 128))
  rc = lib.mdattn_bwd_bf16_static(None, fake, fake, fake, fake, fake, fake, fake, fake, fake, 1, 64, 70000, 128, 128, s, s, s, s, 0.1)
  assert rc == _lib.E_TOOBIG and b"static scratch" in lib.mdattn_strerror(rc)
  # the largest request that fits is accepted by the size check (and then fails the next check: null q)
  rc = lib.mdattn_bwd_bf16_static(None, None, fake, fake, fake, fake, fake, fake, fake, fake, 1, 64, 65536, 128, 128, s, s, s, s, 0.1)
  assert rc == _lib.E_BADARG
