"""The bodies of the XLA custom-call handlers (include/mdattn_marshal.h, what csrc/ffi/mdattn_ffi.cc forwards to) run on
real device buffers, described exactly as XLA describes them (dense, row-major, dtype + dimensions), and held bit for
bit to the torch-side operators of ops.py, which call the C ABI with their own strides.  Covers every custom-call
target, both layouts, the donated carries, the Flux text weights and the absent-k forms."""
import ctypes
import math

import pytest
import torch

from maxdiffusion_amd import ops

pytestmark = pytest.mark.gpu

_DT = {torch.bfloat16: 1, torch.float32: 2, torch.uint8: 3, torch.bool: 3, torch.float8_e4m3fn: 4}


class Buffer(ctypes.Structure):
  _fields_ = [("data", ctypes.c_void_p), ("dtype", ctypes.c_int32), ("rank", ctypes.c_int32), ("dims", ctypes.POINTER(ctypes.c_int64))]


def xb(t: torch.Tensor) -> Buffer:
  assert t.is_contiguous(), "XLA buffers are dense"
  dims = (ctypes.c_int64 * max(t.dim(), 1))(*t.shape)
  b = Buffer(t.data_ptr(), _DT[t.dtype], t.dim(), dims)
  b._keep = (dims, t)
  return b


def xla(lib, name, *args):
  fn = getattr(lib, "mdattn_xla_" + name)
  fn.restype = ctypes.c_int
  err = ctypes.create_string_buffer(512)
  conv = [ctypes.byref(xb(a)) if isinstance(a, torch.Tensor) else a for a in args]
  rc = fn(ctypes.c_void_p(torch.cuda.current_stream().cuda_stream), *conv, err, 512)
  assert rc == 0, err.value.decode()


f, i = ctypes.c_float, ctypes.c_int64


def _qkv(dev, B, Sq, Skv, H, D, seed):
  gen = torch.Generator(device=dev).manual_seed(seed)
  mk = lambda s: torch.randn((B, s, H, D), generator=gen, device=dev).to(torch.bfloat16)
  return mk(Sq), mk(Skv), mk(Skv)


@pytest.mark.parametrize("layout", [0, 1])
def test_forward_bias_and_mask_handlers(dev, lib, layout):
  B, Sq, Skv, H, D = 2, 130, 333, 3, 128
  q, k, v = _qkv(dev, B, Sq, Skv, H, D, 1)
  lay = (lambda t: t.permute(0, 2, 1, 3).contiguous()) if layout else (lambda t: t)   # what XLA holds: [B,H,S,D] dense
  view = (lambda t: t.permute(0, 2, 1, 3)) if layout else (lambda t: t)                # the logical [B,S,H,D] view of it
  qx, kx, vx = lay(q), lay(k), lay(v)
  out, lse = torch.empty((B, Sq, H, D), dtype=torch.bfloat16, device=dev), torch.empty((B, H, Sq), device=dev)
  xla(lib, "fwd_bf16", qx, kx, vx, out, lse, f(0.07), i(layout))
  want, want_l = ops.flash_attention(view(qx), view(kx), view(vx), scale=0.07, return_lse=True)
  assert torch.equal(out, want) and torch.equal(lse, want_l)
  keep = torch.rand((B, Skv), device=dev) < 0.6
  bias = torch.empty((B, (Skv + 31) // 32 * 32), device=dev)
  xla(lib, "key_mask_bias", keep, bias, f(-math.inf))
  assert torch.equal(bias, ops.key_mask_bias(keep))
  xla(lib, "fwd_bf16_bias", qx, kx, vx, bias, out, lse, f(0.07), i(layout))
  want, want_l = ops.flash_attention(view(qx), view(kx), view(vx), scale=0.07, return_lse=True, key_bias=bias)
  assert torch.equal(out, want) and torch.equal(lse, want_l)


def test_ring_merge_and_finalize_handlers(dev, lib):
  B, Sq, H, D = 1, 100, 2, 128
  q, k, v = _qkv(dev, B, Sq, 700, H, D, 2)
  o_x, l_x = ops.new_merge_state(B, Sq, H, D, dev)
  o_w, l_w = ops.new_merge_state(B, Sq, H, D, dev)
  for a, b in ((0, 300), (300, 700)):
    kc, vc = k[:, a:b].contiguous(), v[:, a:b].contiguous()
    xla(lib, "fwd_bf16_merge", q, kc, vc, o_x, l_x, o_x, l_x, f(0.09), i(0))  # donated: inputs alias results
    ops.flash_attention_merge(q, kc, vc, o_w, l_w, scale=0.09)
  assert torch.equal(o_x, o_w) and torch.equal(l_x, l_w)
  cur, cur_l = ops.flash_attention(q, k, v, scale=0.09, return_lse=True)
  xla(lib, "merge", o_x, l_x, cur, cur_l, o_x, l_x)
  ops.merge_partial(o_w, l_w, cur, cur_l)
  assert torch.equal(o_x, o_w) and torch.equal(l_x, l_w)
  fin = torch.empty((B, Sq, H, D), dtype=torch.bfloat16, device=dev)
  xla(lib, "finalize", o_x, fin)
  assert torch.equal(fin, ops.finalize(o_w))


def test_prologue_handlers(dev, lib):
  B, S, H, D = 2, 77, 4, 128
  gen = torch.Generator(device=dev).manual_seed(3)
  rn = lambda *s: torch.randn(s, generator=gen, device=dev)
  q, k = rn(B, S, H * D).to(torch.bfloat16), rn(B, S, H * D).to(torch.bfloat16)
  wq, wk = (1 + 0.1 * rn(H * D)).to(torch.bfloat16), (1 + 0.1 * rn(H * D)).to(torch.bfloat16)
  ang = rn(S, D // 2)
  cos, sin = torch.cos(ang), torch.sin(ang)
  qo, ko = (torch.empty((B, S, H, D), dtype=torch.bfloat16, device=dev) for _ in range(2))
  xla(lib, "norm_rope_fullrow", q, k, wq, wk, cos, sin, qo, ko, f(1e-6), f(1.25), i(H), i(1), i(1))
  wantq, wantk = ops.norm_rope_fullrow(q, k, wq, wk, cos, sin, H, q_mul=1.25)
  assert torch.equal(qo, wantq) and torch.equal(ko, wantk)
  # norm only, no k: the dummies XLA has to pass for absent buffers are ignored
  dummy, dummy_out = torch.zeros(8, device=dev), torch.zeros(8, dtype=torch.bfloat16, device=dev)
  xla(lib, "norm_rope_fullrow", q, q, wq, wq, dummy, dummy, qo, dummy_out, f(1e-6), f(1.0), i(H), i(0), i(0))
  assert torch.equal(qo, ops.norm_rope_fullrow(q, None, wq, None, None, None, H)[0])
  # the fused q|k|v projection form, with and without the projection biases
  qkv, b3 = rn(B, S, 3 * H * D).to(torch.bfloat16), (0.5 * rn(3 * H * D)).to(torch.bfloat16)
  vo = torch.empty((B, S, H, D), dtype=torch.bfloat16, device=dev)
  xla(lib, "norm_rope_qkv", qkv, b3, wq, wk, cos, sin, qo, ko, vo, f(1e-6), f(1.25), i(H), i(1), i(1), i(1))
  want = ops.norm_rope_qkv(qkv, wq, wk, cos, sin, H, bias=b3, q_mul=1.25)
  assert all(torch.equal(a_, b_) for a_, b_ in zip((qo, ko, vo), want))
  xla(lib, "norm_rope_qkv", qkv, wq, wq, wk, cos, sin, qo, ko, dummy_out, f(1e-6), f(1.0), i(H), i(1), i(0), i(0))
  want = ops.norm_rope_qkv(qkv, wq, wk, cos, sin, H)
  assert torch.equal(qo, want[0]) and torch.equal(ko, want[1])
  # per head, with the text-token weights of Flux's double blocks
  q4, k4 = q.view(B, S, H, D), k.view(B, S, H, D)
  w = [(1 + 0.1 * rn(D)).to(torch.bfloat16) for _ in range(4)]
  xla(lib, "norm_rope_perhead", q4, k4, w[0], w[1], w[2], w[3], cos, sin, qo, ko, f(1e-6), f(1.0), i(20), i(1), i(1))
  wantq, wantk = ops.norm_rope_perhead(q4, k4, w[0], w[1], cos, sin, wq_txt=w[2], wk_txt=w[3], n_txt=20)
  assert torch.equal(qo, wantq) and torch.equal(ko, wantk)
  assert not torch.equal(qo, ops.norm_rope_perhead(q4, k4, w[0], w[1], cos, sin)[0])  # the text weights do matter
  # LTX-2 rows: f32 input, interleaved and split tables
  x, wf = rn(B, S, H * D), 1 + 0.1 * rn(H * D)
  ci, si = torch.cos(rn(B, S, H * D)), torch.sin(rn(B, S, H * D))
  xla(lib, "norm_rope_rows", x, wf, ci, si, qo, f(1e-6), i(H), i(1))
  assert torch.equal(qo, ops.norm_rope_rows(x, wf, ci, si, heads=H, mode="interleaved"))
  cs, ss = torch.cos(rn(B, H, S, D // 2)), torch.sin(rn(B, H, S, D // 2))
  xla(lib, "norm_rope_rows", x.to(torch.bfloat16), wf, cs, ss, qo, f(1e-6), i(H), i(2))
  assert torch.equal(qo, ops.norm_rope_rows(x.to(torch.bfloat16), wf, cs, ss, heads=H, mode="split"))
  xla(lib, "norm_rope_rows", x, wf, dummy, dummy, qo, f(1e-6), i(H), i(0))
  assert torch.equal(qo, ops.norm_rope_rows(x, wf, heads=H, mode="none"))


@pytest.mark.parametrize("softmax", ["exp2", "byte_grid"])
def test_fp8_handlers(dev, lib, softmax):
  B, Sq, Skv, H, D = 1, 200, 500, 2, 128
  q, k, v = _qkv(dev, B, Sq, Skv, H, D, 4)
  xs, want = [], []
  for t, pm, p2 in ((q, ops.folded_q_mul(D), 1), (k, 1.0, 1), (v, 1.0, 0)):
    x8, sc = torch.empty(t.shape, dtype=torch.float8_e4m3fn, device=dev), torch.empty(2, device=dev)
    xla(lib, "quant_e4m3", t, x8, sc, f(pm), i(p2))
    w8, wsc = ops.quant_e4m3(t, premul=pm, pow2_scale=bool(p2))
    assert torch.equal(x8.view(torch.uint8), w8) and torch.equal(sc, wsc)
    xs.append((x8, sc))
    want.append((w8, wsc))
  out, lse = torch.empty((B, Sq, H, D), dtype=torch.bfloat16, device=dev), torch.empty((B, H, Sq), device=dev)
  xla(lib, "fwd_fp8", xs[0][0], xs[1][0], xs[2][0], xs[0][1], xs[1][1], xs[2][1], out, lse, f(ops.FOLDED_SCALE), i(0),
      i(ops.FP8_SOFTMAX_MODES[softmax]))
  w_out, w_lse = ops.flash_attention_fp8(want[0][0], want[1][0], want[2][0], want[0][1], want[1][1], want[2][1],
                                         scale=ops.FOLDED_SCALE, return_lse=True, softmax=softmax)
  assert torch.equal(out, w_out) and torch.equal(lse, w_lse)
  bias = ops.key_mask_bias(torch.rand((B, Skv), device=dev) < 0.6)
  xla(lib, "fwd_fp8_bias", xs[0][0], xs[1][0], xs[2][0], xs[0][1], xs[1][1], xs[2][1], bias, out, lse, f(ops.FOLDED_SCALE), i(0))
  w_out, w_lse = ops.flash_attention_fp8(want[0][0], want[1][0], want[2][0], want[0][1], want[1][1], want[2][1],
                                         scale=ops.FOLDED_SCALE, return_lse=True, key_bias=bias)
  assert torch.equal(out, w_out) and torch.equal(lse, w_lse)


def test_backward_handlers(dev, lib):
  B, Sq, Skv, H, D = 2, 150, 260, 3, 128
  q, k, v = _qkv(dev, B, Sq, Skv, H, D, 5)
  dout = torch.randn((B, Sq, H, D), device=dev).to(torch.bfloat16)
  out, lse = ops.flash_attention(q, k, v, scale=0.08, return_lse=True)
  want = ops.flash_attention_backward(q, k, v, out, dout, lse, scale=0.08)
  dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
  ws = torch.empty(lib.mdattn_bwd_workspace_floats(B, H, Sq), device=dev)
  xla(lib, "bwd_bf16", q, k, v, out, dout, lse, dq, dk, dv, ws, f(0.08))
  assert all(torch.equal(a, b) for a, b in zip((dq, dk, dv), want))
  dq, dk, dv = torch.zeros_like(q), torch.zeros_like(k), torch.zeros_like(v)
  xla(lib, "bwd_bf16_static", q, k, v, out, dout, lse, dq, dk, dv, f(0.08))
  assert all(torch.equal(a, b) for a, b in zip((dq, dk, dv), want))
  bias = ops.key_mask_bias(torch.rand((B, Skv), device=dev) < 0.6)
  out, lse = ops.flash_attention(q, k, v, scale=0.08, return_lse=True, key_bias=bias)
  want = ops.flash_attention_backward(q, k, v, out, dout, lse, scale=0.08, key_bias=bias)
  xla(lib, "bwd_bf16_bias", q, k, v, out, dout, lse, bias, dq, dk, dv, ws, f(0.08))
  assert all(torch.equal(a, b) for a, b in zip((dq, dk, dv), want))


def test_prologue_backward_handlers(dev, lib):
  """The three prologue-backward targets on XLA-shaped buffers (dense, the workspace as a result), bit for bit against the
  torch-side operators; absent-k and no-text-weight forms pass small stand-in buffers, as the Python wrappers do."""
  B, S, H, D = 2, 45, 4, 128
  N = H * D
  gen = torch.Generator(device=dev).manual_seed(5)
  rnd = lambda *s: torch.randn(s, generator=gen, device=dev).to(torch.bfloat16)
  q, k, gq, gk = rnd(B, S, N), rnd(B, S, N), rnd(B, S, H, D), rnd(B, S, H, D)
  wq, wk = (1 + 0.1 * rnd(N).float()).to(torch.bfloat16), (1 + 0.1 * rnd(N).float()).to(torch.bfloat16)
  ang = torch.rand((S, D // 2), generator=gen, device=dev) * 6.28
  cos, sin = torch.cos(ang), torch.sin(ang)
  bias = (0.5 * rnd(2 * N).float()).to(torch.bfloat16)
  e = lambda *s, dt=torch.float32: torch.empty(s, dtype=dt, device=dev)
  small_b, small_f = e(8, dt=torch.bfloat16), e(8)
  # full row, q and k, with the projection biases
  dq, dk, dwq, dwk, db = e(B, S, N, dt=torch.bfloat16), e(B, S, N, dt=torch.bfloat16), e(N), e(N), e(2 * N)
  ws = e(min(B * S, 1024) * 4 * N)
  xla(lib, "norm_rope_fullrow_bwd", q, k, gq, gk, wq, wk, cos, sin, bias, dq, dk, dwq, dwk, db, ws, f(1e-6), f(0.5), i(H), i(1), i(1), i(1))
  want = ops.norm_rope_fullrow_backward(q, k, wq, wk, cos, sin, H, gq, gk, q_mul=0.5, bias=bias)
  for got, w_ in zip((dq, dk, dwq, dwk, db), want):
    assert torch.equal(got, w_)
  # q alone, norm only: stand-ins for everything of k, for the tables and for the bias
  ws1 = e(min(B * S, 1024) * N)
  xla(lib, "norm_rope_fullrow_bwd", q, q, gq, gq, wq, wq, small_f, small_f, wq, dq, small_b, dwq, small_f, small_f, ws1, f(1e-6), f(1.0), i(H),
      i(0), i(0), i(0))
  want = ops.norm_rope_fullrow_backward(q, None, wq, None, None, None, H, gq, None)
  assert torch.equal(dq, want[0]) and torch.equal(dwq, want[2])
  # per head, text weights on the first 7 tokens
  q4, k4 = q.view(B, S, H, D), k.view(B, S, H, D)
  wd = [(1 + 0.1 * rnd(D).float()).to(torch.bfloat16) for _ in range(4)]
  dq4, dk4 = e(B, S, H, D, dt=torch.bfloat16), e(B, S, H, D, dt=torch.bfloat16)
  dws = [e(D) for _ in range(4)]
  wsh = e(min(B * S * H, 1024) * 4 * D)
  xla(lib, "norm_rope_perhead_bwd", q4, k4, gq, gk, wd[0], wd[1], wd[2], wd[3], cos, sin, dq4, dk4, dws[0], dws[1], dws[2], dws[3], wsh,
      f(1e-6), f(1.0), i(7), i(1), i(1))
  want = ops.norm_rope_perhead_backward(q4, k4, wd[0], wd[1], cos, sin, gq, gk, wq_txt=wd[2], wk_txt=wd[3], n_txt=7)
  for got, w_ in zip((dq4, dk4, *dws), want):
    assert torch.equal(got, w_)
  # rows (LTX-2), f32 input, split tables
  x = torch.randn((B, S, N), generator=gen, device=dev)
  w32 = 1 + 0.1 * torch.randn(N, generator=gen, device=dev)
  angs = torch.rand((B, H, S, D // 2), generator=gen, device=dev) * 6.28
  cs, sn = torch.cos(angs), torch.sin(angs)
  dx, dw, wsr = e(B, S, N), e(N), e(min(B * S, 1024) * N)
  xla(lib, "norm_rope_rows_bwd", x, gq, w32, cs, sn, dx, dw, wsr, f(1e-6), i(H), i(2))
  want = ops.norm_rope_rows_backward(x, w32, gq, cs, sn, heads=H, mode="split")
  assert torch.equal(dx, want[0]) and torch.equal(dw, want[1])
