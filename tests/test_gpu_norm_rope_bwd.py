"""Parity of the prologue's backward HIP kernels (through the C ABI) against the CPU oracle.

Bars: the input gradients leave the kernel with one bf16 rounding of an f32 result, so they are held to the forward's
bars (max-abs <= 2e-2, mean-abs <= 2e-3 for gradients of unit scale) and to rel-L2 <= 4e-3; the weight gradients are
f32 sums over tokens and are held to rel-L2 <= 1e-4 of the f64 oracle (measured: ~1e-6)."""
import numpy as np
import pytest
import torch

import oracle as O
from helpers import bits_to_dev, bits_to_f32, err_stats, golden, rel_l2, to_dev_bf16, to_np
from maxdiffusion_amd import ops

pytestmark = pytest.mark.gpu


def _t(x, dev):
  return torch.from_numpy(np.ascontiguousarray(x)).to(dev)


def _close_dx(got, ref, what, scale=1.0):
  mx, mean = err_stats(got, ref)
  rl = rel_l2(got, ref)
  print(f"{what}: max-abs {mx:.3e} mean-abs {mean:.3e} rel-l2 {rl:.3e}", flush=True)
  assert mx <= 2e-2 * scale and mean <= 2e-3 * scale and rl <= 4e-3, what


def _close_dw(got, ref, what):
  rl = rel_l2(got, ref)
  print(f"{what}: rel-l2 {rl:.3e}", flush=True)
  assert rl <= 1e-4, what


def test_golden_wan(dev):
  g = golden("norm_rope_bwd.npz")
  H, m = int(g["wan_heads"]), float(g["wan_q_mul"])
  q, k, wq, wk, gq, gk, bias = (bits_to_dev(g["wan_" + n], dev) for n in ("q", "k", "wq", "wk", "gq", "gk", "bias"))
  cos, sin = _t(g["wan_cos"], dev), _t(g["wan_sin"], dev)
  for layout in ("bshd", "bhsd"):
    gq_l = gq if layout == "bshd" else gq.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    gk_l = gk if layout == "bshd" else gk.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    dq, dk, dwq, dwk = ops.norm_rope_fullrow_backward(q, k, wq, wk, cos, sin, H, gq_l, gk_l, q_mul=m)
    _close_dx(to_np(dq), g["wan_dq"], f"wan dq {layout}", scale=0.25)
    _close_dx(to_np(dk), g["wan_dk"], f"wan dk {layout}")
    _close_dw(to_np(dwq), g["wan_dwq"], "wan dwq")
    _close_dw(to_np(dwk), g["wan_dwk"], "wan dwk")
  # q alone, norm only (the cached-text-KV cross-attention case)
  dq, dk, dwq, dwk = ops.norm_rope_fullrow_backward(q, None, wq, None, None, None, H, gq, None)
  assert dk is None and dwk is None
  _close_dx(to_np(dq), g["wan_dq_norm_only"], "wan dq norm only")
  _close_dw(to_np(dwq), g["wan_dwq_norm_only"], "wan dwq norm only")
  # with the projection biases of the fused q|k|v form
  dq, dk, dwq, dwk, db = ops.norm_rope_fullrow_backward(q, k, wq, wk, cos, sin, H, gq, gk, q_mul=m, bias=bias)
  _close_dx(to_np(dq), g["wan_dq_bias"], "wan dq bias", scale=0.25)
  _close_dx(to_np(dk), g["wan_dk_bias"], "wan dk bias")
  _close_dw(to_np(dwq), g["wan_dwq_bias"], "wan dwq bias")
  _close_dw(to_np(dwk), g["wan_dwk_bias"], "wan dwk bias")
  n = q.shape[2]
  want_db = np.concatenate([g["wan_dq_bias"].reshape(-1, n).sum(0), g["wan_dk_bias"].reshape(-1, n).sum(0)])
  _close_dw(to_np(db), want_db, "wan dbias")


def test_golden_flux(dev):
  g = golden("norm_rope_bwd.npz")
  q, k, gq, gk = (bits_to_dev(g["flux_" + n], dev) for n in ("q", "k", "gq", "gk"))
  w = [bits_to_dev(g["flux_" + n], dev) for n in ("wq", "wk", "wq_txt", "wk_txt")]
  cos, sin = _t(g["flux_cos"], dev), _t(g["flux_sin"], dev)
  res = ops.norm_rope_perhead_backward(q, k, w[0], w[1], cos, sin, gq, gk, wq_txt=w[2], wk_txt=w[3], n_txt=int(g["flux_n_txt"]),
                                       q_mul=float(g["flux_q_mul"]))
  _close_dx(to_np(res[0]), g["flux_dq"], "flux dq", scale=0.25)
  _close_dx(to_np(res[1]), g["flux_dk"], "flux dk")
  for got, name in zip(res[2:], ("dwq", "dwk", "dwq_txt", "dwk_txt")):
    _close_dw(to_np(got), g["flux_" + name], "flux " + name)


def test_golden_ltx2(dev):
  g = golden("norm_rope_bwd.npz")
  H = int(g["ltx2_heads"])
  x, gr = bits_to_dev(g["ltx2_x"], dev), bits_to_dev(g["ltx2_g"], dev)
  w = _t(g["ltx2_w"], dev)
  tabs = {"none": (None, None), "interleaved": (_t(g["ltx2_cos_i"], dev), _t(g["ltx2_sin_i"], dev)),
          "split": (_t(g["ltx2_cos_s"], dev), _t(g["ltx2_sin_s"], dev))}
  for mode, (c, s) in tabs.items():
    for f32_in in (False, True):
      xin = x.float() if f32_in else x
      dx, dw = ops.norm_rope_rows_backward(xin, w, gr, c, s, heads=H, mode=mode)
      assert dx.dtype == xin.dtype
      _close_dx(to_np(dx), g["ltx2_dx_" + mode], f"ltx2 dx {mode} f32_in={f32_in}", scale=2.0)
      _close_dw(to_np(dw), g["ltx2_dw_" + mode], f"ltx2 dw {mode}")
      if f32_in:  # f32 output: no bf16 rounding at all
        assert rel_l2(to_np(dx), g["ltx2_dx_" + mode]) <= 1e-5


@pytest.mark.parametrize("layout", ["bshd", "bhsd"])
def test_wan13b_full_size(dev, layout):
  """The Wan-1.3B benchmark shape whole: every token of the Wan-1.3B shape, both tensors, against the f64 oracle."""
  w = O.WORKLOADS["wan1.3b"]
  H, D, S = w.heads, w.head_dim, w.seq
  q, k = O.normal_bf16((1, S, H * D), 0), O.normal_bf16((1, S, H * D), 1)
  gq, gk = O.normal_bf16((1, S, H, D), 7), O.normal_bf16((1, S, H, D), 8)
  wq, wk = O.norm_weight(H * D, 3), O.norm_weight(H * D, 4)
  cos, sin = O.wan_rope_table(w.grid, D)
  m = ops.folded_q_mul(D)
  lay = (lambda t: t) if layout == "bshd" else (lambda t: t.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3))
  dq, dk, dwq, dwk = ops.norm_rope_fullrow_backward(
      to_dev_bf16(q, dev), to_dev_bf16(k, dev), to_dev_bf16(wq, dev), to_dev_bf16(wk, dev), _t(cos, dev), _t(sin, dev), H,
      lay(to_dev_bf16(gq, dev)), lay(to_dev_bf16(gk, dev)), q_mul=m)
  rq, rwq = O.norm_rope_fullrow_bwd(q, wq, cos, sin, H, gq, q_mul=m)
  rk, rwk = O.norm_rope_fullrow_bwd(k, wk, cos, sin, H, gk)
  _close_dx(to_np(dq), rq, "wan1.3b dq", scale=m)
  _close_dx(to_np(dk), rk, "wan1.3b dk")
  _close_dw(to_np(dwq), rwq, "wan1.3b dwq")
  _close_dw(to_np(dwk), rwk, "wan1.3b dwk")


def test_flux_dev_full_size(dev):
  """The Flux-dev benchmark shape whole: 512 text + 4096 image tokens x 24 heads, separate text weights."""
  w = O.WORKLOADS["flux-dev"]
  n_txt, rows, cols = w.grid
  ids = O.flux_ids(n_txt, rows, cols)
  L = ids.shape[0]
  q, k = O.normal_bf16((1, L, w.heads, 128), 0), O.normal_bf16((1, L, w.heads, 128), 1)
  gq, gk = O.normal_bf16((1, L, w.heads, 128), 7), O.normal_bf16((1, L, w.heads, 128), 8)
  wq, wk, wqt, wkt = (O.norm_weight(128, s) for s in (3, 4, 5, 6))
  cos, sin = O.flux_rope_table(ids)
  res = ops.norm_rope_perhead_backward(*(to_dev_bf16(x, dev) for x in (q, k, wq, wk)), _t(cos, dev), _t(sin, dev),
                                       to_dev_bf16(gq, dev), to_dev_bf16(gk, dev), wq_txt=to_dev_bf16(wqt, dev),
                                       wk_txt=to_dev_bf16(wkt, dev), n_txt=n_txt)
  rq, rwq, rwqt = O.norm_rope_perhead_bwd(q, wq, cos, sin, gq, w_txt=wqt, n_txt=n_txt)
  rk, rwk, rwkt = O.norm_rope_perhead_bwd(k, wk, cos, sin, gk, w_txt=wkt, n_txt=n_txt)
  _close_dx(to_np(res[0]), rq, "flux-dev dq")
  _close_dx(to_np(res[1]), rk, "flux-dev dk")
  for got, ref, name in zip(res[2:], (rwq, rwk, rwqt, rwkt), ("dwq", "dwk", "dwq_txt", "dwk_txt")):
    _close_dw(to_np(got), ref, "flux-dev " + name)


def test_wan14b_full_size_sampled_rows(dev):
  """The Wan-14B benchmark shape at full size: the input gradients on a deterministic sample of token rows against the f64
  oracle (a row's gradient depends on that row only); the weight gradients, sums over all 75,600 tokens, against the
  same formula evaluated by torch in f64 on the GPU from the kernel-independent inputs (test harness only)."""
  w = O.WORKLOADS["wan14b"]
  H, D, S = w.heads, w.head_dim, w.seq
  gen = torch.Generator(device=dev).manual_seed(0)
  rnd = lambda *shape: torch.randn(shape, generator=gen, device=dev, dtype=torch.float32).to(torch.bfloat16)
  q, k, gq, gk = rnd(1, S, H * D), rnd(1, S, H * D), rnd(1, S, H, D), rnd(1, S, H, D)
  wq, wk = O.norm_weight(H * D, 3), O.norm_weight(H * D, 4)
  cos, sin = O.wan_rope_table(w.grid, D)
  wq_d, wk_d, cos_d, sin_d = to_dev_bf16(wq, dev), to_dev_bf16(wk, dev), _t(cos, dev), _t(sin, dev)
  m = ops.folded_q_mul(D)
  dq, dk, dwq, dwk = ops.norm_rope_fullrow_backward(q, k, wq_d, wk_d, cos_d, sin_d, H, gq, gk, q_mul=m)
  rows = O.sample_rows(S)
  idx = torch.from_numpy(rows).to(dev)
  for x, g_, wt, dx, mul, name in ((q, gq, wq, dq, m, "q"), (k, gk, wk, dk, 1.0, "k")):
    ref, _ = O.norm_rope_fullrow_bwd(to_np(x[:, idx]), wt, cos[rows], sin[rows], H, to_np(g_[:, idx]), q_mul=mul)
    _close_dx(to_np(dx[:, idx]), ref, f"wan14b d{name} sampled rows", scale=mul)
  # dw = sum_tokens (R^T g * mul) * x * r, evaluated in f64 in chunks of tokens
  for x, g_, got, mul, name in ((q, gq, dwq, m, "q"), (k, gk, dwk, 1.0, "k")):
    acc = torch.zeros(H * D, dtype=torch.float64, device=dev)
    for s0 in range(0, S, 8192):
      xs = x[0, s0:s0 + 8192].double()
      gs = g_[0, s0:s0 + 8192].double().view(-1, H, D // 2, 2)
      c, s_ = cos_d[s0:s0 + 8192].double()[:, None, :], sin_d[s0:s0 + 8192].double()[:, None, :]
      dy = torch.stack([gs[..., 0] * c + gs[..., 1] * s_, gs[..., 1] * c - gs[..., 0] * s_], dim=-1).reshape(-1, H * D) * mul
      r = torch.rsqrt(xs.pow(2).mean(-1, keepdim=True) + 1e-6)
      acc += (dy * xs * r).sum(0)
    _close_dw(to_np(got), acc.cpu().numpy(), f"wan14b dw{name} (all tokens)")


def test_fused_qkv_gradient_buffer_and_determinism(dev):
  """The q | k blocks of a fused [B,S,3*H*D] gradient buffer written in place (dx strides of 3*H*D), equal to the
  dense result bit for bit; two runs give identical bits (no atomics anywhere)."""
  B, H, D, grid = 2, 6, 128, (2, 5, 7)
  S, N = grid[0] * grid[1] * grid[2], 6 * 128
  qkv = to_dev_bf16(O.normal_bf16((B, S, 3 * N), 0), dev)
  gq, gk = to_dev_bf16(O.normal_bf16((B, S, H, D), 7), dev), to_dev_bf16(O.normal_bf16((B, S, H, D), 8), dev)
  wq, wk = to_dev_bf16(O.norm_weight(N, 3), dev), to_dev_bf16(O.norm_weight(N, 4), dev)
  bias = to_dev_bf16(O.bf16_round(0.5 * O.normal_bf16((2 * N,), 9)), dev)
  cos, sin = (_t(t, dev) for t in O.wan_rope_table(grid, D))
  q, k = qkv[:, :, :N], qkv[:, :, N:2 * N]
  dense = ops.norm_rope_fullrow_backward(q.contiguous(), k.contiguous(), wq, wk, cos, sin, H, gq, gk, bias=bias)
  dqkv = torch.zeros_like(qkv)
  fused = ops.norm_rope_fullrow_backward(q, k, wq, wk, cos, sin, H, gq, gk, bias=bias, dq=dqkv[:, :, :N], dk=dqkv[:, :, N:2 * N])
  assert torch.equal(dqkv[:, :, :N], dense[0]) and torch.equal(dqkv[:, :, N:2 * N], dense[1])
  assert not dqkv[:, :, 2 * N:].any()  # the v block is the attention backward's to fill
  for a, b in zip(dense[2:], fused[2:]):
    assert torch.equal(a, b)
  again = ops.norm_rope_fullrow_backward(q, k, wq, wk, cos, sin, H, gq, gk, bias=bias)
  for a, b in zip(fused[2:], again[2:]):
    assert torch.equal(a, b)
  # against the oracle
  x = to_np(qkv)
  rq, rwq = O.norm_rope_fullrow_bwd(x[:, :, :N], to_np(wq), to_np(cos), to_np(sin), H, to_np(gq), bias=to_np(bias[:N]))
  _close_dx(to_np(dense[0]), rq, "fused dq")
  _close_dw(to_np(dense[2]), rwq, "fused dwq")
  _close_dw(to_np(dense[4])[:N], rq.reshape(-1, N).sum(0), "fused dbias q")


def test_edges_and_validation(dev, lib):
  import ctypes
  from maxdiffusion_amd import _lib

  # a single token, and head dims 64 / 256 of the per-head kernel
  H, D = 4, 128
  x, g = O.normal_bf16((1, 1, H * D), 1), O.normal_bf16((1, 1, H, D), 2)
  w = O.norm_weight(H * D, 3)
  dq, _, dwq, _ = ops.norm_rope_fullrow_backward(to_dev_bf16(x, dev), None, to_dev_bf16(w, dev), None, None, None, H, to_dev_bf16(g, dev), None)
  rq, rw = O.norm_rope_fullrow_bwd(x, w, None, None, H, g)
  _close_dx(to_np(dq), rq, "single token dq")
  _close_dw(to_np(dwq), rw, "single token dw")
  for d in (64, 256):
    x, g = O.normal_bf16((1, 19, 3, d), 11), O.normal_bf16((1, 19, 3, d), 12)
    wd = O.norm_weight(d, 13)
    ang = np.random.default_rng(14).uniform(-3, 3, (19, d // 2))
    c, s = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    res = ops.norm_rope_perhead_backward(to_dev_bf16(x, dev), None, to_dev_bf16(wd, dev), None, _t(c, dev), _t(s, dev), to_dev_bf16(g, dev), None)
    rx, rw, _ = O.norm_rope_perhead_bwd(x, wd, c, s, g)
    _close_dx(to_np(res[0]), rx, f"perhead D={d} dx")
    _close_dw(to_np(res[2]), rw, f"perhead D={d} dw")
  # host-side rejections (nothing is launched)
  fake = ctypes.c_void_p(0x1000)
  st = ctypes.byref(_lib.Strides(8 * 512, 512, 128))
  full = lambda **kw: lib.mdattn_norm_rope_fullrow_bwd(*[kw.get(n, v) for n, v in (
      ("stream", None), ("q", fake), ("k", None), ("bias", None), ("gq", fake), ("gk", None), ("dq", fake), ("dk", None), ("wq", fake),
      ("wk", None), ("dwq", fake), ("dwk", None), ("dbias", None), ("cos", None), ("sin", None), ("B", 1), ("S", 8), ("H", 4), ("D", 128),
      ("eps", 1e-6), ("q_mul", 1.0), ("isb", 0), ("iss", 512), ("dsb", 0), ("dss", 512), ("gs", st), ("ws", fake), ("nws", 4096))])
  assert full(ws=None) == _lib.E_BADARG
  assert full(nws=100) == _lib.E_BADARG                      # not even one partial row
  assert full(gk=fake) == _lib.E_BADARG                      # gk without k
  assert full(bias=fake, dbias=fake) == _lib.E_BADARG        # the bias form needs both tensors
  assert full(dq=ctypes.c_void_p(0x1004)) == _lib.E_ALIGN
  assert full(iss=256) == _lib.E_BADARG                      # row stride below H*D
  assert lib.mdattn_norm_rope_bwd_workspace_floats(75600, 10240) == 1024 * 10240
  assert lib.mdattn_norm_rope_bwd_workspace_floats(7, 512) == 7 * 512
