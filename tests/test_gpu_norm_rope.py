"""Parity of the fused RMSNorm + RoPE HIP kernels (through the C ABI) against the CPU oracle.

Bars (the benchmark's stated tolerances): max-abs <= 2e-2 and mean-abs <= 2e-3 against the f32/f64 oracle.
The kernel computes in f32 and rounds once, so the observed error is one bf16 rounding."""
import numpy as np
import pytest
import torch

import oracle as O
from helpers import bits_to_dev, bits_to_f32, err_stats, golden, to_dev_bf16, to_np
from maxdiffusion_amd import ops

pytestmark = pytest.mark.gpu
MAX_ABS, MEAN_ABS = 2e-2, 2e-3


def _assert_close(got, ref, what):
  mx, mean = err_stats(got, ref)
  print(f"{what}: max-abs {mx:.3e} mean-abs {mean:.3e}", flush=True)
  assert mx <= MAX_ABS and mean <= MEAN_ABS, f"{what}: max-abs {mx:.3e} mean-abs {mean:.3e}"
  # one bf16 rounding of |y| < 8 is at most 2^-6 = 1.5625e-2 (half ulp of [4,8)): the kernel rounds once
  assert mx <= 1.6e-2


def _t(x, dev):
  return torch.from_numpy(x).to(dev)


def test_golden_wan(dev):
  g = golden("norm_rope_wan.npz")
  H = int(g["heads"])
  q, k = bits_to_dev(g["q"], dev), bits_to_dev(g["k"], dev)
  wq, wk = bits_to_dev(g["wq"], dev), bits_to_dev(g["wk"], dev)
  cos, sin = _t(g["cos"], dev), _t(g["sin"], dev)
  for layout in ("bshd", "bhsd"):
    qo, ko = ops.norm_rope_fullrow(q, k, wq, wk, cos, sin, H, out_layout=layout)
    assert (qo.permute(0, 2, 1, 3).is_contiguous() if layout == "bhsd" else qo.is_contiguous())
    _assert_close(to_np(qo), g["q_out"], f"wan golden q {layout}")
    _assert_close(to_np(ko), g["k_out"], f"wan golden k {layout}")
  qn, kn = ops.norm_rope_fullrow(q, None, wq, None, None, None, H)  # norm only, q only (cached text KV case)
  assert kn is None
  _assert_close(to_np(qn), g["q_norm_only"], "wan golden norm-only")


def test_golden_flux(dev):
  g = golden("norm_rope_flux.npz")
  q, k = bits_to_dev(g["q"], dev), bits_to_dev(g["k"], dev)
  w = [bits_to_dev(g[n], dev) for n in ("wq", "wk", "wq_txt", "wk_txt")]
  qo, ko = ops.norm_rope_perhead(q, k, w[0], w[1], _t(g["cos"], dev), _t(g["sin"], dev), wq_txt=w[2], wk_txt=w[3], n_txt=int(g["n_txt"]))
  _assert_close(to_np(qo), g["q_out"], "flux golden q")
  _assert_close(to_np(ko), g["k_out"], "flux golden k")


@pytest.mark.parametrize("layout", ["bshd", "bhsd"])
def test_wan13b_full_size(dev, layout):
  w = O.WORKLOADS["wan1.3b"]
  H, D, S = w.heads, w.head_dim, w.seq
  q, k = O.normal_bf16((1, S, H * D), 0), O.normal_bf16((1, S, H * D), 1)
  wq, wk = O.norm_weight(H * D, 3), O.norm_weight(H * D, 4)
  cos, sin = O.wan_rope_table(w.grid, D)
  qo, ko = ops.norm_rope_fullrow(to_dev_bf16(q, dev), to_dev_bf16(k, dev), to_dev_bf16(wq, dev), to_dev_bf16(wk, dev),
                                 _t(cos, dev), _t(sin, dev), H, out_layout=layout)
  _assert_close(to_np(qo), O.norm_rope_fullrow(q, wq, cos, sin, H), "wan1.3b q")
  _assert_close(to_np(ko), O.norm_rope_fullrow(k, wk, cos, sin, H), "wan1.3b k")
  # against the reference's own rounding sequence (norm->bf16, bf16 table, bf16 products): two to four
  # extra roundings, so only a loose bound holds
  flow = O.norm_rope_wan_reference_flow(q, wq, cos, sin, H)
  mx, mean = err_stats(to_np(qo), flow)
  print(f"vs reference rounding flow: max-abs {mx:.3e} mean-abs {mean:.3e}")
  assert mx <= 8e-2 and mean <= 4e-3


def test_flux_dev_full_size(dev):
  w = O.WORKLOADS["flux-dev"]
  n_txt, rows, cols = w.grid
  ids = O.flux_ids(n_txt, rows, cols)
  L = ids.shape[0]
  assert L == w.seq
  q, k = O.normal_bf16((1, L, w.heads, 128), 0), O.normal_bf16((1, L, w.heads, 128), 1)
  wq, wk = O.norm_weight(128, 3), O.norm_weight(128, 4)
  for table_dtype in ("f32", "bf16"):  # bf16: the table precision a bf16 Flux model builds (transformer_flux_flax.py:434)
    cos, sin = O.flux_rope_table(ids, table_dtype=table_dtype)
    qo, ko = ops.norm_rope_perhead(to_dev_bf16(q, dev), to_dev_bf16(k, dev), to_dev_bf16(wq, dev), to_dev_bf16(wk, dev),
                                   _t(cos, dev), _t(sin, dev), out_layout="bhsd")
    _assert_close(to_np(qo), O.norm_rope_perhead(q, wq, cos, sin), f"flux q table {table_dtype}")
    _assert_close(to_np(ko), O.norm_rope_perhead(k, wk, cos, sin), f"flux k table {table_dtype}")


def test_wan14b_full_size_sampled_rows_and_invariants(dev):
  w = O.WORKLOADS["wan14b"]
  H, D, S = w.heads, w.head_dim, w.seq
  gen = torch.Generator(device=dev).manual_seed(0)
  q = torch.randn((1, S, H * D), generator=gen, device=dev, dtype=torch.float32).to(torch.bfloat16)
  k = torch.randn((1, S, H * D), generator=gen, device=dev, dtype=torch.float32).to(torch.bfloat16)
  wq, wk = O.norm_weight(H * D, 3), O.norm_weight(H * D, 4)
  cos, sin = O.wan_rope_table(w.grid, D)
  wq_d, wk_d = to_dev_bf16(wq, dev), to_dev_bf16(wk, dev)
  qo, ko = ops.norm_rope_fullrow(q, k, wq_d, wk_d, _t(cos, dev), _t(sin, dev), H)
  rows = O.sample_rows(S)
  idx = torch.from_numpy(rows).to(dev)
  for x, xo, wt, name in ((q, qo, wq, "q"), (k, ko, wk, "k")):
    ref = O.norm_rope_fullrow(to_np(x[:, idx]), wt, cos[rows], sin[rows], H)
    _assert_close(to_np(xo[:, idx]), ref, f"wan14b {name} sampled rows")
  # size-independent properties over ALL 75 600 rows (torch is the harness here, not the product):
  # (1) de-weighted rows have unit RMS; (2) the rotation keeps every pair's norm, so rope and norm-only agree on them
  qn, _ = ops.norm_rope_fullrow(q, None, wq_d, None, None, None, H)
  y = qn.float().view(1, S, H * D) / wq_d.float()
  rms = y.pow(2).mean(-1).sqrt()
  assert float((rms - 1).abs().max()) < 5e-3
  pn_rope = qo.float().view(1, S, H, D // 2, 2).pow(2).sum(-1)
  pn_norm = qn.float().view(1, S, H, D // 2, 2).pow(2).sum(-1)
  assert float((pn_rope - pn_norm).abs().max()) < 0.5 and float((pn_rope - pn_norm).abs().mean()) < 1e-2


def test_strided_input_batch_inplace_and_edges(dev):
  H, D, S, B = 6, 128, 37, 2
  N = H * D
  cos, sin = O.wan_rope_table((1, 1, S), D)
  wq, wk = O.norm_weight(N, 3), O.norm_weight(N, 4)
  # q and k as slices of one fused [B,S,3*N] projection output: token stride 3N, no copy
  qkv = O.normal_bf16((B, S, 3 * N), 0)
  t = to_dev_bf16(qkv, dev)
  qo, ko = ops.norm_rope_fullrow(t[:, :, :N], t[:, :, N:2 * N], to_dev_bf16(wq, dev), to_dev_bf16(wk, dev), _t(cos, dev), _t(sin, dev), H)
  _assert_close(to_np(qo), O.norm_rope_fullrow(qkv[:, :, :N], wq, cos, sin, H), "strided q")
  _assert_close(to_np(ko), O.norm_rope_fullrow(qkv[:, :, N:2 * N], wk, cos, sin, H), "strided k")
  # per-head kernel on the same fused buffer, viewed [B,S,H,D] with token stride 3N
  w1, w2 = O.norm_weight(D, 5), O.norm_weight(D, 6)
  q4 = t[:, :, :N].unflatten(2, (H, D))
  k4 = t[:, :, N:2 * N].unflatten(2, (H, D))
  qo, ko = ops.norm_rope_perhead(q4, k4, to_dev_bf16(w1, dev), to_dev_bf16(w2, dev), _t(cos, dev), _t(sin, dev))
  _assert_close(to_np(qo), O.norm_rope_perhead(qkv[:, :, :N].reshape(B, S, H, D), w1, cos, sin), "strided perhead q")
  _assert_close(to_np(ko), O.norm_rope_perhead(qkv[:, :, N:2 * N].reshape(B, S, H, D), w2, cos, sin), "strided perhead k")
  # a single token
  one = O.normal_bf16((1, 1, N), 9)
  qo, _ = ops.norm_rope_fullrow(to_dev_bf16(one, dev), None, to_dev_bf16(wq, dev), None, _t(cos[:1], dev), _t(sin[:1], dev), H)
  _assert_close(to_np(qo), O.norm_rope_fullrow(one, wq, cos[:1], sin[:1], H), "single token")
  # head dims 64 and 256 of the per-head kernel
  for d in (64, 256):
    x = O.normal_bf16((1, 19, 3, d), 11)
    wd = O.norm_weight(d, 12)
    ang = np.random.default_rng(13).uniform(-3, 3, (19, d // 2))
    c, s = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    xo, _ = ops.norm_rope_perhead(to_dev_bf16(x, dev), None, to_dev_bf16(wd, dev), None, _t(c, dev), _t(s, dev))
    _assert_close(to_np(xo), O.norm_rope_perhead(x, wd, c, s), f"perhead D={d}")


def test_host_side_validation_raises(dev):
  q = torch.zeros((1, 8, 512), dtype=torch.bfloat16, device=dev)
  w = torch.ones(512, dtype=torch.bfloat16, device=dev)
  with pytest.raises(ValueError, match="not divisible"):
    ops.norm_rope_fullrow(q, None, w, None, None, None, heads=3)
  with pytest.raises(ValueError, match=r"\[S, D/2\]"):
    ops.norm_rope_fullrow(q, None, w, None, torch.zeros(8, 60, device=dev), torch.zeros(8, 60, device=dev), heads=4)
  with pytest.raises(ValueError, match="no CPU path"):
    ops.norm_rope_fullrow(q.cpu(), None, w.cpu(), None, None, None, heads=4)


def test_q_mul_scales_the_query_only(dev):
  """q_mul is folded into the query before its single rounding; the key is untouched."""
  g = golden("norm_rope_wan.npz")
  H = int(g["heads"])
  q, k = bits_to_dev(g["q"], dev), bits_to_dev(g["k"], dev)
  wq, wk = bits_to_dev(g["wq"], dev), bits_to_dev(g["wk"], dev)
  cos, sin = _t(g["cos"], dev), _t(g["sin"], dev)
  m = ops.folded_q_mul(128)
  qo, ko = ops.norm_rope_fullrow(q, k, wq, wk, cos, sin, H, q_mul=m)
  _assert_close(to_np(qo) / m, g["q_out"], "wan golden q with q_mul")
  _assert_close(to_np(ko), g["k_out"], "wan golden k with q_mul")
  f = golden("norm_rope_flux.npz")
  q, k = bits_to_dev(f["q"], dev), bits_to_dev(f["k"], dev)
  w = [bits_to_dev(f[n], dev) for n in ("wq", "wk", "wq_txt", "wk_txt")]
  qo, ko = ops.norm_rope_perhead(q, k, w[0], w[1], _t(f["cos"], dev), _t(f["sin"], dev), wq_txt=w[2], wk_txt=w[3], n_txt=int(f["n_txt"]), q_mul=m)
  _assert_close(to_np(qo) / m, f["q_out"], "flux golden q with q_mul")
  _assert_close(to_np(ko), f["k_out"], "flux golden k with q_mul")


@pytest.mark.parametrize("heads,hidden", [(4, 512), (12, 1536), (40, 5120)])
def test_fused_qkv_projection_prologue(dev, heads, hidden):
  """mdattn_norm_rope_qkv: one launch over the output of a fused q|k|v projection [B,S,3*H*D] -- bias adds of the three
  Linear layers (attention_flax.py:2471-2510), norm_q / norm_k, the head split and the rotation -- against the oracle;
  without a bias it equals the two-tensor entry point bit for bit and leaves v in the fused buffer; in place, the
  fused buffer itself becomes the attention operands and attention on those strided views equals attention on dense
  copies bit for bit."""
  B, grid, D = 2, (3, 6, 7), 128
  S, N = grid[0] * grid[1] * grid[2], heads * 128
  assert N == hidden
  qkv = O.normal_bf16((B, S, 3 * N), 0)
  bias = O.bf16_round(0.5 * O.normal_bf16((3 * N,), 5))
  wq, wk = O.norm_weight(N, 3), O.norm_weight(N, 4)
  cos, sin = O.wan_rope_table(grid, D)
  dq, db, dwq, dwk = (to_dev_bf16(x, dev) for x in (qkv, bias, wq, wk))
  dcos, dsin = _t(cos, dev), _t(sin, dev)
  # (a) no bias: the same arithmetic as the two-tensor entry point on the q and k column blocks; v is the buffer's own block
  q0, k0, v0 = ops.norm_rope_qkv(dq, dwq, dwk, dcos, dsin, heads)
  wq_, wk_ = ops.norm_rope_fullrow(dq[:, :, :N], dq[:, :, N:2 * N], dwq, dwk, dcos, dsin, heads)
  assert torch.equal(q0, wq_) and torch.equal(k0, wk_)
  assert v0.data_ptr() == dq.data_ptr() + 2 * N * 2 and torch.equal(v0.reshape(B, S, N), dq[:, :, 2 * N:])
  # (b) with the projection biases, against the oracle
  for layout in ("bshd", "bhsd"):
    q1, k1, v1 = ops.norm_rope_qkv(dq, dwq, dwk, dcos, dsin, heads, bias=db, out_layout=layout, q_mul=1.0)
    rq, rk, rv = O.norm_rope_qkv(qkv, wq, wk, cos, sin, heads, bias=bias)
    _assert_close(to_np(q1), rq, f"fused qkv q {layout} H={heads}")
    _assert_close(to_np(k1), rk, f"fused qkv k {layout} H={heads}")
    _assert_close(to_np(v1), rv, f"fused qkv v {layout} H={heads}")
    assert not torch.equal(q1, q0.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3) if layout == "bhsd" else q0)  # the bias matters
  # (c) in place: the fused buffer becomes q | k | v, element for element what (b) returned in [B,S,H,D]
  q1, k1, v1 = ops.norm_rope_qkv(dq, dwq, dwk, dcos, dsin, heads, bias=db)
  buf = dq.clone()
  q2, k2, v2 = ops.norm_rope_qkv(buf, dwq, dwk, dcos, dsin, heads, bias=db, inplace=True)
  assert q2.data_ptr() == buf.data_ptr() and v2.data_ptr() == buf.data_ptr() + 2 * N * 2
  assert torch.equal(q2, q1) and torch.equal(k2, k1) and torch.equal(v2, v1)
  # (d) attention straight on the strided views of the fused buffer (row stride 3*H*D) == attention on dense copies
  out_f, lse_f = ops.flash_attention(q2, k2, v2, return_lse=True)
  out_d, lse_d = ops.flash_attention(q1, k1, v1, return_lse=True)
  assert torch.equal(out_f, out_d) and torch.equal(lse_f, lse_d)
  assert out_f.is_contiguous() and out_f.reshape(B, S, N).shape == (B, S, N)  # the [B,S,H*D] rows proj_attn consumes


def test_fused_qkv_rejects_a_bias_without_a_value_output(dev, lib):
  import ctypes
  from maxdiffusion_amd import _lib

  P, fake = ctypes.c_void_p, ctypes.c_void_p(0x1000)
  st = ctypes.byref(_lib.Strides(8 * 1536, 1536, 128))
  args = lambda bias, v_out, stride: (None, fake, bias, fake, fake, v_out, fake, fake, None, None, 1, 8, 4, 128, 1e-6, 1.0, 0, stride, st)
  assert lib.mdattn_norm_rope_qkv(*args(fake, None, 1536)) == _lib.E_BADARG      # bias but nowhere to put v + bias
  assert lib.mdattn_norm_rope_qkv(*args(None, None, 1024)) == _lib.E_BADARG      # row stride below 3*H*D
  assert lib.mdattn_norm_rope_qkv(*args(P(0x1004), fake, 1536)) == _lib.E_ALIGN
