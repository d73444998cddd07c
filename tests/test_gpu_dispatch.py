"""`hip_flash` behind the reference-shaped dispatcher: rank-3 and rank-4 inputs, cross-attention,
compared with a restated `dot_product` registered by the test (the reference's own integration
test compares flash against dot_product the same way, tests/attention_test.py:90-147)."""
from unittest import mock

import numpy as np
import pytest
import torch

import oracle as O
from helpers import err_stats, rel_l2, to_dev_bf16, to_np
from maxdiffusion_amd import attention_op as A

pytestmark = pytest.mark.gpu


def _dot_product_oracle(q, k, v, context):
  """Test-only registry entry: the bf16 dtype flow of _apply_attention_dot on the CPU."""
  h = context["heads"]
  to_hsd = lambda t: np.ascontiguousarray(to_np(A._as_bshd(t, h))[0].transpose(1, 0, 2))
  out = O.attention_dot_product_bf16(to_hsd(q), to_hsd(k), to_hsd(v), context["scale"])
  return torch.from_numpy(out.transpose(1, 0, 2).reshape(1, out.shape[1], -1)).to(q.device).to(q.dtype)


def _op(kernel, heads):
  return A.AttentionOp(mesh=None, attention_kernel=kernel, scale=128**-0.5, heads=heads, dim_head=128, dtype=torch.bfloat16,
                       float32_qk_product=False, split_head_dim=False)


def test_hip_flash_matches_dot_product_rank3_rank4_and_cross(dev):
  H, S, T = 10, 1024, 77
  q, k, v = (O.normal_bf16((1, S, H * 128), s) for s in (0, 1, 2))
  kt, vt = O.normal_bf16((1, T, H * 128), 5), O.normal_bf16((1, T, H * 128), 6)
  qd, kd, vd, ktd, vtd = (to_dev_bf16(x, dev) for x in (q, k, v, kt, vt))
  with mock.patch.dict(A.KERNEL_REGISTRY, {"dot_product": _dot_product_oracle}):
    for name, args in (("self rank-3", (qd, kd, vd)), ("cross rank-3", (qd, ktd, vtd))):
      got = _op("hip_flash", H).apply_attention(*args)
      want = _op("dot_product", H).apply_attention(*args)
      assert got.shape == (1, S, H * 128) and got.dtype == torch.bfloat16
      mx, mean = err_stats(to_np(got), to_np(want))
      print(f"{name}: max-abs {mx:.3e} mean-abs {mean:.3e}")
      assert mx <= 2e-2 and mean <= 2e-3 and rel_l2(to_np(got), to_np(want)) <= 3e-2
      if name.startswith("self"):  # the reference's own criterion for self-attention (attention_test.py:147)
        diff_norm = float((got.float() - want.float()).norm())
        assert diff_norm < 1.0, diff_norm
    # rank-4 [B,H,S,D] inputs, the layout Wan self-attention hands over after rope (attention_flax.py:2673-2684)
    to4 = lambda t: t.view(1, -1, H, 128).permute(0, 2, 1, 3).contiguous()
    got4 = _op("hip_flash", H).apply_attention(to4(qd), to4(kd), to4(vd))
    got3 = _op("hip_flash", H).apply_attention(qd, kd, vd)
    assert got4.shape == (1, S, H * 128) and torch.equal(got4, got3)


def test_f32_inputs_are_accepted_and_returned_in_f32(dev):
  # LTX2 passes f32 q/k (attention_ltx2.py:415-432); the result must come back in q's dtype
  H, S = 2, 128
  q, k, v = (to_dev_bf16(O.normal_bf16((1, S, H * 128), s), dev).float() for s in (0, 1, 2))
  got = _op("hip_flash", H).apply_attention(q, k, v)
  assert got.dtype == torch.float32
  want = _op("hip_flash", H).apply_attention(q.bfloat16(), k.bfloat16(), v.bfloat16())
  assert torch.equal(got, want.float())


def test_fused_prologue_feeds_attention_without_transposes(dev):
  # Wan block order: norm_q/norm_k over H*D -> rope -> attention (attention_flax.py:2655-2684), then the
  # cross-attention with norm only (:2671); compared with the un-fused oracle chain.
  w = O.WORKLOADS["wan1.3b"]
  H, S = w.heads, 3 * 10 * 13
  cos, sin = O.wan_rope_table((3, 10, 13), 128)
  q, k, v = (O.normal_bf16((1, S, H * 128), s) for s in (0, 1, 2))
  wq, wk = O.norm_weight(H * 128, 3), O.norm_weight(H * 128, 4)
  table = torch.from_numpy(O.wan_rope_table_complex((3, 10, 13), 128)).to(dev)  # complex64 [1,1,S,64], as the model passes it
  qn, kn = A.hip_norm_rope(to_dev_bf16(q, dev), to_dev_bf16(k, dev), to_dev_bf16(wq, dev), to_dev_bf16(wk, dev), table, H, out_layout="bhsd")
  out = _op("hip_flash", H).apply_attention(qn.permute(0, 2, 1, 3), kn.permute(0, 2, 1, 3), to_dev_bf16(v, dev).view(1, S, H, 128).permute(0, 2, 1, 3))
  qe, ke = O.norm_rope_fullrow(q, wq, cos, sin, H), O.norm_rope_fullrow(k, wk, cos, sin, H)
  ro, _ = O.attention(qe[0].transpose(1, 0, 2), ke[0].transpose(1, 0, 2), v.reshape(S, H, 128).transpose(1, 0, 2), w.scale)
  got = to_np(out).reshape(S, H, 128).transpose(1, 0, 2)
  mx, mean = err_stats(got, ro)
  assert mx <= 2e-2 and mean <= 2e-3 and rel_l2(got, ro) <= 1.5e-2
  qc, none = A.hip_norm_rope(to_dev_bf16(q, dev), None, to_dev_bf16(wq, dev), None, None, H)  # cross-attention: norm only
  assert none is None
  assert err_stats(to_np(qc), O.norm_rope_fullrow(q, wq, None, None, H))[0] <= 1.6e-2


def test_reference_splash_test_shape_head_dim_64(dev):
  """tests/attention_test.py:90-147 of the reference: B=8, S=4096, H=10, D=64, N(0,1) inputs, criterion
  ||dot_product - flash||_2 < 1.0 over the whole tensor.  Here: hip_flash through the registry against an f32
  attention computed by torch on the GPU (test harness only), and the same criterion."""
  from helpers import torch_attention_f32
  B, S, H, D = 8, 4096, 10, 64
  gen = torch.Generator(device=dev).manual_seed(7)
  q, k, v = (torch.randn((B, S, H * D), generator=gen, device=dev, dtype=torch.float32).to(torch.bfloat16) for _ in range(3))
  op = A.AttentionOp(mesh=None, attention_kernel="hip_flash", scale=D**-0.5, heads=H, dim_head=D, dtype=torch.bfloat16)
  got = op.apply_attention(q, k, v)
  assert got.shape == (B, S, H * D) and got.dtype == torch.bfloat16
  ref, _ = torch_attention_f32(q.view(B, S, H, D), k.view(B, S, H, D), v.view(B, S, H, D), D**-0.5)
  diff = got.float().view(B, S, H, D) - ref
  diff_norm, mx = float(diff.norm()), float(diff.abs().max())
  print(f"B=8 S=4096 H=10 D=64: ||hip_flash - f32 attention||_2 = {diff_norm:.3f}, max-abs {mx:.2e}", flush=True)
  assert diff_norm < 1.0 and mx <= 2e-2
  assert float(diff.norm() / ref.norm()) <= 1.5e-2


def test_wan_i2v_cross_attention_block(dev):
  """The Wan image-to-video cross-attention (attention_flax.py:2690-2777): the same tokens attend to the text states
  (normed q, no mask) and to the image embeddings (raw q; 257 real image tokens padded to 384, the padding excluded by
  encoder_attention_mask_img), and the two results are added.  Prologue hooks in norm-only mode, `hip_flash` twice,
  against the f32 oracle with the padded keys removed."""
  B, H, D, S, T, real, padded = 2, 4, 128, 300, 512, 257, 384
  N = H * D
  scale = D**-0.5
  xq, xkt, xvt = O.normal_bf16((B, S, N), 0), O.normal_bf16((B, T, N), 1), O.normal_bf16((B, T, N), 2)
  xki, xvi = O.normal_bf16((B, padded, N), 3), O.normal_bf16((B, padded, N), 4)
  wq, wk, wki = O.norm_weight(N, 5), O.norm_weight(N, 6), O.norm_weight(N, 7)
  q, kt, vt, ki, vi, tq, tk, tki = (to_dev_bf16(x, dev) for x in (xq, xkt, xvt, xki, xvi, wq, wk, wki))
  keep = torch.zeros((B, padded), dtype=torch.bool, device=dev)
  keep[:, :real] = True

  op = A.AttentionOp(mesh=None, attention_kernel="hip_flash", scale=scale, heads=H, dim_head=D, dtype=torch.bfloat16)
  q_text, _ = A.hip_norm_rope(q, None, tq, None, None, H)        # norm_q on the queries (norm only: no rotary table)
  k_text, _ = A.hip_norm_rope(kt, None, tk, None, None, H)       # norm_k on the text keys
  k_img, _ = A.hip_norm_rope(ki, None, tki, None, None, H)       # norm_added_k on the image keys
  out_text = op.apply_attention(q_text.reshape(B, S, N), k_text.reshape(B, T, N), vt)
  out_img = op.apply_attention(q, k_img.reshape(B, padded, N), vi, attention_mask=keep)
  got = to_np(out_text + out_img)

  for b in range(B):
    hsd = lambda x: np.ascontiguousarray(x.reshape(x.shape[0], H, D).transpose(1, 0, 2))
    qn = O.bf16_round(O.rmsnorm(xq[b], wq))
    o_t, _ = O.attention(hsd(qn), hsd(O.bf16_round(O.rmsnorm(xkt[b], wk))), hsd(xvt[b]), scale)
    o_i, _ = O.attention(hsd(xq[b]), hsd(O.bf16_round(O.rmsnorm(xki[b, :real], wki))), hsd(xvi[b, :real]), scale)
    want = (O.bf16_round(o_t) + O.bf16_round(o_i)).transpose(1, 0, 2).reshape(S, N)
    mx, mean = err_stats(got[b], want)
    print(f"i2v cross-attention, batch {b}: max-abs {mx:.3e} mean-abs {mean:.3e} rel-l2 {rel_l2(got[b], want):.3e}")
    assert mx <= 4e-2 and mean <= 4e-3 and rel_l2(got[b], want) <= 2e-2  # the sum of two bf16 outputs: twice the single-call bars


@pytest.mark.parametrize("D", [40, 80, 96, 8])
def test_head_dims_below_128_are_zero_padded(dev, D):
  """The reference's flash wrappers pad head dims below 128 with zeros (attention_flax.py:223-259), so its registry
  takes SD-1.x style heads of 40 / 80 as well; `hip_flash` pads to the next size its kernels take (64 or 128) and cuts
  the output back.  Forward against the oracle at the true head dim (rank 3, rank 4, with a key mask), gradients
  against torch autograd through an f32 attention on the same inputs."""
  H, S, T = 3, 200, 77
  q, k, v = O.normal_bf16((1, S, H * D), 0), O.normal_bf16((1, T, H * D), 1), O.normal_bf16((1, T, H * D), 2)
  hsd = lambda x, n: np.ascontiguousarray(x.reshape(n, H, D).transpose(1, 0, 2))
  op = A.AttentionOp(mesh=None, attention_kernel="hip_flash", scale=D**-0.5, heads=H, dim_head=D, dtype=torch.bfloat16)
  qd, kd, vd = (to_dev_bf16(x, dev) for x in (q, k, v))
  got = op.apply_attention(qd, kd, vd)
  assert got.shape == (1, S, H * D) and got.dtype == torch.bfloat16
  ro, _ = O.attention(hsd(q, S), hsd(k, T), hsd(v, T), D**-0.5)
  mx, mean = err_stats(hsd(to_np(got), S), ro)
  assert mx <= 2e-2 and mean <= 2e-3, (D, mx, mean)
  to4 = lambda t, n: t.view(1, n, H, D).permute(0, 2, 1, 3).contiguous()
  assert torch.equal(op.apply_attention(to4(qd, S), to4(kd, T), to4(vd, T)), got)
  keep = np.random.default_rng(7).random((1, T)) < 0.6
  gm = op.apply_attention(qd, kd, vd, attention_mask=torch.from_numpy(keep).to(dev))
  rm, _ = O.attention(hsd(q, S), hsd(k, T), hsd(v, T), D**-0.5, kv_mask=keep[0])
  mx, mean = err_stats(hsd(to_np(gm), S), rm)
  assert mx <= 2e-2 and mean <= 2e-3, ("masked", D, mx, mean)
  # gradients flow through the pad and the slice
  ql, kl, vl = (t.clone().requires_grad_(True) for t in (qd, kd, vd))
  g = to_dev_bf16(O.normal_bf16((1, S, H * D), 9), dev)
  op.apply_attention(ql, kl, vl).backward(g)
  qf, kf, vf = (t.float().view(1, -1, H, D).permute(0, 2, 1, 3).detach().requires_grad_(True) for t in (qd, kd, vd))
  ref = torch.softmax(qf @ kf.transpose(-1, -2) * D**-0.5, dim=-1) @ vf
  ref.backward(g.float().view(1, S, H, D).permute(0, 2, 1, 3))
  for name, a, b in (("dq", ql.grad, qf.grad), ("dk", kl.grad, kf.grad), ("dv", vl.grad, vf.grad)):
    assert a.shape == (1, a.shape[1], H * D)
    want = b.permute(0, 2, 1, 3).reshape(a.shape)
    err = float((a.float() - want).abs().max())
    scale = float(want.abs().max())
    assert err <= 2e-2 * max(1.0, scale), (D, name, err, scale)


def test_fp8_registry_entry_pads_head_dims_too(dev):
  H, S, D = 2, 300, 80
  q, k, v = (to_dev_bf16(O.normal_bf16((1, S, H * D), s), dev) for s in (0, 1, 2))
  mk = lambda name: A.AttentionOp(mesh=None, attention_kernel=name, scale=D**-0.5, heads=H, dim_head=D, dtype=torch.bfloat16)
  got, want = mk("hip_flash_fp8").apply_attention(q, k, v), mk("hip_flash").apply_attention(q, k, v)
  assert got.shape == want.shape == (1, S, H * D)
  a, b = got.float().flatten(), want.float().flatten()
  assert float(torch.dot(a, b) / (a.norm() * b.norm())) >= 0.995


def test_registry_folds_the_scale_into_q_on_long_key_sequences(dev):
  """From FOLD_SCALE_MIN_KEYS keys on (no mask, no autograd) `hip_flash` multiplies q by scale * log2(e) itself and
  calls the kernels with scale = ln 2; below, and for a caller that already carries the factor, the scale goes through
  unchanged.  Either way the result meets the bars against the oracle."""
  from maxdiffusion_amd import ops

  H, S, D = 2, 300, 128
  for skv, scale, want in ((A.FOLD_SCALE_MIN_KEYS + 77, D**-0.5, ops.FOLDED_SCALE), (A.FOLD_SCALE_MIN_KEYS - 1, D**-0.5, D**-0.5),
                           (A.FOLD_SCALE_MIN_KEYS, ops.FOLDED_SCALE, ops.FOLDED_SCALE)):
    q, k, v = O.normal_bf16((1, S, H * D), 0), O.normal_bf16((1, skv, H * D), 1), O.normal_bf16((1, skv, H * D), 2)
    if scale == ops.FOLDED_SCALE:  # what the fused prologue hands over with q_mul
      q = O.bf16_round(q * np.float32(ops.folded_q_mul(D)))
    op = A.AttentionOp(mesh=None, attention_kernel="hip_flash", scale=scale, heads=H, dim_head=D, dtype=torch.bfloat16)
    with mock.patch.object(A.ops, "flash_attention", wraps=ops.flash_attention) as spy:
      got = op.apply_attention(to_dev_bf16(q, dev), to_dev_bf16(k, dev), to_dev_bf16(v, dev))
    assert spy.call_args.kwargs["scale"] == want, (skv, scale, spy.call_args.kwargs["scale"])
    hsd = lambda x, n: np.ascontiguousarray(x.reshape(n, H, D).transpose(1, 0, 2))
    ro, _ = O.attention(hsd(q, S), hsd(k, skv), hsd(v, skv), scale)
    mx, mean = err_stats(hsd(to_np(got), S), ro)
    print(f"Skv={skv} scale={scale:.4f}: max-abs {mx:.3e} mean-abs {mean:.3e}")
    assert mx <= 2e-2 and mean <= 2e-3 and rel_l2(hsd(to_np(got), S), ro) <= 1.5e-2, (skv, mx, mean)
