"""Pins the CPU oracle: library routines, closed forms, invariants, brute force, and the
fixtures the reference's own tests hold for this path.  No formula of the oracle is re-typed
here as its own check."""
import math

import numpy as np
import pytest
import scipy.special
import torch

import oracle as O


# ----------------------------------------------------------------------------- dtype helpers
def test_bf16_round_matches_torch():
  rng = np.random.default_rng(0)
  x = np.concatenate([
      rng.standard_normal(100000).astype(np.float32) * 3,
      np.array([0.0, -0.0, 1.0, 1.00390625, 1.0078125, 1.01171875, 3.3895314e38, 1e-40, -1e-40, 65504.0], np.float32),
      (rng.standard_normal(1000) * 1e-30).astype(np.float32),
  ])
  want = torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy()
  np.testing.assert_array_equal(O.bf16_round(x), want)
  bits = O.to_bf16_bits(x)
  np.testing.assert_array_equal(bits.view(np.int16), torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy())
  np.testing.assert_array_equal(O.from_bf16_bits(bits), want)


def test_e4m3_round_matches_torch():
  rng = np.random.default_rng(1)
  x = np.concatenate([
      rng.uniform(-448, 448, 50000).astype(np.float32),
      rng.standard_normal(50000).astype(np.float32),
      (rng.standard_normal(20000) * 0.01).astype(np.float32),
      np.array([0, 448, -448, 2**-9, 2**-10, 1.5 * 2**-9, 0.0009765625, 17.0, 18.0, 19.0, 416.0, 432.0, 447.9], np.float32),
  ])
  want = torch.from_numpy(x).to(torch.float8_e4m3fn).to(torch.float32).numpy()
  np.testing.assert_array_equal(O.e4m3_round(x), want)
  assert O.e4m3_round(np.array([1000.0, -1e9], np.float32)).tolist() == [448.0, -448.0]  # saturating


# ----------------------------------------------------------------------------- RMSNorm
def test_rmsnorm_matches_torch_library():
  rng = np.random.default_rng(2)
  x = rng.standard_normal((3, 17, 1536)).astype(np.float32)
  w = (1 + 0.1 * rng.standard_normal(1536)).astype(np.float32)
  want = torch.nn.functional.rms_norm(torch.from_numpy(x), (1536,), torch.from_numpy(w), eps=1e-6).numpy()
  np.testing.assert_allclose(O.rmsnorm(x, w, 1e-6), want, rtol=2e-6, atol=2e-6)
  xh = x.reshape(3, 17, 12, 128)
  wh = w[:128]
  want = torch.nn.functional.rms_norm(torch.from_numpy(xh), (128,), torch.from_numpy(wh), eps=1e-6).numpy()
  np.testing.assert_allclose(O.rmsnorm(xh, wh, 1e-6), want, rtol=2e-6, atol=2e-6)


def test_rmsnorm_closed_forms():
  c, n, eps = 3.0, 64, 1e-6
  w = np.linspace(0.5, 1.5, n)
  got = O.rmsnorm(np.full((2, n), c), w, eps)
  np.testing.assert_allclose(got, np.broadcast_to(c / math.sqrt(c * c + eps) * w, (2, n)), rtol=1e-14)
  rng = np.random.default_rng(3)
  x = rng.standard_normal((5, n))
  y = O.rmsnorm(x, np.ones(n), 0.0)
  np.testing.assert_allclose(np.sqrt((y * y).mean(-1)), 1.0, rtol=1e-13)  # unit RMS
  np.testing.assert_allclose(O.rmsnorm(1000.0 * x, w, eps), O.rmsnorm(x, w, eps), rtol=1e-5)  # scale equivariance
  np.testing.assert_array_equal(O.rmsnorm(np.zeros((1, n)), w, eps), np.zeros((1, n)))


# ----------------------------------------------------------------------------- Wan rotary table
def test_wan_table_shape_fixture_and_split():
  # tests/wan/wan_transformer_test.py:68-78: latent 21x45x80 (patch 1,2,2 already applied) -> (1,1,75600,64)
  t = O.wan_rope_table_complex((21, 45, 80), 128)
  assert t.shape == (1, 1, 75600, 64) and t.dtype == np.complex64
  # tests/wan/wan_transformer_test.py:51-54: split sizes 22 / 21 / 21
  ang = O.wan_rope_angles((21, 45, 80), 128).reshape(21, 45, 80, 64)
  assert np.all(ang[:, :, :, :22] == ang[:, :1, :1, :22])  # frame pairs ignore row/col
  assert np.all(ang[:, :, :, 22:43] == ang[:1, :, :1, 22:43])  # row pairs
  assert np.all(ang[:, :, :, 43:] == ang[:1, :1, :, 43:])  # col pairs
  assert np.all(ang[1, 0, 0, :22] > 0) and np.all(ang[1, 0, 0, 22:] == 0)
  assert np.all(ang[0, 1, 0, 22:43] > 0) and np.all(ang[0, 0, 1, 43:] > 0)
  np.testing.assert_array_equal(t[0, 0, 0], np.ones(64, np.complex64))  # position (0,0,0)
  np.testing.assert_allclose(np.abs(t), 1.0, atol=1e-6)  # unit modulus


def test_wan_table_brute_force_small_grid():
  # the grid/head_dim of the HF parity test (tests/wan/wan_common_module_parity_test.py:202-213)
  F, H, W, D, theta = 3, 4, 4, 12, 10000.0
  hd = wd = 2 * (D // 6)
  td = D - hd - wd
  cos, sin = O.wan_rope_table((F, H, W), D, theta)
  assert cos.shape == (F * H * W, D // 2)
  n = 0
  for f in range(F):
    for h in range(H):
      for w in range(W):
        exp = []
        for pos, dim in ((f, td), (h, hd), (w, wd)):
          for i in range(dim // 2):
            exp.append(pos / theta ** (2.0 * i / dim))
        np.testing.assert_allclose(cos[n], np.cos(exp), atol=2e-6)
        np.testing.assert_allclose(sin[n], np.sin(exp), atol=2e-6)
        n += 1


# ----------------------------------------------------------------------------- Flux rotary table
def test_flux_table_text_identity_and_split():
  ids = O.flux_ids(5, 4, 6)
  assert ids.shape == (5 + 24, 3)
  np.testing.assert_array_equal(ids[5 + 6 + 2], [0, 1, 2])  # row-major (0,row,col)
  cos, sin = O.flux_rope_table(ids)
  assert cos.shape == (29, 64)
  np.testing.assert_array_equal(cos[:5], 1.0)  # text ids are zero: identity rotation
  np.testing.assert_array_equal(sin[:5], 0.0)
  np.testing.assert_array_equal(sin[:, :8], 0.0)  # axis 0 id is 0 for every token: 8 pairs
  ang = O.flux_rope_angles(ids)
  row = ang[5:].reshape(4, 6, 64)
  assert np.all(row[:, :, 8:36] == row[:, :1, 8:36]) and np.all(row[:, :, 36:] == row[:1, :, 36:])  # 28 / 28 pairs
  r, c = 3, 5
  np.testing.assert_allclose(row[r, c, 8 + 3], r / 10000.0 ** (6 / 56), rtol=1e-6)
  np.testing.assert_allclose(row[r, c, 36 + 27], c / 10000.0 ** (54 / 56), rtol=1e-6)


def test_flux_tuple_form_equals_matrix_form():
  ids = O.flux_ids(3, 5, 5)
  cos, sin = O.flux_rope_table(ids)
  table = O.flux_rope_table_matrix(ids)
  np.testing.assert_array_equal(table[..., 0, 1], -sin)  # packed [cos, -sin, sin, cos]
  rng = np.random.default_rng(4)
  x = rng.standard_normal((2, ids.shape[0], 64 * 2))  # [H, L, D]
  a = O.apply_rope_interleaved(x, cos, sin, seq_axis=-2)
  b = O.apply_rope_matrix_form(x, table.astype(np.float64))
  np.testing.assert_allclose(a, b, atol=1e-12)


# ----------------------------------------------------------------------------- RoPE application
def _rand_table(rng, s, half):
  ang = rng.uniform(-50, 50, (s, half))
  return ang, np.cos(ang), np.sin(ang)


def test_rope_is_complex_multiplication():
  rng = np.random.default_rng(5)
  ang, cos, sin = _rand_table(rng, 7, 8)
  x = rng.standard_normal((2, 7, 3, 16))
  z = (x[..., 0::2] + 1j * x[..., 1::2]) * np.exp(1j * ang)[None, :, None, :]
  want = np.stack([z.real, z.imag], -1).reshape(x.shape)
  np.testing.assert_allclose(O.apply_rope_interleaved(x, cos, sin), want, atol=1e-12)
  xt = x.transpose(0, 2, 1, 3)
  np.testing.assert_allclose(O.apply_rope_interleaved(xt, cos, sin, seq_axis=-2), want.transpose(0, 2, 1, 3), atol=1e-12)


def test_rope_group_properties():
  rng = np.random.default_rng(6)
  a, ca, sa = _rand_table(rng, 5, 4)
  b, cb, sb = _rand_table(rng, 5, 4)
  x = rng.standard_normal((1, 5, 2, 8))
  ab = O.apply_rope_interleaved(O.apply_rope_interleaved(x, ca, sa), cb, sb)
  np.testing.assert_allclose(ab, O.apply_rope_interleaved(x, np.cos(a + b), np.sin(a + b)), atol=1e-12)  # composition
  np.testing.assert_allclose(O.apply_rope_interleaved(O.apply_rope_interleaved(x, ca, sa), ca, -sa), x, atol=1e-12)  # inverse
  y = O.apply_rope_interleaved(x, ca, sa).reshape(1, 5, 2, 4, 2)
  np.testing.assert_allclose((y**2).sum(-1), (x.reshape(1, 5, 2, 4, 2) ** 2).sum(-1), rtol=1e-12)  # pair norms kept


def test_rope_relative_position_property():
  cos, sin = O.wan_rope_table((4, 5, 6), 128)
  rng = np.random.default_rng(7)
  q = rng.standard_normal(128)
  k = rng.standard_normal(128)
  S = 4 * 5 * 6
  qs = O.apply_rope_interleaved(np.broadcast_to(q, (1, S, 1, 128)), cos, sin)[0, :, 0]
  ks = O.apply_rope_interleaved(np.broadcast_to(k, (1, S, 1, 128)), cos, sin)[0, :, 0]
  idx = lambda f, h, w: (f * 5 + h) * 6 + w
  d1 = qs[idx(1, 2, 3)] @ ks[idx(0, 1, 1)]
  d2 = qs[idx(3, 4, 5)] @ ks[idx(2, 3, 3)]  # same offset (1,1,2)
  np.testing.assert_allclose(d1, d2, rtol=1e-5, atol=1e-5)


def test_norm_rope_fused_vs_reference_rounding_flow():
  # The fused f32 flow and the reference's bf16 flow agree to bf16 round-off.
  w = O.WORKLOADS["wan1.3b"]
  S = 3 * 4 * 4
  cos, sin = O.wan_rope_table((3, 4, 4), 128)
  x = O.normal_bf16((1, S, 12 * 128), 0)
  wq = O.norm_weight(12 * 128, 3)
  exact = O.norm_rope_fullrow(x, wq, cos, sin, 12)
  ref_flow = O.norm_rope_wan_reference_flow(x, wq, cos, sin, 12)
  d = np.abs(ref_flow - exact)
  assert d.max() <= 6e-2 and d.mean() <= 4e-3
  norm_only = O.norm_rope_fullrow(x, wq, None, None, 12)
  np.testing.assert_allclose(norm_only.reshape(1, S, -1), O.rmsnorm(x, wq), rtol=1e-14)
  assert w.scale == 128**-0.5


# ----------------------------------------------------------------------------- attention + LSE
def test_attention_lse_matches_scipy_and_out_matches_torch_sdpa():
  rng = np.random.default_rng(8)
  q = rng.standard_normal((3, 50, 128))
  k = rng.standard_normal((3, 77, 128))
  v = rng.standard_normal((3, 77, 128))
  scale = 128**-0.5
  out, lse = O.attention(q, k, v, scale)
  logits = np.einsum("hqd,hkd->hqk", q, k) * scale
  np.testing.assert_allclose(lse, scipy.special.logsumexp(logits, axis=-1), rtol=1e-12)
  want = torch.nn.functional.scaled_dot_product_attention(
      torch.from_numpy(q).float()[None], torch.from_numpy(k).float()[None], torch.from_numpy(v).float()[None], scale=scale)[0].numpy()
  np.testing.assert_allclose(out, want, atol=2e-5)
  o2, l2 = O.attention_rows(q[1, 5:9], k[1], v[1], scale)
  np.testing.assert_allclose(o2, out[1, 5:9], rtol=1e-9, atol=1e-14)
  np.testing.assert_allclose(l2, lse[1, 5:9], rtol=1e-12)


def test_attention_invariants():
  rng = np.random.default_rng(9)
  H, Sq, Skv, D = 2, 9, 33, 16
  q = rng.standard_normal((H, Sq, D))
  k = rng.standard_normal((H, Skv, D))
  v = rng.standard_normal((H, Skv, D))
  out, lse = O.attention(q, k, v, 0.25)
  o0, l0 = O.attention(q, np.zeros_like(k), v, 0.25)  # K = 0: uniform weights
  np.testing.assert_allclose(o0, np.broadcast_to(v.mean(1, keepdims=True), o0.shape), rtol=1e-12)
  np.testing.assert_allclose(l0, math.log(Skv), rtol=1e-12)
  oc, _ = O.attention(q, k, np.full_like(v, 2.5), 0.25)  # V = const
  np.testing.assert_allclose(oc, 2.5, rtol=1e-12)
  perm = rng.permutation(Skv)  # key order is irrelevant
  op, lp = O.attention(q, k[:, perm], v[:, perm], 0.25)
  np.testing.assert_allclose(op, out, rtol=1e-10)
  np.testing.assert_allclose(lp, lse, rtol=1e-12)
  # adding c*q-direction-independent constant to every logit (k + t with q.t const is not general);
  # use the exact shift: duplicate all keys -> out unchanged, lse + ln 2
  od, ld = O.attention(q, np.concatenate([k, k], 1), np.concatenate([v, v], 1), 0.25)
  np.testing.assert_allclose(od, out, rtol=1e-10)
  np.testing.assert_allclose(ld, lse + math.log(2.0), rtol=1e-12)


def test_attention_hand_fixtures_from_reference_tests():
  # tests/ltx2/test_attention_ltx2.py:38-76: zero q/k, two keys, per-example keep masks
  q = np.zeros((1, 1, 2))
  k = np.zeros((1, 2, 2))
  v = np.array([[[1.0, 0.0], [0.0, 1.0]]])
  for mask, want in (([True, False], [1.0, 0.0]), ([False, True], [0.0, 1.0])):
    out, _ = O.attention(q, k, v, 1.0, kv_mask=np.array(mask))
    np.testing.assert_allclose(out[0, 0], want, atol=1e-6)
  # tests/ltx2/test_attention_ltx2.py:91-116: all keys masked -> zeros
  out, lse = O.attention(q, k, np.ones((1, 2, 2)), 1.0, kv_mask=np.array([False, False]))
  np.testing.assert_array_equal(out, np.zeros((1, 1, 2)))
  assert np.isneginf(lse).all()
  out, _ = O.attention(q, k, v, 1.0)  # unmasked: mean of the two values
  np.testing.assert_allclose(out[0, 0], [0.5, 0.5])


def test_dot_product_bf16_flow_within_reference_tolerance():
  # tests/custom_splash_fixed_m_test.py:103-107 holds the 2e-2 max-abs bar on bf16 N(0,1) inputs
  q = O.normal_bf16((2, 256, 128), 0)
  k = O.normal_bf16((2, 300, 128), 1)
  v = O.normal_bf16((2, 300, 128), 2)
  exact, _ = O.attention(q, k, v, 128**-0.5)
  flow = O.attention_dot_product_bf16(q, k, v, 128**-0.5)
  assert np.abs(flow - exact).max() < 2e-2


# ----------------------------------------------------------------------------- merges
def test_merge_equals_attention_over_union():
  rng = np.random.default_rng(10)
  H, Sq, D = 2, 11, 32
  q = rng.standard_normal((H, Sq, D))
  for sizes in ([7], [5, 9], [1, 2, 3, 4, 5, 6, 7, 8], [64, 1, 31]):
    ks = [rng.standard_normal((H, n, D)) for n in sizes]
    vs = [rng.standard_normal((H, n, D)) for n in sizes]
    full_o, full_l = O.attention(q, np.concatenate(ks, 1), np.concatenate(vs, 1), 0.3)
    o, l = O.ring_replay(q, ks, vs, 0.3)
    np.testing.assert_allclose(o, full_o, rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(l, full_l, rtol=1e-12)
    parts = [O.attention(q, kc, vc, 0.3) for kc, vc in zip(ks, vs)]
    o2, l2 = O.merge_scan_ring([p[0] for p in parts], [p[1] for p in parts])  # attention_flax.py:736-772 form
    np.testing.assert_allclose(o2, full_o, rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(l2, full_l, rtol=1e-12)


def test_merge_algebra_and_mlo_form():
  rng = np.random.default_rng(11)
  sh = (3, 5)
  o = [rng.standard_normal(sh + (8,)) for _ in range(3)]
  l = [rng.standard_normal(sh) * 3 for _ in range(3)]
  ab = O.merge_lse(o[0], l[0], o[1], l[1])
  ba = O.merge_lse(o[1], l[1], o[0], l[0])
  np.testing.assert_allclose(ab[0], ba[0], rtol=1e-12)  # commutative
  left = O.merge_lse(*ab, o[2], l[2])
  right = O.merge_lse(o[0], l[0], *O.merge_lse(o[1], l[1], o[2], l[2]))
  np.testing.assert_allclose(left[0], right[0], rtol=1e-10)  # associative
  np.testing.assert_allclose(left[1], right[1], rtol=1e-12)
  n = O.merge_lse(np.zeros(sh + (8,)), np.full(sh, O.LSE_INIT), o[0], l[0])  # neutral element
  np.testing.assert_allclose(n[0], o[0], rtol=1e-15)
  np.testing.assert_allclose(n[1], l[0], rtol=1e-15)
  # (m, l, o) form on un-normalised partials (ring_attention_kernel.py:1120-1130) gives the same result
  m1, m2 = l[0] - 0.7, l[1] + 0.2  # any m with l = exp(lse - m)
  l1, l2 = np.exp(l[0] - m1), np.exp(l[1] - m2)
  mm, ll, oo = O.merge_mlo(m1, l1, o[0] * l1[..., None], m2, l2, o[1] * l2[..., None])
  np.testing.assert_allclose(oo / ll[..., None], ab[0], rtol=1e-10)
  np.testing.assert_allclose(mm + np.log(ll), ab[1], rtol=1e-12)


# ----------------------------------------------------------------------------- LTX-2 rotary forms
def _pair_rotate(x, ang):
  """Neighbouring pairs as complex numbers times exp(i*angle): x [..., 2n], ang [..., n]."""
  z = (x[..., 0::2] + 1j * x[..., 1::2]) * np.exp(1j * ang)
  out = np.empty_like(x)
  out[..., 0::2], out[..., 1::2] = z.real, z.imag
  return out


def test_ltx2_interleaved_form_equals_pair_rotation():
  rng = np.random.default_rng(11)
  B, S, H, D = 2, 5, 3, 16
  x = rng.standard_normal((B, S, H * D))
  ang = rng.uniform(-3, 3, (B, S, H * D // 2))
  cos, sin = np.repeat(np.cos(ang), 2, axis=-1), np.repeat(np.sin(ang), 2, axis=-1)  # attention_ltx2.py:292-295
  got = O.ltx2_apply_rotary_emb(x, cos, sin)
  np.testing.assert_allclose(got, _pair_rotate(x, ang), rtol=0, atol=1e-14)


def test_ltx2_split_form_brute_force_and_permutation_identity():
  rng = np.random.default_rng(12)
  B, S, H, D = 2, 4, 3, 8
  r = D // 2
  x = rng.standard_normal((B, S, H * D))
  ang = rng.uniform(-3, 3, (B, H, S, r))
  got = O.ltx2_apply_split_rotary_emb(x, np.cos(ang), np.sin(ang))
  want = np.empty_like(x)
  for b in range(B):
    for s in range(S):
      for h in range(H):
        for i in range(r):
          f, g = x[b, s, h * D + i], x[b, s, h * D + r + i]
          c, sn = math.cos(ang[b, h, s, i]), math.sin(ang[b, h, s, i])
          want[b, s, h * D + i] = f * c - g * sn
          want[b, s, h * D + r + i] = g * c + f * sn
  np.testing.assert_allclose(got, want, rtol=0, atol=1e-14)
  # a rotation: every (i, i + D/2) pair keeps its length
  xh, gh = x.reshape(B, S, H, 2, r), got.reshape(B, S, H, 2, r)
  np.testing.assert_allclose((gh**2).sum(axis=3), (xh**2).sum(axis=3), rtol=1e-12)
  # interleaving each head's halves turns the split form into the interleaved one
  xi = xh.transpose(0, 1, 2, 4, 3).reshape(B, S, H * D)
  ang_bs = ang.transpose(0, 2, 1, 3).reshape(B, S, H * r)
  via = _pair_rotate(xi, ang_bs).reshape(B, S, H, r, 2).transpose(0, 1, 2, 4, 3).reshape(B, S, H * D)
  np.testing.assert_allclose(got, via, rtol=0, atol=1e-14)


def test_norm_rope_ltx2_modes():
  rng = np.random.default_rng(13)
  x = rng.standard_normal((1, 3, 32))
  w = 1 + 0.1 * rng.standard_normal(32)
  y = O.rmsnorm(x, w)
  np.testing.assert_array_equal(O.norm_rope_ltx2(x, w, None, None, "none"), y)
  zeros = np.zeros((1, 3, 32))
  np.testing.assert_allclose(O.norm_rope_ltx2(x, w, zeros + 1, zeros, "interleaved"), y, atol=1e-15)
  np.testing.assert_allclose(O.norm_rope_ltx2(x, w, np.ones((1, 2, 3, 8)), np.zeros((1, 2, 3, 8)), "split"), y, atol=1e-15)


# ----------------------------------------------------------------------------- backward
def test_attention_bwd_matches_torch_autograd_and_finite_differences():
  import torch

  rng = np.random.default_rng(31)
  H, Sq, Skv, D = 2, 7, 11, 16
  q, k, v, do = (rng.standard_normal(s) for s in ((H, Sq, D), (H, Skv, D), (H, Skv, D), (H, Sq, D)))
  scale = 0.3
  dq, dk, dv = O.attention_bwd(q, k, v, do, scale)
  tq, tk, tv = (torch.tensor(x, dtype=torch.float64, requires_grad=True) for x in (q, k, v))
  out = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, scale=scale)
  out.backward(torch.tensor(do))
  np.testing.assert_allclose(dq, tq.grad.numpy(), rtol=1e-9, atol=1e-12)
  np.testing.assert_allclose(dk, tk.grad.numpy(), rtol=1e-9, atol=1e-12)
  np.testing.assert_allclose(dv, tv.grad.numpy(), rtol=1e-9, atol=1e-12)
  # one directional finite difference per input
  f = lambda a, b, c: float((O.attention(a, b, c, scale)[0] * do).sum())
  eps = 1e-6
  for idx, (x, g) in enumerate(((q, dq), (k, dk), (v, dv))):
    d = rng.standard_normal(x.shape)
    args_p, args_m = [q, k, v], [q, k, v]
    args_p[idx], args_m[idx] = x + eps * d, x - eps * d
    fd = (f(*args_p) - f(*args_m)) / (2 * eps)
    assert abs(fd - float((g * d).sum())) <= 1e-6 * max(1.0, abs(fd))


# ----------------------------------------------------------------------------- fp8 emulation
def test_fp8_emulation_meets_cosine_bar():
  q = O.normal_bf16((2, 128, 128), 0)
  k = O.normal_bf16((2, 512, 128), 1)
  v = O.normal_bf16((2, 512, 128), 2)
  exact, lse = O.attention(q, k, v, 128**-0.5)
  o8, l8 = O.attention_fp8_emulated(q, k, v, 128**-0.5)
  cos = (o8.ravel() @ exact.ravel()) / (np.linalg.norm(o8) * np.linalg.norm(exact))
  assert cos >= 0.995
  assert np.abs(l8 - lse).max() < 0.1
  x8, s = O.quant_e4m3(q)
  assert np.abs(x8).max() == 448.0 and abs(s - np.abs(q).max() / 448.0) < 1e-9
  # power-of-two scales: with exp2, and with the exponential-free softmax (P from the e4m3 byte grid)
  oe, le = O.attention_fp8_emulated(q, k, v, 128**-0.5, pow2_scales=True, code_softmax=False)
  oc, lc = O.attention_fp8_emulated(q, k, v, 128**-0.5, pow2_scales=True)
  for o_, l_ in ((oe, le), (oc, lc)):
    assert (o_.ravel() @ exact.ravel()) / (np.linalg.norm(o_) * np.linalg.norm(exact)) >= 0.995
    assert np.abs(l_ - lse).max() < 0.1
  assert np.abs(lc - le).max() < 0.08 and abs(float(np.mean(lc - le))) < 0.01  # the constant correction centres it


def test_code_softmax_byte_grid():
  """The byte of P~ is round(8 x + 56): exact at the powers of two, never below 0.957 nor above 1.108 of 2^x, mean
  ratio over a binade 1.0404 (the constant the lse is corrected by)."""
  x = np.linspace(-3.0, 5.0, 800001)
  code = np.clip(np.rint(8 * x + 56), 0, 126)
  val = O.dit_attention._e4m3_decode(code).astype(np.float64)
  # the decode agrees with torch's float8_e4m3fn
  bytes_ = torch.arange(0, 127, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
  np.testing.assert_array_equal(O.dit_attention._e4m3_decode(np.arange(127)), bytes_)
  r = val / 2.0**x
  assert 0.957 < r.min() and r.max() < 1.108
  assert abs(np.log2(r.mean()) - 0.0570814) < 2e-4
  for n in range(-3, 6):
    assert O.dit_attention._e4m3_decode(np.rint(8 * n + 56)) == 2.0**n


# ----------------------------------------------------------------------------- workloads
def test_workload_table_matches_baseline_configs():
  w = O.WORKLOADS
  assert (w["wan1.3b"].heads, w["wan1.3b"].seq, math.prod(w["wan1.3b"].grid)) == (12, 4680, 4680)
  assert (w["flux-dev"].heads, w["flux-dev"].seq) == (24, 512 + 64 * 64)
  assert (w["wan14b"].heads, w["wan14b"].seq, math.prod(w["wan14b"].grid), w["wan14b"].cross_kv) == (40, 75600, 75600, 512)
  assert w["wan14b-ring"].seq * w["wan14b-ring"].ring_chunks == 75600
  assert O.attention_flops(1, 40, 75600, 75600, 128) == pytest.approx(1.1705e14, rel=1e-4)
  assert O.normrope_bytes(1, 75600, 40, 128, with_table=False) == pytest.approx(3.097e9, rel=1e-3)
  rows = O.sample_rows(75600)
  assert rows[0] == 0 and rows[-1] == 75599 and 128 in rows and len(rows) > 200


# ----------------------------------------------------------------------------- committed golden vectors
def test_committed_golden_vectors_follow_the_oracle():
  from helpers import bits_to_f32, golden, hsd

  g = golden("attention_small.npz")
  q, k, v = (bits_to_f32(g[n]) for n in ("q", "k", "v"))
  out, lse = O.attention(hsd(q), hsd(k), hsd(v), float(g["scale"]))
  np.testing.assert_allclose(out.transpose(1, 0, 2)[None], g["out"], atol=1e-6)
  np.testing.assert_allclose(lse[None], g["lse"], atol=1e-5)
  g = golden("norm_rope_wan.npz")
  got = O.norm_rope_fullrow(bits_to_f32(g["q"]), bits_to_f32(g["wq"]), g["cos"], g["sin"], int(g["heads"]))
  np.testing.assert_allclose(got, g["q_out"], atol=1e-6)
  g = golden("norm_rope_flux.npz")
  got = O.norm_rope_perhead(bits_to_f32(g["k"]), bits_to_f32(g["wk"]), g["cos"], g["sin"], w_txt=bits_to_f32(g["wk_txt"]), n_txt=int(g["n_txt"]))
  np.testing.assert_allclose(got, g["k_out"], atol=1e-6)
  g = golden("norm_rope_ltx2.npz")
  x = bits_to_f32(g["x"])
  np.testing.assert_allclose(O.norm_rope_ltx2(x, g["w"], g["cos_i"], g["sin_i"], "interleaved"), g["out_interleaved"], atol=1e-6)
  np.testing.assert_allclose(O.norm_rope_ltx2(x, g["w"], g["cos_s"], g["sin_s"], "split"), g["out_split"], atol=1e-6)
  g = golden("attention_bwd_small.npz")
  dq, dk, dv = O.attention_bwd(*(hsd(bits_to_f32(g[n])) for n in ("q", "k", "v", "do")), float(g["scale"]))
  np.testing.assert_allclose(dv.transpose(1, 0, 2)[None], g["dv"], atol=1e-6)
  np.testing.assert_allclose(dq.transpose(1, 0, 2)[None], g["dq"], atol=1e-6)
  g = golden("merge_small.npz")
  o_run, l_run = np.zeros((1, 2, 70, 128)), np.full((1, 2, 70), O.LSE_INIT)
  for ob, lb in zip(g["parts_o"], g["parts_l"]):
    o_run, l_run = O.merge_lse(o_run, l_run, bits_to_f32(ob).transpose(0, 2, 1, 3), lb)
  np.testing.assert_allclose(o_run.transpose(0, 2, 1, 3), g["o_merged"], atol=1e-6)
