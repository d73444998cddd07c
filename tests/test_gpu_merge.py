"""Chunk merge + ring replay on the device against the oracle (the benchmark's ring-shard configuration: 8 chunks of 9,450 tokens)."""
import numpy as np
import pytest
import torch

import oracle as O
from helpers import bits_to_dev, err_stats, golden, hsd, rel_l2, to_dev_bf16, to_np, torch_attention_f32
from maxdiffusion_amd import ops

pytestmark = pytest.mark.gpu


def test_golden_merge(dev):
  g = golden("merge_small.npz")
  o_run, l_run = ops.new_merge_state(1, 70, 2, 128, dev)
  for ob, lb in zip(g["parts_o"], g["parts_l"]):
    ops.merge_partial(o_run, l_run, bits_to_dev(ob, dev), torch.from_numpy(lb).to(dev))
  assert err_stats(to_np(o_run), g["o_merged"])[0] < 1e-6
  assert err_stats(to_np(l_run), g["lse_merged"])[0] < 1e-5
  fin = ops.finalize(o_run)
  assert fin.dtype == torch.bfloat16
  assert torch.equal(fin, o_run.to(torch.bfloat16))  # round-to-nearest-even cast


def test_merge_f32_partials_layouts_and_neutral_element(dev):
  rng = np.random.default_rng(0)
  B, S, H, D = 2, 33, 3, 128
  o1, o2 = rng.standard_normal((B, S, H, D)).astype(np.float32), rng.standard_normal((B, S, H, D)).astype(np.float32)
  l1, l2 = (rng.standard_normal((B, H, S)) * 4).astype(np.float32), (rng.standard_normal((B, H, S)) * 4).astype(np.float32)
  want_o, want_l = O.merge_lse(o1.transpose(0, 2, 1, 3), l1, o2.transpose(0, 2, 1, 3), l2)
  for layout in ("bshd", "bhsd"):
    o_run, l_run = ops.new_merge_state(B, S, H, D, dev, layout=layout)
    ops.merge_partial(o_run, l_run, torch.from_numpy(o1).to(dev), torch.from_numpy(l1).to(dev))  # into the neutral element
    assert err_stats(to_np(o_run), o1)[0] < 1e-6 and err_stats(to_np(l_run), l1)[0] < 1e-6
    cur = torch.from_numpy(o2).to(dev).permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)  # a [B,H,S,D] partial
    ops.merge_partial(o_run, l_run, cur, torch.from_numpy(l2).to(dev))
    assert err_stats(to_np(o_run), want_o.transpose(0, 2, 1, 3))[0] < 2e-6
    assert err_stats(to_np(l_run), want_l)[0] < 2e-6
  # an empty partial (lse = -inf) leaves the state untouched; two empty states stay empty with out = 0
  o_run, l_run = ops.new_merge_state(1, 8, 1, 128, dev)
  o_run.fill_(1.5); l_run.fill_(0.25)
  ops.merge_partial(o_run, l_run, torch.zeros_like(o_run), torch.full_like(l_run, float("-inf")))
  assert float((o_run - 1.5).abs().max()) == 0 and float((l_run - 0.25).abs().max()) == 0
  l_run.fill_(float("-inf"))
  ops.merge_partial(o_run, l_run, torch.ones_like(o_run), torch.full_like(l_run, float("-inf")))
  assert float(o_run.abs().max()) == 0 and bool(torch.isneginf(l_run).all())


def test_ring_replay_small_unequal_chunks(dev):
  # tests/ring_fixed_m_test.py:156-189 (2 x 2048 shards) and its ragged-tail case :173-180, re-expressed on one GPU
  H = 5
  q = O.normal_bf16((1, 300, H, 128), 0)
  sizes = [2048, 2048, 1, 63, 777]
  ks = [O.normal_bf16((1, n, H, 128), 10 + i) for i, n in enumerate(sizes)]
  vs = [O.normal_bf16((1, n, H, 128), 20 + i) for i, n in enumerate(sizes)]
  o_run, l_run = ops.new_merge_state(1, 300, H, 128, dev)
  qd = to_dev_bf16(q, dev)
  for kc, vc in zip(ks, vs):
    o, l = ops.flash_attention(qd, to_dev_bf16(kc, dev), to_dev_bf16(vc, dev), return_lse=True)
    ops.merge_partial(o_run, l_run, o, l)
  ro, rl = O.attention(hsd(q), hsd(np.concatenate(ks, 1)), hsd(np.concatenate(vs, 1)), 128**-0.5)
  out = to_np(ops.finalize(o_run))
  mx, mean = err_stats(hsd(out), ro)
  print(f"ring small: max-abs {mx:.3e} mean-abs {mean:.3e}")
  assert mx < 2e-2 and mean < 2e-3 and rel_l2(hsd(out), ro) < 1.5e-2
  assert err_stats(to_np(l_run)[0], rl)[0] < 1e-3


@pytest.mark.parametrize("layout", ["bshd", "bhsd"])
@pytest.mark.parametrize("variant,D", [(0, 128), (1, 128), (3, 128), (0, 64)])
def test_fused_ring_step_equals_attention_then_merge(dev, request, layout, variant, D):
  """mdattn_fwd_bf16_merge (attention + merge in the attention kernel's epilogue) against the two separate calls
  and against the oracle, with ragged chunks, through both schedules and both layouts of the carry, at both head dims."""
  ops.set_fwd_schedule(variant)
  request.addfinalizer(lambda: ops.set_fwd_schedule(0))
  H, Sq = 3, 333
  q = O.normal_bf16((1, Sq, H, D), 0)
  sizes = [4200, 1, 63, 777, 3100]
  ks = [O.normal_bf16((1, n, H, D), 10 + i) for i, n in enumerate(sizes)]
  vs = [O.normal_bf16((1, n, H, D), 20 + i) for i, n in enumerate(sizes)]
  qd = to_dev_bf16(q, dev)
  o_f, l_f = ops.new_merge_state(1, Sq, H, D, dev, layout=layout)
  o_s, l_s = ops.new_merge_state(1, Sq, H, D, dev, layout=layout)
  for kc, vc in zip(ks, vs):
    kd, vd = to_dev_bf16(kc, dev), to_dev_bf16(vc, dev)
    ops.flash_attention_merge(qd, kd, vd, o_f, l_f)
    o, l = ops.flash_attention(qd, kd, vd, return_lse=True)
    ops.merge_partial(o_s, l_s, o, l)
  # the separate path rounds each chunk's output to bf16 before the merge, the fused one does not
  assert float((o_f - o_s).abs().max()) < 8e-3
  assert float((l_f - l_s).abs().max()) < 1e-5
  ro, rl = O.attention(hsd(q), hsd(np.concatenate(ks, 1)), hsd(np.concatenate(vs, 1)), D**-0.5)
  out = to_np(ops.finalize(o_f))
  mx, mean = err_stats(hsd(out), ro)
  mx_s = err_stats(hsd(to_np(ops.finalize(o_s))), ro)[0]
  print(f"fused ring step ({layout}, variant {variant}, D={D}): max-abs {mx:.3e} (separate calls {mx_s:.3e}) mean-abs {mean:.3e}")
  assert mx < 2e-2 and mean < 2e-3 and rel_l2(hsd(out), ro) < 1.5e-2
  assert err_stats(to_np(l_f)[0], rl)[0] < 1e-3


def test_fused_ring_step_neutral_start_and_folded_scale(dev):
  """A single fused step from the neutral start is the attention itself (f32, unrounded), also with the softmax
  scale carried by q (scale = ln 2)."""
  H, Sq, Skv = 2, 100, 5000
  q, k, v = O.normal_bf16((1, Sq, H, 128), 0), O.normal_bf16((1, Skv, H, 128), 1), O.normal_bf16((1, Skv, H, 128), 2)
  for folded in (False, True):
    qd = to_dev_bf16(O.bf16_round(q * np.float32(ops.folded_q_mul(128))) if folded else q, dev)
    sc = ops.FOLDED_SCALE if folded else None
    o_run, l_run = ops.new_merge_state(1, Sq, H, 128, dev)
    ops.flash_attention_merge(qd, to_dev_bf16(k, dev), to_dev_bf16(v, dev), o_run, l_run, scale=sc)
    out, lse = ops.flash_attention(qd, to_dev_bf16(k, dev), to_dev_bf16(v, dev), scale=sc, return_lse=True)
    assert float((o_run - out.float()).abs().max()) < 4e-3  # out is the bf16 rounding of what o_run holds
    assert float((l_run - lse).abs().max()) < 1e-6
    assert to_np(ops.finalize(o_run)).tobytes() == to_np(out).tobytes()


def test_wan14b_ring_shard_replay_full_size(dev):
  """Config 3: a 9 450-token Q chunk x 40 heads against 8 successive 9 450-token KV chunks; the merged
  result must equal full 75 600-token attention for that Q chunk."""
  w = O.WORKLOADS["wan14b-ring"]
  C, n = w.seq, w.ring_chunks
  gen = torch.Generator(device=dev).manual_seed(3)
  mk = lambda s: torch.randn((1, s, w.heads, 128), generator=gen, device=dev, dtype=torch.float32).to(torch.bfloat16)
  q, k, v = mk(C), mk(C * n), mk(C * n)
  o_run, l_run = ops.new_merge_state(1, C, w.heads, 128, dev)
  for i in range(n):
    o, l = ops.flash_attention(q, k[:, i * C:(i + 1) * C], v[:, i * C:(i + 1) * C], scale=w.scale, return_lse=True)
    ops.merge_partial(o_run, l_run, o, l)
  merged = ops.finalize(o_run)
  full, full_l = ops.flash_attention(q, k, v, scale=w.scale, return_lse=True)  # one pass over all 75 600 keys
  assert float((merged.float() - full.float()).abs().max()) < 2e-3
  assert float((l_run - full_l).abs().max()) < 1e-4
  for h0 in range(0, w.heads, 8):  # and both against the torch f32 reference on the whole chunk
    ro, rl = torch_attention_f32(q[:, :, h0:h0 + 8], k[:, :, h0:h0 + 8], v[:, :, h0:h0 + 8], w.scale, q_block=1024)
    d = (merged[:, :, h0:h0 + 8].float() - ro).abs()
    assert float(d.max()) <= 2e-2 and float(d.mean()) <= 2e-3
    assert float((merged[:, :, h0:h0 + 8].float() - ro).norm() / ro.norm()) <= 1.5e-2
    assert float((l_run[:, h0:h0 + 8] - rl).abs().max()) <= 1e-3
  rows = O.sample_rows(C, n_random=24)
  idx = torch.from_numpy(rows).to(dev)
  for h in (0, 21, 39):  # CPU oracle on sampled rows
    co, cl = O.attention_rows(to_np(q[0, idx, h]), to_np(k[0, :, h]), to_np(v[0, :, h]), w.scale)
    assert err_stats(to_np(merged[0, idx, h]), co)[0] <= 2e-2 and rel_l2(to_np(merged[0, idx, h]), co) <= 1.5e-2
    assert err_stats(to_np(l_run[0, h, idx]), cl)[0] <= 1e-3


def test_wan14b_ring_shard_fused_hops_full_size(dev):
  """Config 3 the way the benchmark runs it: the prologue carries the softmax scale (q * D^-1/2 * log2 e, kernel
  given scale = ln 2) and each of the 8 hops is ONE launch of mdattn_fwd_bf16_merge (attention and merge in the
  attention kernel's epilogue).  The merged result must equal the one-pass attention over all 75 600 keys, the torch
  f32 reference on the whole chunk and the CPU oracle on sampled rows."""
  w = O.WORKLOADS["wan14b-ring"]
  C, n, H, D = w.seq, w.ring_chunks, w.heads, 128
  gen = torch.Generator(device=dev).manual_seed(3)
  mk = lambda s: torch.randn((1, s, H, D), generator=gen, device=dev, dtype=torch.float32).to(torch.bfloat16)
  q = (mk(C).float() * ops.folded_q_mul(D, w.scale)).to(torch.bfloat16)  # what the prologue hands over
  k, v = mk(C * n), mk(C * n)
  sc = ops.FOLDED_SCALE
  o_run, l_run = ops.new_merge_state(1, C, H, D, dev)
  for i in range(n):
    ops.flash_attention_merge(q, k[:, i * C:(i + 1) * C], v[:, i * C:(i + 1) * C], o_run, l_run, scale=sc)
  merged = ops.finalize(o_run)
  full, full_l = ops.flash_attention(q, k, v, scale=sc, return_lse=True)  # one pass over all 75 600 keys
  d_o, d_l = float((merged.float() - full.float()).abs().max()), float((l_run - full_l).abs().max())
  print(f"fused ring hops vs one pass: out {d_o:.3e} lse {d_l:.3e}", flush=True)
  assert d_o < 2e-3 and d_l < 1e-4
  for h0 in range(0, H, 8):
    ro, rl = torch_attention_f32(q[:, :, h0:h0 + 8], k[:, :, h0:h0 + 8], v[:, :, h0:h0 + 8], sc, q_block=1024)
    d = (merged[:, :, h0:h0 + 8].float() - ro).abs()
    assert float(d.max()) <= 2e-2 and float(d.mean()) <= 2e-3
    assert float((merged[:, :, h0:h0 + 8].float() - ro).norm() / ro.norm()) <= 1.5e-2
    assert float((l_run[:, h0:h0 + 8] - rl).abs().max()) <= 1e-3
  rows = O.sample_rows(C, n_random=24)
  idx = torch.from_numpy(rows).to(dev)
  for h in (0, 21, 39):
    co, cl = O.attention_rows(to_np(q[0, idx, h]), to_np(k[0, :, h]), to_np(v[0, :, h]), sc)
    assert err_stats(to_np(merged[0, idx, h]), co)[0] <= 2e-2 and rel_l2(to_np(merged[0, idx, h]), co) <= 1.5e-2
    assert err_stats(to_np(l_run[0, h, idx]), cl)[0] <= 1e-3
