"""Key padding masks: `[B,Skv]` keep-masks through the additive-bias entry point (HIP, through the C ABI).

Oracle: dense softmax with the masked keys excluded; rows without a kept key return 0
(models/attention_flax.py:1552-1554).  Hand fixtures follow the reference's own mask tests
(tests/ltx2/test_attention_ltx2.py:38-116)."""
import math

import numpy as np
import pytest
import torch

import oracle as O
from helpers import err_stats, hsd, rel_l2, to_dev_bf16, to_np
from maxdiffusion_amd import attention_op, ops

pytestmark = pytest.mark.gpu
MAX_ABS, MEAN_ABS, LSE_ABS, REL_L2 = 2e-2, 2e-3, 1e-3, 1.5e-2


def test_mask_bias_kernel(dev):
  keep = torch.tensor([[1, 0, 1, 1, 0], [0, 0, 0, 0, 1]], dtype=torch.bool, device=dev)
  bias = ops.key_mask_bias(keep)
  assert bias.shape == (2, 32) and bias.dtype == torch.float32
  want = torch.full((2, 32), -math.inf)
  want[0, [0, 2, 3]] = 0.0
  want[1, 4] = 0.0
  assert torch.equal(bias.cpu(), want)
  assert torch.equal(ops.key_mask_bias(keep, masked_value=-10000.0).cpu(), torch.where(want == 0, want, torch.tensor(-10000.0)))


@pytest.mark.parametrize("sq,skv,kind", [(70, 333, "random"), (257, 512, "prefix"), (64, 97, "holes"), (33, 64, "one")])
def test_masked_attention_against_oracle(dev, sq, skv, kind):
  B, H = 2, 3
  q, k, v = O.normal_bf16((B, sq, H, 128), 0), O.normal_bf16((B, skv, H, 128), 1), O.normal_bf16((B, skv, H, 128), 2)
  rng = np.random.default_rng(5)
  keep = np.ones((B, skv), bool)
  if kind == "random":
    keep = rng.random((B, skv)) < 0.6
  elif kind == "prefix":  # padding masks: batch 0 keeps 300 keys, batch 1 keeps 77
    keep[0, 300:] = False
    keep[1, 77:] = False
  elif kind == "holes":  # whole 32-key tiles masked out, first tile included
    keep[0, :32] = False
    keep[1, 32:64] = False
    keep[1, 90:] = False
  else:  # a single kept key: out = that key's value row, lse = its logit
    keep[:] = False
    keep[0, 40] = True
    keep[1, 63] = True
  bias = ops.key_mask_bias(torch.from_numpy(keep).to(dev))
  out, lse = ops.flash_attention(to_dev_bf16(q, dev), to_dev_bf16(k, dev), to_dev_bf16(v, dev), return_lse=True, key_bias=bias)
  out, lse = to_np(out), to_np(lse)
  for b in range(B):
    ro, rl = O.attention(hsd(q[b:b + 1]), hsd(k[b:b + 1]), hsd(v[b:b + 1]), 128**-0.5, kv_mask=keep[b])
    mx, mean = err_stats(hsd(out[b:b + 1]), ro)
    lmx = float(np.abs(lse[b] - rl).max())
    print(f"mask {kind} Sq={sq} Skv={skv} batch {b}: out max-abs {mx:.3e} mean-abs {mean:.3e} rel-l2 {rel_l2(hsd(out[b:b+1]), ro):.3e} lse {lmx:.3e}", flush=True)
    assert mx <= MAX_ABS and mean <= MEAN_ABS and rel_l2(hsd(out[b:b + 1]), ro) <= REL_L2 and lmx <= LSE_ABS
  # the same mask with the softmax scale carried by q (scale = ln 2 for the kernel): the masked kernel keeps its
  # multiply, the result is the one of the plain call on these inputs
  qf = O.bf16_round((q * np.float32(ops.folded_q_mul(128))).astype(np.float32))
  out2, lse2 = ops.flash_attention(to_dev_bf16(qf, dev), to_dev_bf16(k, dev), to_dev_bf16(v, dev), scale=ops.FOLDED_SCALE,
                                   return_lse=True, key_bias=bias)
  for b in range(B):
    ro, rl = O.attention(hsd(qf[b:b + 1]), hsd(k[b:b + 1]), hsd(v[b:b + 1]), ops.FOLDED_SCALE, kv_mask=keep[b])
    mx, mean = err_stats(hsd(to_np(out2)[b:b + 1]), ro)
    assert mx <= MAX_ABS and mean <= MEAN_ABS and float(np.abs(to_np(lse2)[b] - rl).max()) <= LSE_ABS


def test_all_keys_masked_rows_return_zero_and_all_kept_equals_unmasked(dev):
  B, S, H = 2, 100, 2
  q, k, v = (to_dev_bf16(O.normal_bf16((B, S, H, 128), s), dev) for s in (0, 1, 2))
  keep = torch.ones((B, S), dtype=torch.bool, device=dev)
  keep[1] = False  # batch 1: nothing to attend to
  out, lse = ops.flash_attention(q, k, v, return_lse=True, key_bias=ops.key_mask_bias(keep))
  base, lse0 = ops.flash_attention(q, k, v, return_lse=True)
  # same arithmetic up to where the scale is applied (before instead of inside the exp2 argument): bf16 ulps
  assert torch.allclose(out[0].float(), base[0].float(), atol=2e-3, rtol=1e-2) and torch.allclose(lse[0], lse0[0], atol=1e-5)
  assert torch.count_nonzero(out[1]) == 0 and bool(torch.isneginf(lse[1]).all())


def test_reference_hand_fixture_and_dispatcher(dev):
  # tests/ltx2/test_attention_ltx2.py:38-76: two keys, the second masked -> every query returns v[0]
  H, D = 2, 128
  q = torch.randn(1, 5, H * D, device=dev).to(torch.bfloat16)
  k = torch.randn(1, 2, H * D, device=dev).to(torch.bfloat16)
  v = torch.randn(1, 2, H * D, device=dev).to(torch.bfloat16)
  op = attention_op.AttentionOp(attention_kernel="hip_flash", heads=H, dim_head=D, scale=D**-0.5)
  got = op.apply_attention(q, k, v, attention_mask=torch.tensor([[1, 0]], device=dev))
  assert got.shape == (1, 5, H * D)
  assert torch.equal(got, v[:, :1].expand(1, 5, H * D))
  # :91-116: everything masked -> zeros
  got = op.apply_attention(q, k, v, attention_mask=torch.tensor([[0, 0]], device=dev))
  assert torch.count_nonzero(got) == 0
