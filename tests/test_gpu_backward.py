"""Backward of the bf16 attention forward (HIP, through the C ABI) against the f64 oracle
(kernels/splash_attention/base.py:108-160 restated with the scale inside).

Gradients are bf16 results of bf16 inputs: the bar is a relative L2 error of 6e-3 per tensor and a max-abs error of
1.5 % of the tensor's largest gradient (observed: 2.4e-3 and 0.6 %, one bf16 rounding of P / dS and of the result)."""
import numpy as np
import pytest
import torch

import oracle as O
from helpers import bits_to_dev, golden, hsd, rel_l2, to_dev_bf16, to_np
from maxdiffusion_amd import ops

pytestmark = pytest.mark.gpu


def _check(got, ref, what):
  if float(np.abs(ref).max()) < 1e-9:
    # a gradient that is exactly zero (one key: p = 1, ds = 0): the kernel's value is the bf16 rounding of `out`
    # inside delta = rowsum(dout * out), a few 1e-2 of |dout||v||k| at most
    print(f"{what}: exact gradient is 0, got max-abs {float(np.abs(got).max()):.3e}", flush=True)
    assert float(np.abs(got).max()) <= 0.25, what
    return
  r = rel_l2(got, ref)
  mx = float(np.abs(got - ref).max()) / max(float(np.abs(ref).max()), 1e-30)
  print(f"{what}: rel-l2 {r:.3e} max-abs/max|ref| {mx:.3e}", flush=True)
  assert r <= 6e-3 and mx <= 1.5e-2, what


def _run(q, k, v, do, dev, scale=None, layout="bshd"):
  qd, kd, vd, dod = (to_dev_bf16(x, dev) for x in (q, k, v, do))
  if layout == "bhsd":
    f = lambda t: t.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    qd, kd, vd = f(qd), f(kd), f(vd)
  out, lse = ops.flash_attention(qd, kd, vd, scale=scale, return_lse=True, out_layout=layout)
  if layout == "bhsd":
    dod = dod.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
  dq, dk, dv = ops.flash_attention_backward(qd, kd, vd, out, dod, lse, scale=scale)
  assert dq.stride() == qd.stride() and dk.stride() == kd.stride()
  return to_np(dq), to_np(dk), to_np(dv)


@pytest.mark.parametrize("sq,skv", [(1, 1), (31, 65), (257, 63), (300, 333), (64, 1025), (513, 512)])
def test_backward_ragged_shapes(dev, sq, skv):
  B, H = 2, 3
  q, do = O.normal_bf16((B, sq, H, 128), 0), O.normal_bf16((B, sq, H, 128), 3)
  k, v = O.normal_bf16((B, skv, H, 128), 1), O.normal_bf16((B, skv, H, 128), 2)
  dq, dk, dv = _run(q, k, v, do, dev)
  for b in range(B):
    rq, rk, rv = O.attention_bwd(hsd(q[b:b + 1]), hsd(k[b:b + 1]), hsd(v[b:b + 1]), hsd(do[b:b + 1]), 128**-0.5)
    _check(hsd(dq[b:b + 1]), rq, f"dq Sq={sq} Skv={skv} b{b}")
    _check(hsd(dk[b:b + 1]), rk, f"dk Sq={sq} Skv={skv} b{b}")
    _check(hsd(dv[b:b + 1]), rv, f"dv Sq={sq} Skv={skv} b{b}")


def test_backward_layout_scale_and_sharp_logits(dev):
  H, sq, skv = 4, 200, 260
  q = O.bf16_round(O.normal_bf16((1, sq, H, 128), 0) * np.float32(4.0))
  k, v, do = O.normal_bf16((1, skv, H, 128), 1), O.normal_bf16((1, skv, H, 128), 2), O.normal_bf16((1, sq, H, 128), 3)
  for layout in ("bshd", "bhsd"):
    dq, dk, dv = _run(q, k, v, do, dev, scale=0.07, layout=layout)
    rq, rk, rv = O.attention_bwd(hsd(q), hsd(k), hsd(v), hsd(do), 0.07)
    _check(hsd(dq), rq, f"dq {layout} sharp")
    _check(hsd(dk), rk, f"dk {layout} sharp")
    _check(hsd(dv), rv, f"dv {layout} sharp")


@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("sq,skv", [(1, 1), (257, 63), (300, 333), (513, 512)])
def test_backward_scale_carried_by_q(dev, D, sq, skv):
  """scale = ln 2 on a q that already carries D^-1/2 * log2(e) (what the prologue's q_mul produces for the forward):
  scale * log2(e) is 1 and the library takes the kernels whose logits leave the MFMAs in log2 units.  dq is the
  gradient with respect to the q that was passed."""
  import math
  B, H = 2, 3
  q = O.bf16_round(O.normal_bf16((B, sq, H, D), 0) * np.float32(D**-0.5 * math.log2(math.e)))
  do = O.normal_bf16((B, sq, H, D), 3)
  k, v = O.normal_bf16((B, skv, H, D), 1), O.normal_bf16((B, skv, H, D), 2)
  dq, dk, dv = _run(q, k, v, do, dev, scale=math.log(2.0))
  for b in range(B):
    rq, rk, rv = O.attention_bwd(hsd(q[b:b + 1]), hsd(k[b:b + 1]), hsd(v[b:b + 1]), hsd(do[b:b + 1]), math.log(2.0))
    _check(hsd(dq[b:b + 1]), rq, f"folded D={D} dq Sq={sq} Skv={skv} b{b}")
    _check(hsd(dk[b:b + 1]), rk, f"folded D={D} dk Sq={sq} Skv={skv} b{b}")
    _check(hsd(dv[b:b + 1]), rv, f"folded D={D} dv Sq={sq} Skv={skv} b{b}")


def test_backward_accepts_dout_in_another_layout_than_out(dev):
  """out stored [B,H,S,D], dout contiguous [B,S,H,D] (what autograd hands over): the wrapper has to re-lay dout like
  out, element by element."""
  H, sq, skv = 3, 130, 200
  q, k, v, do = (O.normal_bf16((1, s_, H, 128), i) for i, s_ in enumerate((sq, skv, skv, sq)))
  qd, kd, vd, dod = (to_dev_bf16(x, dev) for x in (q, k, v, do))
  out, lse = ops.flash_attention(qd, kd, vd, return_lse=True, out_layout="bhsd")
  assert out.stride() != dod.stride()
  dq, dk, dv = ops.flash_attention_backward(qd, kd, vd, out, dod, lse)
  rq, rk, rv = O.attention_bwd(hsd(q), hsd(k), hsd(v), hsd(do), 128**-0.5)
  _check(hsd(to_np(dq)), rq, "dq, dout bshd / out bhsd")
  _check(hsd(to_np(dk)), rk, "dk, dout bshd / out bhsd")
  _check(hsd(to_np(dv)), rv, "dv, dout bshd / out bhsd")


def test_backward_wan13b_shape_against_torch_autograd_on_gpu(dev):
  """configs[0] size (12 heads x 4680 tokens): whole tensors against torch's f32 autograd (test harness only)."""
  w = O.WORKLOADS["wan1.3b"]
  H, S = w.heads, w.seq
  gen = torch.Generator(device=dev).manual_seed(7)
  q, k, v, do = (torch.randn((1, S, H, 128), generator=gen, device=dev, dtype=torch.float32).to(torch.bfloat16) for _ in range(4))
  out, lse = ops.flash_attention(q, k, v, scale=w.scale, return_lse=True)
  dq, dk, dv = ops.flash_attention_backward(q, k, v, out, do, lse, scale=w.scale)
  tq, tk, tv = (x.float().permute(0, 2, 1, 3).detach().requires_grad_(True) for x in (q, k, v))
  ref = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, scale=w.scale)
  ref.backward(do.float().permute(0, 2, 1, 3))
  for name, got, t in (("dq", dq, tq), ("dk", dk, tk), ("dv", dv, tv)):
    _check(to_np(got), to_np(t.grad.permute(0, 2, 1, 3)), f"wan1.3b {name}")


@pytest.mark.parametrize("folded", [False, True])
def test_backward_wan14b_usp_shard_full_size(dev, folded):
  """The shape `bench.py --workload wan14b-usp --with-backward` times (20 heads x 18,900 tokens), whole tensors,
  head by head against torch's f32 autograd on the GPU (test harness only); `folded`: q carries the softmax scale and
  scale = ln 2, which selects the kernels whose logits leave the MFMAs in log2 units."""
  import math
  H, S, D = 20, 18900, 128
  gen = torch.Generator(device=dev).manual_seed(11)
  q, k, v, do = (torch.randn((1, S, H, D), generator=gen, device=dev, dtype=torch.float32).to(torch.bfloat16) for _ in range(4))
  scale = D**-0.5
  if folded:
    q = (q.float() * (scale * math.log2(math.e))).to(torch.bfloat16)
    scale = math.log(2.0)
  out, lse = ops.flash_attention(q, k, v, scale=scale, return_lse=True)
  dq, dk, dv = ops.flash_attention_backward(q, k, v, out, do, lse, scale=scale)
  worst = {}
  for h in (range(H) if not folded else (0, 7, 13, 19)):
    tq, tk, tv = (x[:, :, h].float().detach().requires_grad_(True) for x in (q, k, v))  # [1,S,D]
    p = torch.softmax((tq @ tk.transpose(1, 2)) * scale, dim=-1)
    (p @ tv).backward(do[:, :, h].float())
    for name, got, t in (("dq", dq, tq), ("dk", dk, tk), ("dv", dv, tv)):
      g, r = got[:, :, h].float(), t.grad
      rel = float((g - r).norm() / r.norm())
      mx = float((g - r).abs().max() / r.abs().max())
      worst[name] = max(worst.get(name, (0.0, 0.0)), (rel, mx))
      assert rel <= 6e-3 and mx <= 1.5e-2, (name, h, rel, mx)
    del p, tq, tk, tv
  print(f"usp backward folded={folded}: worst (rel-l2, max-abs/max|ref|) {worst}", flush=True)


def test_autograd_function(dev):
  from maxdiffusion_amd import attention_op

  H, S = 2, 150
  q, k, v = (to_dev_bf16(O.normal_bf16((1, S, H, 128), s), dev).requires_grad_(True) for s in (0, 1, 2))
  out = attention_op.hip_flash_attention_autograd(q, k, v, 128**-0.5)
  g = to_dev_bf16(O.normal_bf16((1, S, H, 128), 3), dev)
  out.backward(g)
  rq, rk, rv = O.attention_bwd(hsd(to_np(q)), hsd(to_np(k)), hsd(to_np(v)), hsd(to_np(g)), 128**-0.5)
  _check(hsd(to_np(q.grad)), rq, "autograd dq")
  _check(hsd(to_np(k.grad)), rk, "autograd dk")
  _check(hsd(to_np(v.grad)), rv, "autograd dv")


def test_backward_golden(dev):
  g = golden("attention_bwd_small.npz")
  q, k, v, do = (bits_to_dev(g[n], dev) for n in ("q", "k", "v", "do"))
  out, lse = ops.flash_attention(q, k, v, scale=float(g["scale"]), return_lse=True)
  dq, dk, dv = ops.flash_attention_backward(q, k, v, out, do, lse, scale=float(g["scale"]))
  _check(to_np(dq), g["dq"], "golden dq")
  _check(to_np(dk), g["dk"], "golden dk")
  _check(to_np(dv), g["dv"], "golden dv")


@pytest.mark.parametrize("sq,skv", [(1, 1), (31, 65), (257, 63), (300, 333), (513, 512)])
def test_backward_head_dim_64(dev, sq, skv):
  # LTX-2's audio stream: heads of 64 (models/ltx2/transformer_ltx2.py:788-789)
  B, H, D = 2, 3, 64
  q, do = O.normal_bf16((B, sq, H, D), 0), O.normal_bf16((B, sq, H, D), 3)
  k, v = O.normal_bf16((B, skv, H, D), 1), O.normal_bf16((B, skv, H, D), 2)
  for layout in ("bshd", "bhsd"):
    dq, dk, dv = _run(q, k, v, do, dev, layout=layout)
    for b in range(B):
      rq, rk, rv = O.attention_bwd(hsd(q[b:b + 1]), hsd(k[b:b + 1]), hsd(v[b:b + 1]), hsd(do[b:b + 1]), D**-0.5)
      _check(hsd(dq[b:b + 1]), rq, f"D=64 dq Sq={sq} Skv={skv} b{b} {layout}")
      _check(hsd(dk[b:b + 1]), rk, f"D=64 dk Sq={sq} Skv={skv} b{b} {layout}")
      _check(hsd(dv[b:b + 1]), rv, f"D=64 dv Sq={sq} Skv={skv} b{b} {layout}")


@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("sq,skv,kind", [(70, 333, "random"), (257, 512, "prefix"), (64, 97, "holes"), (33, 64, "one"), (40, 50, "none")])
def test_backward_with_key_mask(dev, D, sq, skv, kind):
  """Gradients through mdattn_fwd_bf16_bias: masked keys get exactly zero dk and dv; a batch element without any kept
  key (forward: out = 0, lse = -inf) gets zero gradients everywhere."""
  B, H = 2, 3
  q, do = O.normal_bf16((B, sq, H, D), 0), O.normal_bf16((B, sq, H, D), 3)
  k, v = O.normal_bf16((B, skv, H, D), 1), O.normal_bf16((B, skv, H, D), 2)
  rng = np.random.default_rng(5)
  keep = np.ones((B, skv), bool)
  if kind == "random":
    keep = rng.random((B, skv)) < 0.6
  elif kind == "prefix":
    keep[0, 300:] = False
    keep[1, 77:] = False
  elif kind == "holes":
    keep[0, :32] = False
    keep[1, 32:64] = False
    keep[1, 90:] = False
  elif kind == "one":
    keep[:] = False
    keep[0, 40] = True
    keep[1, 63] = True
  else:  # batch 1 keeps nothing
    keep[1] = False
  qd, kd, vd, dod = (to_dev_bf16(x, dev) for x in (q, k, v, do))
  bias = ops.key_mask_bias(torch.from_numpy(keep).to(dev))
  out, lse = ops.flash_attention(qd, kd, vd, return_lse=True, key_bias=bias)
  dq, dk, dv = (to_np(t) for t in ops.flash_attention_backward(qd, kd, vd, out, dod, lse, key_bias=bias))
  assert np.isfinite(dq).all() and np.isfinite(dk).all() and np.isfinite(dv).all()
  for b in range(B):
    rq, rk, rv = O.attention_bwd(hsd(q[b:b + 1]), hsd(k[b:b + 1]), hsd(v[b:b + 1]), hsd(do[b:b + 1]), D**-0.5, kv_mask=keep[b])
    assert not dk[b][~keep[b]].any() and not dv[b][~keep[b]].any()
    if not keep[b].any():
      assert not dq[b].any()
      continue
    _check(hsd(dq[b:b + 1]), rq, f"masked {kind} D={D} dq b{b}")
    _check(hsd(dk[b:b + 1]), rk, f"masked {kind} D={D} dk b{b}")
    _check(hsd(dv[b:b + 1]), rv, f"masked {kind} D={D} dv b{b}")


def test_backward_seeded_sweep_of_shapes_layouts_masks_and_scale_kinds(dev):
  """Thirty seeded draws of (batch, heads, Sq, Skv, head dim, layout, sharpness, key mask or not, scale carried by q or
  not) against torch's f32 autograd on the GPU (test harness only)."""
  import math
  import random
  rnd = random.Random(21)
  gen = torch.Generator(device=dev).manual_seed(21)
  for it in range(30):
    B, H, D = rnd.choice([1, 1, 2]), rnd.choice([1, 2, 3, 5]), rnd.choice([128, 128, 64])
    sq = rnd.choice([1, 7, 31, 32, 33, 64, 100, 127, 128, 129, 255, 256, 257, 300, 513, 1000])
    skv = rnd.choice([1, 2, 5, 31, 32, 33, 63, 64, 65, 100, 127, 128, 129, 500, 1023, 1025, 2100])
    layout, mult = rnd.choice(["bshd", "bhsd"]), rnd.choice([1.0, 1.0, 2.0, 4.0])
    masked, folded = rnd.random() < 0.4, rnd.random() < 0.4
    q, k, v, do = ((torch.randn((B, s_, H, D), generator=gen, device=dev) * m).to(torch.bfloat16)
                   for s_, m in ((sq, mult), (skv, 1.0), (skv, 1.0), (sq, 1.0)))
    scale = D**-0.5
    if folded and not masked:
      q = (q.float() * (scale * math.log2(math.e))).to(torch.bfloat16)
      scale = math.log(2.0)
    keep = None
    if masked:
      keep = torch.rand((B, skv), generator=gen, device=dev) < 0.7
      keep[:, rnd.randrange(skv)] = True  # every batch element keeps a key
    if layout == "bhsd":
      q, k, v = (t.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3) for t in (q, k, v))
    bias = ops.key_mask_bias(keep) if masked else None
    out, lse = ops.flash_attention(q, k, v, scale=scale, return_lse=True, out_layout=layout, key_bias=bias)
    dq, dk, dv = ops.flash_attention_backward(q, k, v, out, do, lse, scale=scale, key_bias=bias)
    tq, tk, tv = (x.float().permute(0, 2, 1, 3).detach().requires_grad_(True) for x in (q, k, v))  # [B,H,S,D]
    s = (tq @ tk.transpose(2, 3)) * scale
    if masked:
      s = s.masked_fill(~keep[:, None, None, :], float("-inf"))
    (torch.softmax(s, dim=-1) @ tv).backward(do.float().permute(0, 2, 1, 3))
    what = f"draw {it}: B={B} H={H} D={D} Sq={sq} Skv={skv} {layout} x{mult} masked={masked} folded={folded and not masked}"
    for name, got, t in (("dq", dq, tq), ("dk", dk, tk), ("dv", dv, tv)):
      g, r = got.float(), t.grad.permute(0, 2, 1, 3)
      assert bool(torch.isfinite(g).all()), f"{what} {name}"
      den = float(r.norm())
      if den < 1e-6:  # one key: the exact gradient is zero (see _check)
        assert float(g.abs().max()) <= 0.25, f"{what} {name}"
        continue
      rel, mx = float((g - r).norm()) / den, float((g - r).abs().max() / r.abs().max())
      # sharper logits (x2, x4) put more weight on fewer probabilities: the bf16 rounding of P and dS weighs more
      assert rel <= (6e-3 if mult == 1.0 else 1e-2) and mx <= (1.5e-2 if mult == 1.0 else 3e-2), f"{what} {name}: rel-l2 {rel:.2e} max {mx:.2e}"


@pytest.mark.parametrize("D", [128, 64])
def test_backward_over_kv_chunks_with_the_merged_lse(dev, D):
  """The backward of a ring / chunked forward: every KV chunk is differentiated against the MERGED (out, lse) of the
  whole key range; dq is the sum over the chunks and each chunk's dk / dv are the slices of the unsplit gradients
  (the reference's ring backward does exactly this, kernels/splash_attention/ring_attention_kernel.py:1134-1230)."""
  B, H, Sq, Skv = 2, 3, 200, 333
  cuts = [0, 96, 231, Skv]  # ragged chunks
  q, do = (to_dev_bf16(O.normal_bf16((B, Sq, H, D), s), dev) for s in (0, 3))
  k, v = (to_dev_bf16(O.normal_bf16((B, Skv, H, D), s), dev) for s in (1, 2))
  scale = D**-0.5
  # forward chunk by chunk through the fused merge, as a ring does
  o_run, l_run = ops.new_merge_state(B, Sq, H, D, dev)
  for a, b in zip(cuts[:-1], cuts[1:]):
    ops.flash_attention_merge(q, k[:, a:b], v[:, a:b], o_run, l_run, scale=scale)
  out = ops.finalize(o_run)
  out1, lse1 = ops.flash_attention(q, k, v, scale=scale, return_lse=True)
  assert float((l_run - lse1).abs().max()) <= 1e-3
  dq1, dk1, dv1 = ops.flash_attention_backward(q, k, v, out1, do, lse1, scale=scale)
  dq = torch.zeros_like(dq1, dtype=torch.float32)
  dk, dv = torch.empty_like(dk1), torch.empty_like(dv1)
  for a, b in zip(cuts[:-1], cuts[1:]):
    dq_c, dk_c, dv_c = ops.flash_attention_backward(q, k[:, a:b].contiguous(), v[:, a:b].contiguous(), out, do, l_run, scale=scale)
    dq += dq_c.float()
    dk[:, a:b], dv[:, a:b] = dk_c, dv_c
  for got, want, name in ((dq, dq1, "dq"), (dk, dk1, "dk"), (dv, dv1, "dv")):
    rl = rel_l2(to_np(got.to(torch.bfloat16)), to_np(want))
    print(f"D={D} {name}: chunked vs unsplit rel-l2 {rl:.3e}", flush=True)
    assert rl <= 1e-2, name  # bf16 roundings of the merged out and of the partial dq
