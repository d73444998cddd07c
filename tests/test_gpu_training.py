"""Training reaches the HIP kernels: loss = sum(apply_attention(hip_norm_rope(...)) * g) differentiated by torch autograd
end to end -- prologue backward, attention backward -- against an f64 autograd reference built from library routines
(torch.nn.functional.rms_norm, a complex-multiply rotation, scaled_dot_product_attention) on the CPU.

The reference's trainer differentiates straight through `apply_attention` and the inline norm + rope
(trainers/wan_trainer.py:169, models/attention_flax.py:2655-2677); here the registry entry `hip_flash` and the prologue
hooks carry their own backward.  Bars: every tensor on the HIP path is bf16 between kernels (q, k, out, dq, dk, dx), so
gradients are held to rel-L2 <= 1e-2 and cosine >= 0.9999 of the f64 reference (measured: 3e-3 .. 4.5e-3)."""
import numpy as np
import pytest
import torch

import oracle as O
from helpers import cosine, rel_l2, to_dev_bf16
from maxdiffusion_amd import attention_op as A
from maxdiffusion_amd import ops

pytestmark = pytest.mark.gpu


def _leaf(x, dev, dtype=torch.bfloat16):
  t = to_dev_bf16(x, dev) if dtype == torch.bfloat16 else torch.from_numpy(x).to(dev)
  return t.requires_grad_(True)


def _rope_complex(y, cos, sin):
  yc = torch.view_as_complex(y.reshape(*y.shape[:-1], -1, 2))
  rot = torch.complex(torch.tensor(cos, dtype=torch.float64), torch.tensor(sin, dtype=torch.float64))[None, :, None, :]
  return torch.view_as_real(yc * rot).reshape(y.shape)


def _check(got, ref, what):
  g, r = got.detach().float().cpu().numpy(), ref.detach().numpy()
  rl, cs = rel_l2(g, r), cosine(g, r)
  print(f"{what}: rel-l2 {rl:.3e} cosine {cs:.6f}", flush=True)
  assert rl <= 1e-2 and cs >= 0.9999, what


@pytest.mark.parametrize("rank4,masked", [(True, False), (False, True)])
def test_wan_prologue_and_attention_end_to_end(dev, rank4, masked):
  B, H, D, grid = 2, 3, 128, (2, 5, 9)
  S, N = grid[0] * grid[1] * grid[2], 3 * 128
  scale = D**-0.5
  xq, xk, xv = O.normal_bf16((B, S, N), 0), O.normal_bf16((B, S, N), 1), O.normal_bf16((B, S, N), 2)
  wq, wk = O.norm_weight(N, 3), O.norm_weight(N, 4)
  g = O.normal_bf16((B, S, N), 5)
  cos, sin = O.wan_rope_table(grid, D)
  keep = np.ones((B, S), bool)
  if masked:
    keep[0, 40:] = False
    keep[1, ::3] = False

  q, k, v, tq, tk = (_leaf(x, dev) for x in (xq, xk, xv, wq, wk))
  freqs = torch.complex(torch.from_numpy(cos), torch.from_numpy(sin)).to(dev)[None, None]  # as WanRotaryPosEmbed returns it
  qn, kn = A.hip_norm_rope(q, k, tq, tk, freqs, H, out_layout="bhsd" if rank4 else "bshd")
  assert qn.requires_grad and kn.requires_grad
  op = A.AttentionOp(attention_kernel="hip_flash", scale=scale, heads=H, dim_head=D, residual_checkpoint_name="attn_out")
  if rank4:  # FlaxWanAttention hands [B,H,S,D] (attention_flax.py:2673-2677)
    out = op.apply_attention(qn.permute(0, 2, 1, 3), kn.permute(0, 2, 1, 3), v.view(B, S, H, D).permute(0, 2, 1, 3))
  else:
    out = op.apply_attention(qn.reshape(B, S, N), kn.reshape(B, S, N), v, attention_mask=torch.from_numpy(keep).to(dev) if masked else None)
  assert out.shape == (B, S, N) and out.requires_grad
  (out.float() * to_dev_bf16(g, dev).float()).sum().backward()

  rq, rk, rv, rwq, rwk = (torch.tensor(x, dtype=torch.float64, requires_grad=True) for x in (xq, xk, xv, wq, wk))
  yq = _rope_complex(torch.nn.functional.rms_norm(rq, (N,), rwq, eps=1e-6).reshape(B, S, H, D), cos, sin).transpose(1, 2)
  yk = _rope_complex(torch.nn.functional.rms_norm(rk, (N,), rwk, eps=1e-6).reshape(B, S, H, D), cos, sin).transpose(1, 2)
  am = torch.from_numpy(keep)[:, None, None, :] if (masked and not rank4) else None
  ro = torch.nn.functional.scaled_dot_product_attention(yq, yk, rv.reshape(B, S, H, D).transpose(1, 2), attn_mask=am, scale=scale)
  (ro.transpose(1, 2).reshape(B, S, N) * torch.tensor(g, dtype=torch.float64)).sum().backward()
  _check(out, ro.transpose(1, 2).reshape(B, S, N), "forward")
  for got, ref, name in ((q, rq, "d q_in"), (k, rk, "d k_in"), (v, rv, "d v"), (tq, rwq, "d wq"), (tk, rwk, "d wk")):
    assert got.grad is not None and got.grad.dtype == got.dtype and got.grad.shape == got.shape
    _check(got.grad, ref.grad, name)
  if masked and not rank4:  # masked keys receive no gradient through the attention
    assert not v.grad[0, 40:].any()


@pytest.mark.parametrize("with_bias", [True, False])
def test_fused_projection_prologue_and_attention_end_to_end(dev, with_bias):
  """One fused q|k|v projection output [B,S,3*H*D] (the three Linears of attention_flax.py:2653-2663 as one GEMM, their
  biases added by the prologue): gradients for the fused buffer, the biases and the norm weights."""
  B, H, D, grid = 2, 3, 128, (2, 5, 9)
  S, N = grid[0] * grid[1] * grid[2], 3 * 128
  scale = D**-0.5
  xqkv = O.normal_bf16((B, S, 3 * N), 0)
  xb = (0.5 * O.normal_bf16((3 * N,), 1)).astype(np.float32)
  wq, wk = O.norm_weight(N, 3), O.norm_weight(N, 4)
  g = O.normal_bf16((B, S, N), 5)
  cos, sin = O.wan_rope_table(grid, D)

  qkv, tq, tk = (_leaf(x, dev) for x in (xqkv, wq, wk))
  tb = _leaf(xb, dev) if with_bias else None
  freqs = torch.complex(torch.from_numpy(cos), torch.from_numpy(sin)).to(dev)[None, None]
  qn, kn, vn = A.hip_norm_rope_qkv(qkv, tq, tk, freqs, H, bias=tb)
  assert qn.requires_grad and kn.requires_grad and vn.requires_grad
  op = A.AttentionOp(attention_kernel="hip_flash", scale=scale, heads=H, dim_head=D)
  out = op.apply_attention(qn.permute(0, 2, 1, 3), kn.permute(0, 2, 1, 3), vn.permute(0, 2, 1, 3))
  (out.float() * to_dev_bf16(g, dev).float()).sum().backward()
  with pytest.raises(ValueError, match="inplace"):
    A.hip_norm_rope_qkv(qkv, tq, tk, freqs, H, bias=tb, inplace=True)

  rqkv, rwq, rwk = (torch.tensor(x, dtype=torch.float64, requires_grad=True) for x in (xqkv, wq, wk))
  xb16 = to_dev_bf16(xb, "cpu").double().numpy() if with_bias else np.zeros(3 * N)  # the bias as the kernel sees it: bf16
  rb = torch.tensor(xb16, dtype=torch.float64, requires_grad=True)
  u = rqkv + rb
  yq = _rope_complex(torch.nn.functional.rms_norm(u[..., :N], (N,), rwq, eps=1e-6).reshape(B, S, H, D), cos, sin).transpose(1, 2)
  yk = _rope_complex(torch.nn.functional.rms_norm(u[..., N:2 * N], (N,), rwk, eps=1e-6).reshape(B, S, H, D), cos, sin).transpose(1, 2)
  ro = torch.nn.functional.scaled_dot_product_attention(yq, yk, u[..., 2 * N:].reshape(B, S, H, D).transpose(1, 2), scale=scale)
  ro = ro.transpose(1, 2).reshape(B, S, N)
  (ro * torch.tensor(g, dtype=torch.float64)).sum().backward()
  _check(out, ro, "forward")
  checks = [(qkv, rqkv, "d qkv"), (tq, rwq, "d wq"), (tk, rwk, "d wk")] + ([(tb, rb, "d bias")] if with_bias else [])
  for got, ref, name in checks:
    assert got.grad is not None and got.grad.dtype == got.dtype and got.grad.shape == got.shape
    _check(got.grad, ref.grad, name)
  for blk, name in ((slice(0, N), "q"), (slice(N, 2 * N), "k"), (slice(2 * N, 3 * N), "v")):  # each column block on its own
    _check(qkv.grad[..., blk], rqkv.grad[..., blk], "d qkv block " + name)


def test_flux_prologue_and_attention_end_to_end(dev):
  B, H, D, n_txt = 1, 4, 128, 7
  ids = O.flux_ids(n_txt, 5, 6)
  L = ids.shape[0]
  scale = D**-0.5
  xq, xk, xv = (O.normal_bf16((B, L, H, D), s) for s in (0, 1, 2))
  ws = [O.norm_weight(D, s) for s in (3, 4, 5, 6)]
  g = O.normal_bf16((B, L, H * D), 7)
  cos, sin = O.flux_rope_table(ids)
  q, k, v = (_leaf(x, dev) for x in (xq, xk, xv))
  tw = [_leaf(w, dev) for w in ws]
  qn, kn = A.hip_norm_rope(q, k, tw[0], tw[1], (torch.from_numpy(cos).to(dev), torch.from_numpy(sin).to(dev)), H, per_head=True,
                           wq_txt=tw[2], wk_txt=tw[3], n_txt=n_txt)
  op = A.AttentionOp(attention_kernel="hip_flash", scale=scale, heads=H, dim_head=D)
  out = op.apply_attention(qn.reshape(B, L, H * D), kn.reshape(B, L, H * D), v.reshape(B, L, H * D))
  (out.float() * to_dev_bf16(g, dev).float()).sum().backward()

  rq, rk, rv = (torch.tensor(x, dtype=torch.float64, requires_grad=True) for x in (xq, xk, xv))
  rw = [torch.tensor(w, dtype=torch.float64, requires_grad=True) for w in ws]
  norm = lambda x, w_img, w_txt: torch.cat([torch.nn.functional.rms_norm(x[:, :n_txt], (D,), w_txt, eps=1e-6),
                                            torch.nn.functional.rms_norm(x[:, n_txt:], (D,), w_img, eps=1e-6)], dim=1)
  yq = _rope_complex(norm(rq, rw[0], rw[2]), cos, sin).transpose(1, 2)
  yk = _rope_complex(norm(rk, rw[1], rw[3]), cos, sin).transpose(1, 2)
  ro = torch.nn.functional.scaled_dot_product_attention(yq, yk, rv.transpose(1, 2), scale=scale).transpose(1, 2).reshape(B, L, H * D)
  (ro * torch.tensor(g, dtype=torch.float64)).sum().backward()
  _check(out, ro, "forward")
  for got, ref, name in ((q, rq, "d q"), (k, rk, "d k"), (v, rv, "d v"), (tw[0], rw[0], "d wq"), (tw[1], rw[1], "d wk"),
                         (tw[2], rw[2], "d wq_txt"), (tw[3], rw[3], "d wk_txt")):
    _check(got.grad, ref.grad, name)


@pytest.mark.parametrize("rope_type", ["interleaved", "split"])
def test_ltx2_prologue_and_attention_end_to_end(dev, rope_type):
  """LTX-2: f32 activations and f32 norm weights (attention_ltx2.py:415-432), head dim 64, per-head tables."""
  B, S, H, D = 2, 50, 4, 64
  N = H * D
  scale = D**-0.5
  rng = np.random.default_rng(3)
  xq, xk, xv = (rng.standard_normal((B, S, N)).astype(np.float32) for _ in range(3))
  wq, wk = (1 + 0.1 * rng.standard_normal(N)).astype(np.float32), (1 + 0.1 * rng.standard_normal(N)).astype(np.float32)
  g = O.normal_bf16((B, S, N), 7)
  if rope_type == "interleaved":
    ang = rng.uniform(-3, 3, (B, S, N // 2))
    cos, sin = np.repeat(np.cos(ang), 2, -1).astype(np.float32), np.repeat(np.sin(ang), 2, -1).astype(np.float32)
  else:
    ang = rng.uniform(-3, 3, (B, H, S, D // 2))
    cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
  q, k, v, tq, tk = (_leaf(x, dev, torch.float32) for x in (xq, xk, xv, wq, wk))
  tabs = (torch.from_numpy(cos).to(dev), torch.from_numpy(sin).to(dev))
  qn, kn = A.hip_norm_rope_ltx2(q, k, tq, tk, H, rotary_emb=tabs, rope_type=rope_type)
  op = A.AttentionOp(attention_kernel="hip_flash", scale=scale, heads=H, dim_head=D)
  out = op.apply_attention(qn.reshape(B, S, N), kn.reshape(B, S, N), v)
  assert out.dtype == torch.bfloat16  # q, k come out of the prologue as bf16; v is cast by the registry entry
  (out.float() * to_dev_bf16(g, dev).float()).sum().backward()

  rq, rk, rv, rwq, rwk = (torch.tensor(x, dtype=torch.float64, requires_grad=True) for x in (xq, xk, xv, wq, wk))
  c, s_ = torch.tensor(cos, dtype=torch.float64), torch.tensor(sin, dtype=torch.float64)

  def rot(y):
    if rope_type == "interleaved":
      yr = y.reshape(B, S, N // 2, 2)
      return y * c + torch.stack([-yr[..., 1], yr[..., 0]], dim=-1).reshape(B, S, N) * s_
    yh = y.reshape(B, S, H, 2, D // 2).permute(0, 2, 1, 3, 4)
    a1, a2 = yh[..., 0, :], yh[..., 1, :]
    return torch.stack([a1 * c - a2 * s_, a2 * c + a1 * s_], dim=-2).permute(0, 2, 1, 3, 4).reshape(B, S, N)

  heads_first = lambda t: t.reshape(B, S, H, D).transpose(1, 2)
  yq, yk = rot(torch.nn.functional.rms_norm(rq, (N,), rwq, eps=1e-6)), rot(torch.nn.functional.rms_norm(rk, (N,), rwk, eps=1e-6))
  ro = torch.nn.functional.scaled_dot_product_attention(heads_first(yq), heads_first(yk), heads_first(rv), scale=scale)
  ro = ro.transpose(1, 2).reshape(B, S, N)
  (ro * torch.tensor(g, dtype=torch.float64)).sum().backward()
  _check(out, ro, "forward")
  for got, ref, name in ((q, rq, "d q_in"), (k, rk, "d k_in"), (v, rv, "d v"), (tq, rwq, "d wq"), (tk, rwk, "d wk")):
    assert got.grad.dtype == torch.float32
    _check(got.grad, ref.grad, name)


def test_no_grad_path_is_unchanged(dev):
  """Without autograd recording the registry entry and the hook call the plain operators (no lse, nothing saved)."""
  B, S, H, D = 1, 40, 2, 128
  q, k, v = (to_dev_bf16(O.normal_bf16((B, S, H * D), s), dev) for s in (0, 1, 2))
  op = A.AttentionOp(attention_kernel="hip_flash", scale=D**-0.5, heads=H, dim_head=D)
  plain = op.apply_attention(q, k, v)
  qg = q.clone().requires_grad_(True)
  with torch.no_grad():
    assert not op.apply_attention(qg, k, v).requires_grad
  tracked = op.apply_attention(qg, k, v)
  assert tracked.requires_grad and torch.equal(tracked.detach(), plain)
