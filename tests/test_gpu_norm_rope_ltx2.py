"""LTX-2's attention prologue (full-row RMSNorm with an f32 weight, then the interleaved or the split rotation with
per-batch, per-head tables) through the C ABI, against the CPU oracle.  Same bars as the Wan / Flux prologue."""
import numpy as np
import pytest
import torch

import oracle as O
from helpers import bits_to_dev, err_stats, golden, to_dev_bf16, to_np
from maxdiffusion_amd import attention_op, ops

pytestmark = pytest.mark.gpu
MAX_ABS, MEAN_ABS = 2e-2, 2e-3


def _assert_close(got, ref, what):
  mx, mean = err_stats(got, ref)
  print(f"{what}: max-abs {mx:.3e} mean-abs {mean:.3e}", flush=True)
  assert mx <= 1.6e-2 and mean <= MEAN_ABS, what  # one bf16 rounding of |y| < 8


def _tables(rng, B, S, H, D, mode):
  if mode == "interleaved":  # attention_ltx2.py:292-295: [B,S,H*D], every angle repeated for its pair
    ang = rng.uniform(-3.1, 3.1, (B, S, H * D // 2))
    return np.repeat(np.cos(ang), 2, -1).astype(np.float32), np.repeat(np.sin(ang), 2, -1).astype(np.float32)
  ang = rng.uniform(-3.1, 3.1, (B, H, S, D // 2))  # :323-324
  return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)


@pytest.mark.parametrize("H,D", [(32, 128), (32, 64), (5, 64), (48, 128)])
@pytest.mark.parametrize("mode", ["none", "interleaved", "split"])
@pytest.mark.parametrize("f32_in", [False, True])
def test_rows_against_oracle(dev, H, D, mode, f32_in):
  rng = np.random.default_rng(21)
  B, S = 2, 37
  x = rng.standard_normal((B, S, H * D)).astype(np.float32)
  if not f32_in:
    x = O.bf16_round(x)
  w = (1 + 0.1 * rng.standard_normal(H * D)).astype(np.float32)
  cos = sin = None
  if mode != "none":
    cos, sin = _tables(rng, B, S, H, D, mode)
  ref = O.norm_rope_ltx2(x, w, cos, sin, mode)
  xd = torch.from_numpy(x).to(dev) if f32_in else to_dev_bf16(x, dev)
  t = lambda a: None if a is None else torch.from_numpy(a).to(dev)
  for layout in ("bshd", "bhsd"):
    out = ops.norm_rope_rows(xd, t(w), t(cos), t(sin), heads=H, mode=mode, out_layout=layout)
    assert out.shape == (B, S, H, D) and out.dtype == torch.bfloat16
    _assert_close(to_np(out).reshape(B, S, H * D), ref, f"ltx2 {mode} H={H} D={D} f32_in={f32_in} {layout}")


def test_call_flow_of_the_attention_module(dev):
  # attention_ltx2.py:566-585: q gets rotary_emb; k gets k_rotary_emb, else rotary_emb for self-attention, else nothing
  rng = np.random.default_rng(22)
  B, Sq, Sk, H, D = 1, 20, 12, 4, 64
  q = rng.standard_normal((B, Sq, H * D)).astype(np.float32)
  k_self = rng.standard_normal((B, Sq, H * D)).astype(np.float32)
  k_cross = rng.standard_normal((B, Sk, H * D)).astype(np.float32)
  wq, wk = (1 + 0.1 * rng.standard_normal(H * D)).astype(np.float32), (1 + 0.1 * rng.standard_normal(H * D)).astype(np.float32)
  t = lambda a: torch.from_numpy(a).to(dev)
  for mode in ("interleaved", "split"):
    tab_q, tab_k = _tables(rng, B, Sq, H, D, mode), _tables(rng, B, Sk, H, D, mode)
    emb_q, emb_k = tuple(t(a) for a in tab_q), tuple(t(a) for a in tab_k)
    qo, ko = attention_op.hip_norm_rope_ltx2(t(q), t(k_self), t(wq), t(wk), H, rotary_emb=emb_q, rope_type=mode)
    _assert_close(to_np(qo).reshape(B, Sq, -1), O.norm_rope_ltx2(q, wq, *tab_q, mode), f"{mode} self q")
    _assert_close(to_np(ko).reshape(B, Sq, -1), O.norm_rope_ltx2(k_self, wk, *tab_q, mode), f"{mode} self k")
    qo, ko = attention_op.hip_norm_rope_ltx2(t(q), t(k_cross), t(wq), t(wk), H, rotary_emb=emb_q, rope_type=mode, is_self_attention=False)
    _assert_close(to_np(ko).reshape(B, Sk, -1), O.norm_rope_ltx2(k_cross, wk, None, None, "none"), f"{mode} cross k: norm only")
    qo, ko = attention_op.hip_norm_rope_ltx2(t(q), t(k_cross), t(wq), t(wk), H, rotary_emb=emb_q, k_rotary_emb=emb_k, rope_type=mode,
                                            is_self_attention=False)
    _assert_close(to_np(ko).reshape(B, Sk, -1), O.norm_rope_ltx2(k_cross, wk, *tab_k, mode), f"{mode} cross k with its own table")
    # q_mul (softmax scale carried by the prologue) goes into the f32 query scale: q scaled, k untouched
    m = ops.folded_q_mul(D)
    qo, ko = attention_op.hip_norm_rope_ltx2(t(q), t(k_self), t(wq), t(wk), H, rotary_emb=emb_q, rope_type=mode, q_mul=m)
    _assert_close(to_np(qo).reshape(B, Sq, -1) / m, O.norm_rope_ltx2(q, wq, *tab_q, mode), f"{mode} self q with q_mul")
    _assert_close(to_np(ko).reshape(B, Sq, -1), O.norm_rope_ltx2(k_self, wk, *tab_q, mode), f"{mode} self k with q_mul")
  with pytest.raises(ValueError, match="not supported"):
    attention_op.hip_norm_rope_ltx2(t(q), None, t(wq), t(wk), H, rope_type="rotate_half")


def test_golden_ltx2(dev):
  g = golden("norm_rope_ltx2.npz")
  x, H = bits_to_dev(g["x"], dev), int(g["heads"])
  t = lambda a: torch.from_numpy(a).to(dev)
  B, S, N = x.shape
  for mode, cs in (("none", (None, None)), ("interleaved", (g["cos_i"], g["sin_i"])), ("split", (g["cos_s"], g["sin_s"]))):
    cos, sin = (None if a is None else t(a) for a in cs)
    out = ops.norm_rope_rows(x, t(g["w"]), cos, sin, heads=H, mode=mode)
    _assert_close(to_np(out).reshape(B, S, N), g[f"out_{mode}"], f"ltx2 golden {mode}")
