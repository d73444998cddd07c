"""Writes the committed golden vectors (inputs + expected outputs) for the hot path.

    python tests/golden/make_golden.py

Every expected output comes from the numpy oracle in float64 (oracle/dit_attention.py), whose
functions are pinned by tests/test_oracle.py; inputs are bf16 bit patterns.  The reference
(JAX) cannot be imported in this image, so no vector here was produced by running it.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import oracle as O  # noqa: E402


def bits(x):
  return O.to_bf16_bits(x)


def main():
  # Wan-flavour prologue: grid 3x4x4 (the HF parity grid), 4 heads x 128
  grid, H, D = (3, 4, 4), 4, 128
  S = 3 * 4 * 4
  q = O.normal_bf16((1, S, H * D), 0)
  k = O.normal_bf16((1, S, H * D), 1)
  wq, wk = O.norm_weight(H * D, 3), O.norm_weight(H * D, 4)
  cos, sin = O.wan_rope_table(grid, D)
  np.savez_compressed(
      os.path.join(HERE, "norm_rope_wan.npz"), q=bits(q), k=bits(k), wq=bits(wq), wk=bits(wk), cos=cos, sin=sin, heads=H,
      q_out=O.norm_rope_fullrow(q, wq, cos, sin, H).astype(np.float32),
      k_out=O.norm_rope_fullrow(k, wk, cos, sin, H).astype(np.float32),
      q_norm_only=O.norm_rope_fullrow(q, wq, None, None, H).astype(np.float32))

  # Flux-flavour prologue: 5 text tokens + 4x6 image tokens, 3 heads x 128, separate text weights
  ids = O.flux_ids(5, 4, 6)
  L = ids.shape[0]
  q = O.normal_bf16((1, L, 3, 128), 0)
  k = O.normal_bf16((1, L, 3, 128), 1)
  wq, wk, wqt, wkt = (O.norm_weight(128, s) for s in (3, 4, 5, 6))
  cos, sin = O.flux_rope_table(ids)
  np.savez_compressed(
      os.path.join(HERE, "norm_rope_flux.npz"), q=bits(q), k=bits(k), wq=bits(wq), wk=bits(wk), wq_txt=bits(wqt), wk_txt=bits(wkt),
      cos=cos, sin=sin, n_txt=5,
      q_out=O.norm_rope_perhead(q, wq, cos, sin, w_txt=wqt, n_txt=5).astype(np.float32),
      k_out=O.norm_rope_perhead(k, wk, cos, sin, w_txt=wkt, n_txt=5).astype(np.float32))

  # attention + lse: ragged Sq and Skv (neither a multiple of 32 or 64), 2 heads; plus a sharpened case
  q = O.normal_bf16((1, 70, 2, 128), 0)
  k = O.normal_bf16((1, 100, 2, 128), 1)
  v = O.normal_bf16((1, 100, 2, 128), 2)
  out, lse = O.attention(q[0].transpose(1, 0, 2), k[0].transpose(1, 0, 2), v[0].transpose(1, 0, 2), 128**-0.5)
  qs = O.bf16_round(q * 6.0)
  outs, lses = O.attention(qs[0].transpose(1, 0, 2), k[0].transpose(1, 0, 2), v[0].transpose(1, 0, 2), 128**-0.5)
  np.savez_compressed(
      os.path.join(HERE, "attention_small.npz"), q=bits(q), k=bits(k), v=bits(v), scale=128**-0.5,
      out=out.transpose(1, 0, 2)[None].astype(np.float32), lse=lse[None].astype(np.float32),
      q_sharp=bits(qs), out_sharp=outs.transpose(1, 0, 2)[None].astype(np.float32), lse_sharp=lses[None].astype(np.float32))

  # merge: three unequal KV chunks of the same attention problem
  splits = [0, 37, 38, 100]
  parts_o, parts_l = [], []
  for a, b in zip(splits[:-1], splits[1:]):
    o, l = O.attention(q[0].transpose(1, 0, 2), k[0, a:b].transpose(1, 0, 2), v[0, a:b].transpose(1, 0, 2), 128**-0.5)
    parts_o.append(O.bf16_round(o.transpose(1, 0, 2)[None]))  # partials as the kernel hands them over: bf16
    parts_l.append(l[None].astype(np.float32))
  o_run = np.zeros((1, 70, 2, 128))
  l_run = np.full((1, 2, 70), O.LSE_INIT)
  for o, l in zip(parts_o, parts_l):
    o_t, l_run = O.merge_lse(o_run.transpose(0, 2, 1, 3), l_run, o.transpose(0, 2, 1, 3), l)
    o_run = o_t.transpose(0, 2, 1, 3)
  np.savez_compressed(
      os.path.join(HERE, "merge_small.npz"), parts_o=np.stack([bits(o) for o in parts_o]), parts_l=np.stack(parts_l),
      o_merged=o_run.astype(np.float32), lse_merged=l_run.astype(np.float32))
  for f in sorted(os.listdir(HERE)):
    if f.endswith(".npz"):
      print(f, os.path.getsize(os.path.join(HERE, f)))

  # LTX-2 prologue: 2 batches x 9 tokens, 4 heads x 64, both rotation forms (tables as LTX2RotaryPosEmbed shapes them)
  rng = np.random.default_rng(40)
  B, S, H, D = 2, 9, 4, 64
  x = O.normal_bf16((B, S, H * D), 0)
  w = (1 + 0.1 * rng.standard_normal(H * D)).astype(np.float32)
  ang_i = rng.uniform(-3, 3, (B, S, H * D // 2))
  ang_s = rng.uniform(-3, 3, (B, H, S, D // 2))
  cos_i, sin_i = np.repeat(np.cos(ang_i), 2, -1).astype(np.float32), np.repeat(np.sin(ang_i), 2, -1).astype(np.float32)
  cos_s, sin_s = np.cos(ang_s).astype(np.float32), np.sin(ang_s).astype(np.float32)
  np.savez_compressed(
      os.path.join(HERE, "norm_rope_ltx2.npz"), x=bits(x), w=w, heads=H, cos_i=cos_i, sin_i=sin_i, cos_s=cos_s, sin_s=sin_s,
      out_none=O.norm_rope_ltx2(x, w, None, None, "none").astype(np.float32),
      out_interleaved=O.norm_rope_ltx2(x, w, cos_i, sin_i, "interleaved").astype(np.float32),
      out_split=O.norm_rope_ltx2(x, w, cos_s, sin_s, "split").astype(np.float32))

  # backward: ragged Sq and Skv, 2 heads
  q = O.normal_bf16((1, 45, 2, 128), 0)
  k = O.normal_bf16((1, 70, 2, 128), 1)
  v = O.normal_bf16((1, 70, 2, 128), 2)
  do = O.normal_bf16((1, 45, 2, 128), 3)
  t = lambda a: a[0].transpose(1, 0, 2)
  dq, dk, dv = O.attention_bwd(t(q), t(k), t(v), t(do), 128**-0.5)
  u = lambda a: a.transpose(1, 0, 2)[None].astype(np.float32)
  np.savez_compressed(os.path.join(HERE, "attention_bwd_small.npz"), q=bits(q), k=bits(k), v=bits(v), do=bits(do),
                      scale=128**-0.5, dq=u(dq), dk=u(dk), dv=u(dv))
  prologue_bwd()


def prologue_bwd():
  """Backward of the three prologue forms on the shapes of the forward fixtures (norm_rope_wan/flux/ltx2.npz)."""
  grid, H, D = (3, 4, 4), 4, 128
  S = 3 * 4 * 4
  q, k = O.normal_bf16((1, S, H * D), 0), O.normal_bf16((1, S, H * D), 1)
  wq, wk = O.norm_weight(H * D, 3), O.norm_weight(H * D, 4)
  gq, gk = O.normal_bf16((1, S, H, D), 7), O.normal_bf16((1, S, H, D), 8)
  bias = O.bf16_round(0.5 * O.normal_bf16((2 * H * D,), 9))
  cos, sin = O.wan_rope_table(grid, D)
  f = lambda a: a.astype(np.float32)
  dq, dwq = O.norm_rope_fullrow_bwd(q, wq, cos, sin, H, gq, q_mul=0.125)
  dk, dwk = O.norm_rope_fullrow_bwd(k, wk, cos, sin, H, gk)
  dqb, dwqb = O.norm_rope_fullrow_bwd(q, wq, cos, sin, H, gq, q_mul=0.125, bias=bias[:H * D])
  dkb, dwkb = O.norm_rope_fullrow_bwd(k, wk, cos, sin, H, gk, bias=bias[H * D:])
  dqn, dwqn = O.norm_rope_fullrow_bwd(q, wq, None, None, H, gq)
  wan = dict(q=bits(q), k=bits(k), wq=bits(wq), wk=bits(wk), gq=bits(gq), gk=bits(gk), bias=bits(bias), cos=cos, sin=sin, heads=H,
             q_mul=0.125, dq=f(dq), dk=f(dk), dwq=f(dwq), dwk=f(dwk), dq_bias=f(dqb), dk_bias=f(dkb), dwq_bias=f(dwqb),
             dwk_bias=f(dwkb), dq_norm_only=f(dqn), dwq_norm_only=f(dwqn))

  ids = O.flux_ids(5, 4, 6)
  L = ids.shape[0]
  q, k = O.normal_bf16((1, L, 3, 128), 0), O.normal_bf16((1, L, 3, 128), 1)
  gq, gk = O.normal_bf16((1, L, 3, 128), 7), O.normal_bf16((1, L, 3, 128), 8)
  wq, wk, wqt, wkt = (O.norm_weight(128, s) for s in (3, 4, 5, 6))
  cos, sin = O.flux_rope_table(ids)
  dq, dwq, dwqt = O.norm_rope_perhead_bwd(q, wq, cos, sin, gq, q_mul=0.125, w_txt=wqt, n_txt=5)
  dk, dwk, dwkt = O.norm_rope_perhead_bwd(k, wk, cos, sin, gk, w_txt=wkt, n_txt=5)
  flux = dict(q=bits(q), k=bits(k), gq=bits(gq), gk=bits(gk), wq=bits(wq), wk=bits(wk), wq_txt=bits(wqt), wk_txt=bits(wkt), cos=cos,
              sin=sin, n_txt=5, q_mul=0.125, dq=f(dq), dk=f(dk), dwq=f(dwq), dwk=f(dwk), dwq_txt=f(dwqt), dwk_txt=f(dwkt))

  rng = np.random.default_rng(40)
  B, S, H, D = 2, 9, 4, 64
  x = O.normal_bf16((B, S, H * D), 0)
  g = O.normal_bf16((B, S, H, D), 7)
  w = (1 + 0.1 * rng.standard_normal(H * D)).astype(np.float32)
  # general full-size tables: the two members of a pair carry different values
  cos_i, sin_i = (rng.uniform(-1, 1, (B, S, H * D)).astype(np.float32) for _ in range(2))
  cos_s, sin_s = (rng.uniform(-1, 1, (B, H, S, D // 2)).astype(np.float32) for _ in range(2))
  ltx = dict(x=bits(x), g=bits(g), w=w, heads=H, cos_i=cos_i, sin_i=sin_i, cos_s=cos_s, sin_s=sin_s)
  for mode, c_, s_ in (("none", None, None), ("interleaved", cos_i, sin_i), ("split", cos_s, sin_s)):
    dx, dw = O.norm_rope_ltx2_bwd(x, w, c_, s_, mode, g.reshape(B, S, H * D))
    ltx["dx_" + mode], ltx["dw_" + mode] = f(dx), f(dw)
  np.savez_compressed(os.path.join(HERE, "norm_rope_bwd.npz"), **{"wan_" + k_: v for k_, v in wan.items()},
                      **{"flux_" + k_: v for k_, v in flux.items()}, **{"ltx2_" + k_: v for k_, v in ltx.items()})


if __name__ == "__main__":
  if len(sys.argv) > 1 and sys.argv[1] == "prologue_bwd":
    prologue_bwd()
  else:
    main()
