"""Seeded synthetic inputs for the five benchmark configurations (test infrastructure).

Values are N(0,1) rounded to bf16, norm weights 1 + 0.1*N(0,1) rounded to bf16, drawn
from numpy's default_rng with seeds q=0, k=1, v=2, wq=3, wk=4 (the reference's own
kernel tests seed q/k/v with PRNGKey(0/1/2), tests/custom_splash_fixed_m_test.py:55-57).
"""
from __future__ import annotations

import dataclasses

import numpy as np

from .dit_attention import bf16_round

__all__ = ["Workload", "WORKLOADS", "normal_bf16", "norm_weight", "attention_flops", "normrope_bytes", "sample_rows"]

SEED_Q, SEED_K, SEED_V, SEED_WQ, SEED_WK = 0, 1, 2, 3, 4


@dataclasses.dataclass(frozen=True)
class Workload:
  name: str
  heads: int
  head_dim: int
  seq: int  # query tokens
  kv_seq: int  # key/value tokens of the self-attention
  norm: str  # "fullrow" (Wan) | "perhead" (Flux) | "rows" (LTX-2)
  rope: str  # "wan" | "flux" | "ltx2"
  grid: tuple  # wan: (ppf, pph, ppw); flux: (n_txt, rows, cols)
  cross_kv: int = 0  # text tokens of the cross-attention that follows (0: none)
  ring_chunks: int = 0  # >0: Q chunk of `seq` tokens against this many KV chunks of `kv_seq`

  @property
  def scale(self) -> float:
    return float(self.head_dim) ** -0.5


WORKLOADS = {
    # the five benchmark configurations: Wan-1.3B, Flux-dev, Wan-14B (self + 512-key cross), its ring shard, its fp8 form
    "wan1.3b": Workload("wan1.3b", 12, 128, 4680, 4680, "fullrow", "wan", (3, 30, 52)),
    "flux-dev": Workload("flux-dev", 24, 128, 4608, 4608, "perhead", "flux", (512, 64, 64)),
    "wan14b": Workload("wan14b", 40, 128, 75600, 75600, "fullrow", "wan", (21, 45, 80), cross_kv=512),
    "wan14b-ring": Workload("wan14b-ring", 40, 128, 9450, 9450, "fullrow", "wan", (21, 45, 80), ring_chunks=8),
    "wan14b-fp8": Workload("wan14b-fp8", 40, 128, 75600, 75600, "fullrow", "wan", (21, 45, 80)),
    # single-GPU replays of the other context-parallel shards of configs[2] (attention_flax.py:875-986, :1305-1315):
    # pure Ulysses over 8 GPUs = 5 heads at the full sequence; Ulysses 2 x ring 4 = 20 heads, a Q chunk of 18,900
    # tokens against 4 KV chunks of 18,900
    "wan14b-ulysses": Workload("wan14b-ulysses", 5, 128, 75600, 75600, "fullrow", "wan", (21, 45, 80)),
    "wan14b-usp": Workload("wan14b-usp", 20, 128, 18900, 18900, "fullrow", "wan", (21, 45, 80), ring_chunks=4),
    # LTX-2 shapes (models/ltx2/transformer_ltx2.py:788-789): 32 heads, head dim 128 for the video stream and 64 for
    # the audio stream; full-row RMSNorm with f32 weights, interleaved RoPE with per-batch, per-head f32 tables
    "ltx2-video": Workload("ltx2-video", 32, 128, 13376, 13376, "rows", "ltx2", ()),
    "ltx2-audio": Workload("ltx2-audio", 32, 64, 13376, 13376, "rows", "ltx2", ()),
}


def normal_bf16(shape, seed: int, chunk_rows: int = 1 << 16) -> np.ndarray:
  """N(0,1) rounded to bf16 (float32 storage)."""
  rng = np.random.default_rng(seed)
  return bf16_round(rng.standard_normal(shape, dtype=np.float32))


def norm_weight(n: int, seed: int) -> np.ndarray:
  rng = np.random.default_rng(seed)
  return bf16_round(1.0 + 0.1 * rng.standard_normal(n, dtype=np.float32))


def attention_flops(batch: int, heads: int, sq: int, skv: int, d: int) -> float:
  """4*B*H*Sq*Skv*D: QK^T and PV at 2 FLOP per MAC (the convention of max_utils.py:880-887)."""
  return 4.0 * batch * heads * sq * skv * d


def normrope_bytes(batch: int, seq: int, heads: int, d: int, with_table: bool = True, per_element_table: bool = False) -> float:
  """Q and K each read once and written once in bf16, + weights, + the f32 cos/sin table ([S, D/2] shared by the
  heads, or, per_element_table, LTX-2's interleaved form: cos and sin of the size of the tensor, for q and for k)."""
  if per_element_table:
    return (8.0 + 16.0) * batch * seq * heads * d + 2 * heads * d * 4
  b = 8.0 * batch * seq * heads * d + 2 * heads * d * 2
  if with_table:
    b += seq * (d // 2) * 8
  return b


def sample_rows(seq: int, n_random: int = 200, seed: int = 7, tile: int = 128) -> np.ndarray:
  """Deterministic sample of query rows: first rows, tile-boundary rows, the ragged tail,
  and `n_random` uniformly drawn rows."""
  fixed = [0, 1, 31, 32, 63, 64, tile - 1, tile, 2 * tile - 1, 2 * tile, seq // 2]
  tail = list(range(max(seq - 17, 0), seq))
  rng = np.random.default_rng(seed)
  rnd = rng.integers(0, seq, size=n_random).tolist()
  rows = sorted({r for r in fixed + tail + rnd if 0 <= r < seq})
  return np.asarray(rows, dtype=np.int64)
