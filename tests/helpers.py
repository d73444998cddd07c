"""Shared helpers of the GPU parity tests."""
import numpy as np

def to_dev_bf16(x: np.ndarray, device):
  """float32 numpy array holding bf16-representable values -> torch bf16 tensor on `device`."""
  import torch

  import oracle as O

  bits = O.to_bf16_bits(x).view(np.int16)
  return torch.from_numpy(bits).view(torch.bfloat16).to(device)


def to_np(t) -> np.ndarray:
  return t.detach().float().cpu().numpy()


def err_stats(got: np.ndarray, ref: np.ndarray):
  d = np.abs(got.astype(np.float64) - ref.astype(np.float64))
  return float(d.max()), float(d.mean())


def rel_l2(got: np.ndarray, ref: np.ndarray) -> float:
  g = got.astype(np.float64).ravel()
  r = ref.astype(np.float64).ravel()
  return float(np.linalg.norm(g - r) / max(np.linalg.norm(r), 1e-30))


def cosine(got: np.ndarray, ref: np.ndarray) -> float:
  g = got.astype(np.float64).ravel()
  r = ref.astype(np.float64).ravel()
  return float(g @ r / max(np.linalg.norm(g) * np.linalg.norm(r), 1e-30))


def golden(name: str):
  import os

  return np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", name))


def bits_to_dev(b: np.ndarray, device):
  import torch

  return torch.from_numpy(np.ascontiguousarray(b).view(np.int16)).view(torch.bfloat16).to(device)


def bits_to_f32(b: np.ndarray) -> np.ndarray:
  import oracle as O

  return O.from_bf16_bits(b)


def hsd(x_bshd: np.ndarray) -> np.ndarray:
  """[1,S,H,D] -> [H,S,D] for the oracle."""
  return np.ascontiguousarray(x_bshd[0].transpose(1, 0, 2))


def torch_attention_f32(q, k, v, scale, q_block=2048):
  """Plain torch fp32 reference on the GPU (test harness only): q,k,v logical [B,S,H,D] -> out f32, lse f32."""
  import torch

  b, sq, h, d = q.shape
  out = torch.empty((b, sq, h, d), dtype=torch.float32, device=q.device)
  lse = torch.empty((b, h, sq), dtype=torch.float32, device=q.device)
  kf = k.permute(0, 2, 3, 1).float()  # [B,H,D,Skv]
  vf = v.permute(0, 2, 1, 3).float()  # [B,H,Skv,D]
  for s0 in range(0, sq, q_block):
    qb = q[:, s0:s0 + q_block].permute(0, 2, 1, 3).float()  # [B,H,bq,D]
    s = torch.matmul(qb, kf) * scale
    l = torch.logsumexp(s, dim=-1)
    p = torch.exp(s - l[..., None])
    out[:, s0:s0 + q_block] = torch.matmul(p, vf).permute(0, 2, 1, 3)
    lse[:, :, s0:s0 + q_block] = l
  return out, lse


def structured_logits(sq, skv, d, profile, seed=5):
  """q, k such that the logit of (row, key j) is gain[row] * beta[j] * 4 (natural units) plus small noise:
  the shape of beta along the key axis decides when and how often a row's reference point has to move."""
  import oracle as O

  rng = np.random.default_rng(seed)
  u = np.ones(d, np.float32)
  t = np.arange(skv, dtype=np.float32) / max(skv - 1, 1)
  beta = {
      "ascending": 2 * t - 1,                                   # the maximum grows with every tile
      "descending": 1 - 2 * t,                                  # the first key is the maximum
      "plateau": np.where(t < 0.5, 0.0, 0.3).astype(np.float32),  # many keys a little above the reference
      "late_spike": np.where(np.arange(skv) == (skv * 3) // 4, 3.0, -0.2 * t).astype(np.float32),
  }[profile]
  gain = np.array([0.25, 0.5, 1.0, 2.0, 4.0, 8.0], np.float32)[np.arange(sq) % 6]
  amp = np.float32(4.0 / (d * d**-0.5))                         # scale * <u, u> * amp == 4
  q = O.bf16_round(gain[:, None] * u[None] * amp + 0.05 * rng.standard_normal((sq, d)).astype(np.float32))
  k = O.bf16_round(beta[:, None] * u[None] + 0.05 * rng.standard_normal((skv, d)).astype(np.float32))
  return q, k
