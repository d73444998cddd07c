"""Host-side operators of the DiT attention hot path (torch tensors in HBM -> libmdattn.so).

torch is used for device memory and the current HIP stream only; every computation below is
a hand-written HIP kernel reached through the C ABI.  Tensors are logical [B, S, H, D] views
(any strides, D contiguous), so a [B, H, S, D] buffer is passed as ``x.permute(0, 2, 1, 3)``
and the reference's rank-3 [B, S, H*D] as ``x.view(B, S, H, D)`` -- never copied.
"""
from __future__ import annotations

import ctypes
import math

import torch

from . import _lib
from ._lib import Strides

__all__ = [
    "norm_rope_fullrow", "norm_rope_qkv", "norm_rope_perhead", "norm_rope_rows",
    "norm_rope_fullrow_backward", "norm_rope_perhead_backward", "norm_rope_rows_backward", "flash_attention", "flash_attention_backward", "flash_attention_backward_static", "flash_attention_fp8", "quant_e4m3", "key_mask_bias",
    "merge_partial", "flash_attention_merge", "finalize", "new_merge_state", "LSE_INIT", "FOLDED_SCALE", "folded_q_mul", "set_fwd_schedule", "FWD_SCHEDULES", "FP8_SOFTMAX_MODES",
]

LSE_INIT = -1e30

FWD_SCHEDULES = {"auto": 0, "pipelined8": 1, "pipelined4": 2, "flat": 3}


def set_fwd_schedule(schedule) -> int:
  """Test and tuning hook: forces the schedule of the bf16 forward at head dim 128 for the whole process ("auto"
  restores the choice by shape).  Returns the previous setting."""
  rc = _lib.load().mdattn_set_fwd_schedule(FWD_SCHEDULES.get(schedule, schedule))
  if rc < 0:
    _lib.check(rc, "mdattn_set_fwd_schedule")
  return rc

# Folding the softmax scale into the prologue: norm_rope_*(..., q_mul=folded_q_mul(D)) emits q * D^-1/2 * log2(e)
# (still one rounding), and the attention entry points, given scale=FOLDED_SCALE = ln 2, see scale * log2(e) == 1:
# their logits come out of the MFMA in log2 units and need no multiply.  Results are those of scale = D^-1/2.
FOLDED_SCALE = math.log(2.0)


def folded_q_mul(head_dim: int, scale: float | None = None) -> float:
  return (head_dim**-0.5 if scale is None else scale) * math.log2(math.e)


def _ptr(t):
  return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _stream():
  return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _check_dev(*ts):
  for t in ts:
    if t is not None and not t.is_cuda:
      raise ValueError("mdattn operators need tensors in device memory (cuda/HIP); there is no CPU path")


def _strides(t: torch.Tensor) -> Strides:
  if t.dim() != 4 or t.stride(3) != 1:
    raise ValueError(f"expected a [B,S,H,D] view with contiguous D, got shape {tuple(t.shape)} strides {t.stride()}")
  return Strides(t.stride(0), t.stride(1), t.stride(2))


def _alloc_like_layout(b, s, h, d, layout: str, dtype, device):
  """Returns a logical [B,S,H,D] view over a fresh buffer laid out as `layout`."""
  if layout == "bshd":
    return torch.empty((b, s, h, d), dtype=dtype, device=device)
  if layout == "bhsd":
    return torch.empty((b, h, s, d), dtype=dtype, device=device).permute(0, 2, 1, 3)
  raise ValueError(f"unknown layout {layout!r} (want 'bshd' or 'bhsd')")


def _table(t, s, d, name):
  if t is None:
    return None
  if t.dtype != torch.float32 or tuple(t.shape) != (s, d // 2) or not t.is_contiguous():
    raise ValueError(f"{name} must be a contiguous float32 [S, D/2] = [{s}, {d // 2}] tensor, got {tuple(t.shape)} {t.dtype}")
  return t


def norm_rope_fullrow(q, k, wq, wk, cos, sin, heads: int, eps: float = 1e-6, out_layout: str = "bshd", q_mul: float = 1.0):
  """q, k: bf16 [B, S, H*D] (k may be None) -> (q_out, k_out) logical [B,S,H,D] views in `out_layout`.

  RMSNorm over H*D, then rotation of interleaved pairs by the [S, D/2] table (cos/sin None: norm only).
  `q_mul` is multiplied into q_out before its single rounding (see FOLDED_Q_MUL / FOLDED_SCALE).
  """
  _check_dev(q, k, wq, wk, cos, sin)
  if q.dim() != 3 or q.dtype != torch.bfloat16 or q.stride(2) != 1:
    raise ValueError("q must be bf16 [B, S, H*D] with a contiguous last axis")
  b, s, n = q.shape
  if n % heads:
    raise ValueError(f"inner dim {n} is not divisible by heads={heads}")
  d = n // heads
  if k is not None and (k.shape != q.shape or k.dtype != q.dtype or k.stride() != q.stride()):
    raise ValueError("k must match q in shape, dtype and strides")
  cos, sin = _table(cos, s, d, "cos"), _table(sin, s, d, "sin")
  q_out = _alloc_like_layout(b, s, heads, d, out_layout, torch.bfloat16, q.device)
  k_out = _alloc_like_layout(b, s, heads, d, out_layout, torch.bfloat16, q.device) if k is not None else None
  st = _strides(q_out)
  rc = _lib.load().mdattn_norm_rope_fullrow(
      _stream(), _ptr(q), _ptr(k), _ptr(q_out), _ptr(k_out), _ptr(wq), _ptr(wk), _ptr(cos), _ptr(sin),
      b, s, heads, d, eps, q_mul, q.stride(0), q.stride(1), ctypes.byref(st))
  _lib.check(rc, "mdattn_norm_rope_fullrow")
  return q_out, k_out


def norm_rope_qkv(qkv, wq, wk, cos, sin, heads: int, bias=None, eps: float = 1e-6, out_layout: str = "bshd", q_mul: float = 1.0,
                  inplace: bool = False):
  """The prologue over the output of one fused q|k|v projection: qkv bf16 [B, S, 3*H*D] (column blocks q | k | v).

  bias bf16 [3*H*D] or None: the projections' biases, added in f32 before the statistics.  Returns (q, k, v) logical
  [B,S,H,D] views.  Without bias v is a view of the fused buffer itself (never copied).  inplace=True writes q, k
  (and the biased v) back into the fused buffer, which then holds the three attention operands."""
  _check_dev(qkv, wq, wk, cos, sin, bias)
  if qkv.dim() != 3 or qkv.dtype != torch.bfloat16 or qkv.stride(2) != 1 or qkv.shape[2] % (3 * heads):
    raise ValueError("qkv must be bf16 [B, S, 3*H*D] with a contiguous last axis")
  b, s, n3 = qkv.shape
  n = n3 // 3
  d = n // heads
  cos, sin = _table(cos, s, d, "cos"), _table(sin, s, d, "sin")
  if bias is not None and (bias.dtype != torch.bfloat16 or bias.numel() != n3 or not bias.is_contiguous()):
    raise ValueError("bias must be a contiguous bf16 [3*H*D] tensor")
  blocks = [qkv[:, :, i * n:(i + 1) * n].unflatten(2, (heads, d)) for i in range(3)]  # views of the fused buffer
  if inplace:
    q_out, k_out = blocks[0], blocks[1]
    v_out = blocks[2] if bias is not None else None
  else:
    q_out = _alloc_like_layout(b, s, heads, d, out_layout, torch.bfloat16, qkv.device)
    k_out = _alloc_like_layout(b, s, heads, d, out_layout, torch.bfloat16, qkv.device)
    v_out = _alloc_like_layout(b, s, heads, d, out_layout, torch.bfloat16, qkv.device) if bias is not None else None
  st = _strides(q_out)
  rc = _lib.load().mdattn_norm_rope_qkv(
      _stream(), _ptr(qkv), _ptr(bias), _ptr(q_out), _ptr(k_out), _ptr(v_out), _ptr(wq), _ptr(wk), _ptr(cos), _ptr(sin),
      b, s, heads, d, eps, q_mul, qkv.stride(0), qkv.stride(1), ctypes.byref(st))
  _lib.check(rc, "mdattn_norm_rope_qkv")
  return q_out, k_out, (v_out if v_out is not None else blocks[2])


def norm_rope_rows(x, w, cos=None, sin=None, heads: int = 1, mode: str = "none", eps: float = 1e-6, out_layout: str = "bshd"):
  """One tensor x [B,S,H*D] (bf16 or f32) -> bf16 logical [B,S,H,D]: full-row RMSNorm with the f32 weight w [H*D],
  then `mode` "none", "interleaved" (cos/sin f32 [B,S,H*D]) or "split" (cos/sin f32 [B,H,S,D/2])."""
  _check_dev(x, w, cos, sin)
  if x.dim() != 3 or x.dtype not in (torch.bfloat16, torch.float32) or x.stride(2) != 1:
    raise ValueError("x must be bf16 or f32 [B, S, H*D] with a contiguous last axis")
  b, s, n = x.shape
  if n % heads:
    raise ValueError(f"inner dim {n} is not divisible by heads={heads}")
  d = n // heads
  modes = {"none": 0, "interleaved": 1, "split": 2}
  if mode not in modes:
    raise ValueError(f"mode={mode!r} not supported. Choose between 'none', 'interleaved' and 'split'.")
  if w.dtype != torch.float32 or w.numel() != n or not w.is_contiguous():
    raise ValueError("w must be a contiguous f32 [H*D] tensor")
  if mode != "none":
    want = (b, s, n) if mode == "interleaved" else (b, heads, s, d // 2)
    for name, t in (("cos", cos), ("sin", sin)):
      if t is None or tuple(t.shape) != want or t.dtype != torch.float32 or not t.is_contiguous():
        raise ValueError(f"{name} must be a contiguous f32 tensor of shape {want} for mode={mode!r}")
  out = _alloc_like_layout(b, s, heads, d, out_layout, torch.bfloat16, x.device)
  st = _strides(out)
  rc = _lib.load().mdattn_norm_rope_rows(
      _stream(), _ptr(x), int(x.dtype == torch.float32), _ptr(out), _ptr(w), _ptr(cos if mode != "none" else None),
      _ptr(sin if mode != "none" else None), modes[mode], b, s, heads, d, eps, x.stride(0), x.stride(1), ctypes.byref(st))
  _lib.check(rc, "mdattn_norm_rope_rows")
  return out


def norm_rope_perhead(q, k, wq, wk, cos, sin, eps: float = 1e-6, wq_txt=None, wk_txt=None, n_txt: int = 0,
                      out_layout: str = "bshd", q_mul: float = 1.0):
  """q, k: bf16 logical [B, S, H, D] views (k may be None); RMSNorm over D per head, then RoPE.
  `q_mul` is multiplied into q_out before its single rounding."""
  _check_dev(q, k, wq, wk, wq_txt, wk_txt, cos, sin)
  if q.dtype != torch.bfloat16:
    raise ValueError("q must be bf16")
  b, s, h, d = q.shape
  if k is not None and (k.shape != q.shape or k.stride() != q.stride() or k.dtype != q.dtype):
    raise ValueError("k must match q in shape, dtype and strides")
  cos, sin = _table(cos, s, d, "cos"), _table(sin, s, d, "sin")
  q_out = _alloc_like_layout(b, s, h, d, out_layout, torch.bfloat16, q.device)
  k_out = _alloc_like_layout(b, s, h, d, out_layout, torch.bfloat16, q.device) if k is not None else None
  si, so = _strides(q), _strides(q_out)
  rc = _lib.load().mdattn_norm_rope_perhead(
      _stream(), _ptr(q), _ptr(k), _ptr(q_out), _ptr(k_out), _ptr(wq), _ptr(wk), _ptr(wq_txt), _ptr(wk_txt), n_txt,
      _ptr(cos), _ptr(sin), b, s, h, d, eps, q_mul, ctypes.byref(si), ctypes.byref(so))
  _lib.check(rc, "mdattn_norm_rope_perhead")
  return q_out, k_out


def _bwd_workspace(rows: int, columns: int, device):
  n = _lib.load().mdattn_norm_rope_bwd_workspace_floats(rows, columns)
  return torch.empty(n, dtype=torch.float32, device=device), n


def _grad_view(g, like_shape, name):
  if g.dim() != 4 or tuple(g.shape) != tuple(like_shape) or g.dtype != torch.bfloat16:
    raise ValueError(f"{name} must be a bf16 logical [B,S,H,D] = {tuple(like_shape)} view, got {tuple(g.shape)} {g.dtype}")
  if g.stride(3) != 1:
    g = g.contiguous()
  return g


def norm_rope_fullrow_backward(q, k, wq, wk, cos, sin, heads: int, gq, gk, eps: float = 1e-6, q_mul: float = 1.0, bias=None,
                               dq=None, dk=None):
  """Backward of `norm_rope_fullrow` (and, with `bias` bf16 [2*H*D], of the q | k blocks of `norm_rope_qkv`).

  q, k: the saved bf16 [B,S,H*D] inputs (k may be None, then gk is None); gq, gk: bf16 logical [B,S,H,D] gradients of
  the prologue's outputs.  Returns (dq, dk, dwq, dwk) -- dq, dk bf16 shaped and strided like q, k (or written into
  the given dq / dk, which may be the column blocks of a fused gradient buffer), dwq, dwk f32 [H*D] -- plus dbias
  f32 [2*H*D] when bias is given."""
  _check_dev(q, k, wq, wk, cos, sin, gq, gk, bias, dq, dk)
  if q.dim() != 3 or q.dtype != torch.bfloat16 or q.stride(2) != 1:
    raise ValueError("q must be bf16 [B, S, H*D] with a contiguous last axis")
  b, s, n = q.shape
  if n % heads:
    raise ValueError(f"inner dim {n} is not divisible by heads={heads}")
  d = n // heads
  has_k = k is not None
  if has_k and (k.shape != q.shape or k.dtype != q.dtype or k.stride() != q.stride()):
    raise ValueError("k must match q in shape, dtype and strides")
  if has_k != (gk is not None):
    raise ValueError("gk must be given exactly when k is")
  cos, sin = _table(cos, s, d, "cos"), _table(sin, s, d, "sin")
  gq = _grad_view(gq, (b, s, heads, d), "gq")
  if has_k:
    gk = _grad_view(gk, (b, s, heads, d), "gk")
    if gk.stride() != gq.stride():
      gk = torch.empty_strided(gq.shape, gq.stride(), dtype=gk.dtype, device=gk.device).copy_(gk)
  if bias is not None and (not has_k or bias.dtype != torch.bfloat16 or bias.numel() != 2 * n or not bias.is_contiguous()):
    raise ValueError("bias must be a contiguous bf16 [2*H*D] tensor (q | k blocks) and needs k")
  if dq is None:
    dq = torch.empty_strided(q.shape, q.stride(), dtype=torch.bfloat16, device=q.device)
  if has_k and dk is None:
    dk = torch.empty_strided(q.shape, q.stride(), dtype=torch.bfloat16, device=q.device)
  for name, t in (("dq", dq), ("dk", dk)):
    if t is not None and (t.shape != q.shape or t.dtype != torch.bfloat16 or t.stride(2) != 1 or (has_k and t.stride() != dq.stride())):
      raise ValueError(f"{name} must be bf16 [B, S, H*D] with a contiguous last axis (dq and dk sharing their strides)")
  dwq = torch.empty(n, dtype=torch.float32, device=q.device)
  dwk = torch.empty(n, dtype=torch.float32, device=q.device) if has_k else None
  dbias = torch.empty(2 * n, dtype=torch.float32, device=q.device) if bias is not None else None
  ws, nws = _bwd_workspace(b * s, (2 if has_k else 1) * (2 if bias is not None else 1) * n, q.device)
  st = _strides(gq)
  rc = _lib.load().mdattn_norm_rope_fullrow_bwd(
      _stream(), _ptr(q), _ptr(k), _ptr(bias), _ptr(gq), _ptr(gk), _ptr(dq), _ptr(dk), _ptr(wq), _ptr(wk), _ptr(dwq), _ptr(dwk),
      _ptr(dbias), _ptr(cos), _ptr(sin), b, s, heads, d, eps, q_mul, q.stride(0), q.stride(1), dq.stride(0), dq.stride(1),
      ctypes.byref(st), _ptr(ws), nws)
  _lib.check(rc, "mdattn_norm_rope_fullrow_bwd")
  return (dq, dk, dwq, dwk) if bias is None else (dq, dk, dwq, dwk, dbias)


def norm_rope_perhead_backward(q, k, wq, wk, cos, sin, gq, gk, eps: float = 1e-6, wq_txt=None, wk_txt=None, n_txt: int = 0,
                               q_mul: float = 1.0):
  """Backward of `norm_rope_perhead`: q, k the saved bf16 logical [B,S,H,D] inputs (k may be None), gq, gk the
  gradients of its outputs.  Returns (dq, dk, dwq, dwk, dwq_txt, dwk_txt): dq, dk bf16 laid out like q; the weight
  gradients f32 [D] (the *_txt ones None when no text weights were given)."""
  _check_dev(q, k, wq, wk, wq_txt, wk_txt, cos, sin, gq, gk)
  if q.dtype != torch.bfloat16:
    raise ValueError("q must be bf16")
  b, s, h, d = q.shape
  has_k = k is not None
  if has_k and (k.shape != q.shape or k.stride() != q.stride() or k.dtype != q.dtype):
    raise ValueError("k must match q in shape, dtype and strides")
  if has_k != (gk is not None):
    raise ValueError("gk must be given exactly when k is")
  cos, sin = _table(cos, s, d, "cos"), _table(sin, s, d, "sin")
  gq = _grad_view(gq, q.shape, "gq")
  if has_k:
    gk = _grad_view(gk, q.shape, "gk")
    if gk.stride() != gq.stride():
      gk = torch.empty_strided(gq.shape, gq.stride(), dtype=gk.dtype, device=gk.device).copy_(gk)
  dq = torch.empty_strided(q.shape, q.stride(), dtype=torch.bfloat16, device=q.device)
  dk = torch.empty_strided(q.shape, q.stride(), dtype=torch.bfloat16, device=q.device) if has_k else None
  f32 = lambda: torch.empty(d, dtype=torch.float32, device=q.device)
  dwq, dwk = f32(), (f32() if has_k else None)
  dwq_t = f32() if wq_txt is not None else None
  dwk_t = f32() if (wk_txt is not None and has_k) else None
  ws, nws = _bwd_workspace(b * s * h, 4 * d, q.device)
  si, sd, sg = _strides(q), _strides(dq), _strides(gq)
  rc = _lib.load().mdattn_norm_rope_perhead_bwd(
      _stream(), _ptr(q), _ptr(k), _ptr(gq), _ptr(gk), _ptr(dq), _ptr(dk), _ptr(wq), _ptr(wk), _ptr(wq_txt),
      _ptr(wk_txt if has_k else None), n_txt, _ptr(dwq), _ptr(dwk), _ptr(dwq_t), _ptr(dwk_t), _ptr(cos), _ptr(sin), b, s, h, d, eps, q_mul,
      ctypes.byref(si), ctypes.byref(sd), ctypes.byref(sg), _ptr(ws), nws)
  _lib.check(rc, "mdattn_norm_rope_perhead_bwd")
  return dq, dk, dwq, dwk, dwq_t, dwk_t


def norm_rope_rows_backward(x, w, g, cos=None, sin=None, heads: int = 1, mode: str = "none", eps: float = 1e-6):
  """Backward of `norm_rope_rows`: x the saved [B,S,H*D] input (bf16 or f32), g the bf16 logical [B,S,H,D] gradient of
  its output.  Returns (dx in x's dtype and strides, dw f32 [H*D])."""
  _check_dev(x, w, cos, sin, g)
  if x.dim() != 3 or x.dtype not in (torch.bfloat16, torch.float32) or x.stride(2) != 1:
    raise ValueError("x must be bf16 or f32 [B, S, H*D] with a contiguous last axis")
  b, s, n = x.shape
  if n % heads:
    raise ValueError(f"inner dim {n} is not divisible by heads={heads}")
  d = n // heads
  modes = {"none": 0, "interleaved": 1, "split": 2}
  if mode not in modes:
    raise ValueError(f"mode={mode!r} not supported. Choose between 'none', 'interleaved' and 'split'.")
  if w.dtype != torch.float32 or w.numel() != n or not w.is_contiguous():
    raise ValueError("w must be a contiguous f32 [H*D] tensor")
  if mode != "none":
    want = (b, s, n) if mode == "interleaved" else (b, heads, s, d // 2)
    for name, t in (("cos", cos), ("sin", sin)):
      if t is None or tuple(t.shape) != want or t.dtype != torch.float32 or not t.is_contiguous():
        raise ValueError(f"{name} must be a contiguous f32 tensor of shape {want} for mode={mode!r}")
  g = _grad_view(g, (b, s, heads, d), "g")
  dx = torch.empty_strided(x.shape, x.stride(), dtype=x.dtype, device=x.device)
  dw = torch.empty(n, dtype=torch.float32, device=x.device)
  ws, nws = _bwd_workspace(b * s, n, x.device)
  st = _strides(g)
  rc = _lib.load().mdattn_norm_rope_rows_bwd(
      _stream(), _ptr(x), int(x.dtype == torch.float32), _ptr(g), _ptr(dx), _ptr(w), _ptr(dw), _ptr(cos if mode != "none" else None),
      _ptr(sin if mode != "none" else None), modes[mode], b, s, heads, d, eps, x.stride(0), x.stride(1), dx.stride(0), dx.stride(1),
      ctypes.byref(st), _ptr(ws), nws)
  _lib.check(rc, "mdattn_norm_rope_rows_bwd")
  return dx, dw


def key_mask_bias(keep: torch.Tensor, masked_value: float = -math.inf) -> torch.Tensor:
  """[B,Skv] keep-mask (bool / uint8) -> additive key bias f32 [B, Skv rounded up to 32] for `flash_attention`."""
  _check_dev(keep)
  if keep.dim() != 2:
    raise ValueError(f"keep mask must have shape [batch, kv_length], got {tuple(keep.shape)}")
  keep8 = keep.to(torch.uint8).contiguous() if keep.dtype != torch.uint8 else keep.contiguous()
  b, skv = keep8.shape
  stride = (skv + 31) // 32 * 32
  bias = torch.empty((b, stride), dtype=torch.float32, device=keep.device)
  rc = _lib.load().mdattn_key_mask_bias(_stream(), _ptr(keep8), _ptr(bias), b, skv, stride, float(masked_value))
  _lib.check(rc, "mdattn_key_mask_bias")
  return bias


def flash_attention(q, k, v, scale: float | None = None, return_lse: bool = False, out_layout: str = "bshd", out=None,
                    key_bias: torch.Tensor | None = None):
  """softmax(scale * q k^T [+ key_bias]) v, non-causal.  q [B,Sq,H,D], k/v [B,Skv,H,D] logical views, bf16.

  `key_bias` f32 [B, >= Skv rounded up to 32] (see `key_mask_bias`) is added to the scaled logits of each key;
  -inf excludes a key.  Returns out (logical [B,Sq,H,D] in `out_layout`) and, if asked, lse f32 [B,H,Sq] (natural log).
  """
  _check_dev(q, k, v)
  if not (q.dtype == k.dtype == v.dtype == torch.bfloat16):
    raise ValueError("flash_attention needs bf16 q, k, v")
  b, sq, h, d = q.shape
  if k.shape != v.shape or k.shape[0] != b or k.shape[2] != h or k.shape[3] != d:
    raise ValueError(f"inconsistent shapes q{tuple(q.shape)} k{tuple(k.shape)} v{tuple(v.shape)}")
  skv = k.shape[1]
  if scale is None:
    scale = 1.0 / math.sqrt(d)
  if out is None:
    out = _alloc_like_layout(b, sq, h, d, out_layout, torch.bfloat16, q.device)
  lse = torch.empty((b, h, sq), dtype=torch.float32, device=q.device) if return_lse else None
  sq_, sk_, sv_, so_ = _strides(q), _strides(k), _strides(v), _strides(out)
  if key_bias is None:
    rc = _lib.load().mdattn_fwd_bf16(
        _stream(), _ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(lse), b, h, sq, skv, d,
        ctypes.byref(sq_), ctypes.byref(sk_), ctypes.byref(sv_), ctypes.byref(so_), float(scale))
    _lib.check(rc, "mdattn_fwd_bf16")
  else:
    _check_dev(key_bias)
    if key_bias.dtype != torch.float32 or key_bias.dim() != 2 or key_bias.shape[0] != b or key_bias.stride(1) != 1:
      raise ValueError("key_bias must be an f32 [batch, padded kv_length] tensor with a contiguous last axis")
    if key_bias.shape[1] != (skv + 31) // 32 * 32:
      # a shorter bias whose padding still covers Skv would silently exclude the trailing keys
      raise ValueError(f"key_bias must have kv_length rounded up to 32 = {(skv + 31) // 32 * 32} columns (padding filled with "
                       f"the masked value), got {key_bias.shape[1]}")
    rc = _lib.load().mdattn_fwd_bf16_bias(
        _stream(), _ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(lse), b, h, sq, skv, d,
        ctypes.byref(sq_), ctypes.byref(sk_), ctypes.byref(sv_), ctypes.byref(so_), float(scale),
        _ptr(key_bias), key_bias.stride(0))
    _lib.check(rc, "mdattn_fwd_bf16_bias")
  return (out, lse) if return_lse else out


def flash_attention_backward(q, k, v, out, dout, lse, scale: float | None = None, key_bias: torch.Tensor | None = None):
  """Gradients of `flash_attention`: q, out, dout [B,Sq,H,D]; k, v [B,Skv,H,D] logical views, bf16; lse f32 [B,H,Sq] as
  returned by the forward; `key_bias` the additive key bias the forward was given, if any.  Returns (dq, dk, dv) shaped
  and laid out like q, k, v."""
  _check_dev(q, k, v, out, dout, lse)
  if not all(t.dtype == torch.bfloat16 for t in (q, k, v, out, dout)):
    raise ValueError("flash_attention_backward needs bf16 q, k, v, out, dout")
  b, sq, h, d = q.shape
  skv = k.shape[1]
  if out.shape != q.shape or dout.shape != q.shape or k.shape != v.shape or tuple(lse.shape) != (b, h, sq):
    raise ValueError("inconsistent shapes")
  if dout.stride() != out.stride():  # the kernels walk out and dout with one set of strides: re-lay dout like out
    dout = torch.empty_strided(out.shape, out.stride(), dtype=dout.dtype, device=dout.device).copy_(dout)
  if scale is None:
    scale = 1.0 / math.sqrt(d)
  lse = lse.contiguous()
  dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
  if dq.stride() != q.stride() or dk.stride() != k.stride() or dv.stride() != v.stride():
    raise ValueError("q, k, v must be dense tensors (their gradients take the same strides)")
  lib = _lib.load()
  nws = lib.mdattn_bwd_workspace_floats(b, h, sq)
  ws = torch.empty(nws, dtype=torch.float32, device=q.device)
  sq_, sk_, sv_, so_ = _strides(q), _strides(k), _strides(v), _strides(out)
  args = (_stream(), _ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(dout), _ptr(lse), _ptr(dq), _ptr(dk), _ptr(dv), _ptr(ws), nws,
          b, h, sq, skv, d, ctypes.byref(sq_), ctypes.byref(sk_), ctypes.byref(sv_), ctypes.byref(so_), float(scale))
  if key_bias is None:
    _lib.check(lib.mdattn_bwd_bf16(*args), "mdattn_bwd_bf16")
  else:
    _check_dev(key_bias)
    if key_bias.dtype != torch.float32 or tuple(key_bias.shape) != (b, (skv + 31) // 32 * 32) or key_bias.stride(1) != 1:
      raise ValueError("key_bias must be the f32 [batch, kv_length rounded up to 32] tensor the forward was given")
    _lib.check(lib.mdattn_bwd_bf16_bias(*args, _ptr(key_bias), key_bias.stride(0)), "mdattn_bwd_bf16_bias")
  return dq, dk, dv


def flash_attention_backward_static(q, k, v, out, dout, lse, dq, dk, dv, scale: float | None = None):
  """`flash_attention_backward` into caller-provided dq, dk, dv (strides of q, k, v) through the entry point that
  allocates nothing: its lse / delta scratch is a static device array of the library (32 MiB per GPU), so the call can
  sit in code that must not allocate (HIP graph capture).  Raises MdattnError (code E_TOOBIG) when B*H*ceil32(Sq)
  exceeds 4,194,304 rows.  Calls that overlap on one GPU share the scratch and race."""
  _check_dev(q, k, v, out, dout, lse, dq, dk, dv)
  if not all(t.dtype == torch.bfloat16 for t in (q, k, v, out, dout, dq, dk, dv)):
    raise ValueError("flash_attention_backward_static needs bf16 tensors")
  b, sq, h, d = q.shape
  if out.shape != q.shape or dout.shape != q.shape or k.shape != v.shape or tuple(lse.shape) != (b, h, sq) or not lse.is_contiguous():
    raise ValueError("inconsistent shapes")
  if dout.stride() != out.stride() or dq.stride() != q.stride() or dk.stride() != k.stride() or dv.stride() != v.stride():
    raise ValueError("dout must share out's strides and dq, dk, dv those of q, k, v")
  if dq.shape != q.shape or dk.shape != k.shape or dv.shape != v.shape:
    raise ValueError("dq, dk, dv must be shaped like q, k, v")
  if scale is None:
    scale = 1.0 / math.sqrt(d)
  sq_, sk_, sv_, so_ = _strides(q), _strides(k), _strides(v), _strides(out)
  rc = _lib.load().mdattn_bwd_bf16_static(
      _stream(), _ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(dout), _ptr(lse), _ptr(dq), _ptr(dk), _ptr(dv),
      b, h, sq, k.shape[1], d, ctypes.byref(sq_), ctypes.byref(sk_), ctypes.byref(sv_), ctypes.byref(so_), float(scale))
  _lib.check(rc, "mdattn_bwd_bf16_static")
  return dq, dk, dv


def quant_e4m3(x: torch.Tensor, premul: float = 1.0, pow2_scale: bool = False):
  """Per-tensor absmax quantisation of a contiguous bf16 tensor -> (uint8 e4m3 bytes, f32[2] scale buffer).

  `premul` is multiplied into x before the single rounding (x * premul ~= x8 * scale[0]); `pow2_scale` rounds the
  scale up to a power of two.  q with premul=folded_q_mul(D) and pow2_scale=True, k with pow2_scale=True and
  flash_attention_fp8(..., scale=FOLDED_SCALE) let the fp8 kernel apply the whole logit scale inside its MFMAs."""
  _check_dev(x)
  if x.dtype != torch.bfloat16 or not x.is_contiguous():
    raise ValueError("quant_e4m3 needs a contiguous bf16 tensor")
  x8 = torch.empty(x.shape, dtype=torch.uint8, device=x.device)
  scale = torch.empty(2, dtype=torch.float32, device=x.device)
  rc = _lib.load().mdattn_quant_e4m3(_stream(), _ptr(x), _ptr(x8), _ptr(scale), x.numel(), float(premul), int(bool(pow2_scale)))
  _lib.check(rc, "mdattn_quant_e4m3")
  return x8, scale


FP8_SOFTMAX_MODES = {"exp2": 0, "byte_grid": 1}


def flash_attention_fp8(q8, k8, v8, q_scale, k_scale, v_scale, scale: float | None = None, return_lse: bool = False,
                        out_layout: str = "bshd", softmax: str = "exp2", key_bias: torch.Tensor | None = None):
  """fp8-e4m3 variant: q8/k8/v8 uint8 logical [B,S,H,D] views, *_scale device f32 tensors (element 0 is used).

  softmax="exp2": exact exponentials; the lse is the logsumexp of the quantised logits and the pair (out, lse) can be
  merged like a bf16 partial.  softmax="byte_grid": with power-of-two q and k scales and the softmax scale carried by
  q (see `quant_e4m3`) P is a piecewise-linear exponential read off the e4m3 byte grid (12 % faster; out keeps its
  accuracy, the lse is only good to about 0.08); with any other scales it is the same as "exp2".
  `key_bias` (see `key_mask_bias`): additive per-key bias, -inf excludes a key; always the exact-exponential softmax."""
  if softmax not in FP8_SOFTMAX_MODES:
    raise ValueError(f"softmax={softmax!r} not supported. Choose between 'exp2' and 'byte_grid'.")
  _check_dev(q8, k8, v8, q_scale, k_scale, v_scale)
  b, sq, h, d = q8.shape
  skv = k8.shape[1]
  if scale is None:
    scale = 1.0 / math.sqrt(d)
  out = _alloc_like_layout(b, sq, h, d, out_layout, torch.bfloat16, q8.device)
  lse = torch.empty((b, h, sq), dtype=torch.float32, device=q8.device) if return_lse else None
  sq_, sk_, sv_, so_ = _strides(q8), _strides(k8), _strides(v8), _strides(out)
  args = (_stream(), _ptr(q8), _ptr(k8), _ptr(v8), _ptr(out), _ptr(lse), b, h, sq, skv, d,
          ctypes.byref(sq_), ctypes.byref(sk_), ctypes.byref(sv_), ctypes.byref(so_), float(scale),
          _ptr(q_scale), _ptr(k_scale), _ptr(v_scale))
  if key_bias is None:
    _lib.check(_lib.load().mdattn_fwd_fp8(*args, FP8_SOFTMAX_MODES[softmax]), "mdattn_fwd_fp8")
  else:
    _check_dev(key_bias)
    if key_bias.dtype != torch.float32 or tuple(key_bias.shape) != (b, (skv + 31) // 32 * 32) or key_bias.stride(1) != 1:
      raise ValueError(f"key_bias must be an f32 [batch, kv_length rounded up to 32] = [{b}, {(skv + 31) // 32 * 32}] tensor")
    _lib.check(_lib.load().mdattn_fwd_fp8_bias(*args, _ptr(key_bias), key_bias.stride(0)), "mdattn_fwd_fp8_bias")
  return (out, lse) if return_lse else out


def new_merge_state(b, s, h, d, device, layout: str = "bshd"):
  """(o_run f32 zeros as a logical [B,S,H,D] view, lse_run f32 [B,H,S] filled with -1e30)."""
  o = _alloc_like_layout(b, s, h, d, layout, torch.float32, device)
  o.zero_()
  lse = torch.full((b, h, s), LSE_INIT, dtype=torch.float32, device=device)
  return o, lse


def merge_partial(o_run, lse_run, o_cur, lse_cur):
  """In-place LSE-space merge of (o_cur, lse_cur) into (o_run, lse_run)."""
  _check_dev(o_run, lse_run, o_cur, lse_cur)
  b, s, h, d = o_run.shape
  if o_run.dtype != torch.float32 or o_cur.shape != o_run.shape or o_cur.dtype not in (torch.bfloat16, torch.float32):
    raise ValueError("o_run must be f32 and o_cur bf16/f32 of the same logical shape")
  for t in (lse_run, lse_cur):
    if t.dtype != torch.float32 or tuple(t.shape) != (b, h, s) or not t.is_contiguous():
      raise ValueError("lse tensors must be contiguous f32 [B,H,S]")
  sr, sc = _strides(o_run), _strides(o_cur)
  rc = _lib.load().mdattn_merge(
      _stream(), _ptr(o_run), _ptr(lse_run), _ptr(o_cur), _ptr(lse_cur), int(o_cur.dtype == torch.float32),
      b, h, s, d, ctypes.byref(sr), ctypes.byref(sc))
  _lib.check(rc, "mdattn_merge")
  return o_run, lse_run


def flash_attention_merge(q, k, v, o_run, lse_run, scale: float | None = None):
  """One ring step in one launch: attention of q [B,Sq,H,D] against the chunk k/v [B,Skv,H,D] (bf16 logical views),
  merged in place into (o_run f32 logical [B,Sq,H,D], lse_run f32 [B,H,Sq]) as `merge_partial` would merge the
  result of `flash_attention`; the chunk's own output is never stored."""
  _check_dev(q, k, v, o_run, lse_run)
  if not (q.dtype == k.dtype == v.dtype == torch.bfloat16):
    raise ValueError("flash_attention_merge needs bf16 q, k, v")
  b, sq, h, d = q.shape
  if k.shape != v.shape or k.shape[0] != b or k.shape[2] != h or k.shape[3] != d:
    raise ValueError(f"inconsistent shapes q{tuple(q.shape)} k{tuple(k.shape)} v{tuple(v.shape)}")
  if o_run.dtype != torch.float32 or tuple(o_run.shape) != (b, sq, h, d):
    raise ValueError("o_run must be an f32 logical [B,Sq,H,D] view")
  if lse_run.dtype != torch.float32 or tuple(lse_run.shape) != (b, h, sq) or not lse_run.is_contiguous():
    raise ValueError("lse_run must be contiguous f32 [B,H,Sq]")
  if scale is None:
    scale = 1.0 / math.sqrt(d)
  sq_, sk_, sv_, sr_ = _strides(q), _strides(k), _strides(v), _strides(o_run)
  rc = _lib.load().mdattn_fwd_bf16_merge(
      _stream(), _ptr(q), _ptr(k), _ptr(v), _ptr(o_run), _ptr(lse_run), b, h, sq, k.shape[1], d,
      ctypes.byref(sq_), ctypes.byref(sk_), ctypes.byref(sv_), ctypes.byref(sr_), float(scale))
  _lib.check(rc, "mdattn_fwd_bf16_merge")
  return o_run, lse_run


def finalize(o_run: torch.Tensor) -> torch.Tensor:
  """f32 -> bf16 cast of a merged accumulator, same memory layout."""
  _check_dev(o_run)
  if o_run.dtype != torch.float32:
    raise ValueError("finalize needs an f32 tensor")
  out = torch.empty_like(o_run, dtype=torch.bfloat16)  # preserves strides of dense permuted views
  if out.stride() != o_run.stride():
    raise ValueError("finalize needs a dense tensor")
  rc = _lib.load().mdattn_finalize(_stream(), _ptr(o_run), _ptr(out), o_run.numel())
  _lib.check(rc, "mdattn_finalize")
  return out
