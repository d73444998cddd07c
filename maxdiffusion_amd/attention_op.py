"""Host-side mirror of maxdiffusion's attention plug-in surface for the `hip_flash` kernel.

Same names, argument meaning and error behaviour as the reference (paths relative to
``src/maxdiffusion/``):

  KERNEL_REGISTRY / register_kernel   models/attention_flax.py:1589-1597
  _check_attention_inputs             models/attention_flax.py:99-106
  _apply_attention                    models/attention_flax.py:1870-1968
  AttentionOp.apply_attention         models/attention_flax.py:2241-2273 (NNXAttentionOp)

Arrays are torch tensors in device memory (the image has no JAX); `jax_plugin.py` registers
the same kernels with a live maxdiffusion install.  Only the MI355X kernels are registered:
an unknown name raises ValueError exactly like the reference, and no name is ever demoted
to a CPU implementation.
"""
from __future__ import annotations

import math

import torch

from . import ops

__all__ = [
    "KERNEL_REGISTRY", "register_kernel", "AttentionOp", "hip_flash_kernel", "hip_flash_fp8_kernel",
    "hip_norm_rope", "hip_norm_rope_qkv", "hip_norm_rope_ltx2", "hip_flash_attention_autograd", "HIP_KERNEL_NAMES",
]

KERNEL_REGISTRY = {}

# Names chosen to contain none of "ring", "ulysses", "custom", "tokamax": the reference keys axis-rule
# injection and block-size plumbing on those substrings (pyconfig.py:237-238, max_utils.py:781-786).
HIP_KERNEL_NAMES = ("hip_flash", "hip_flash_fp8")

# Kernel names the reference demotes to dot_product below flash_min_seq_length
# (attention_flax.py:1905-1912).  The HIP kernels are not in the list: they serve every length.
_FLASH_MIN_LENGTH_GATED = ("flash", "tokamax_flash", "ulysses", "ulysses_custom", "ulysses_custom_fixed_m", "ulysses_ring")


def register_kernel(name: str):
  def decorator(func):
    KERNEL_REGISTRY[name] = func
    return func

  return decorator


def _check_attention_inputs(query, key, value) -> None:
  assert key.ndim == value.ndim, "k, v must have same rank."
  assert query.shape[:-3] == key.shape[:-3] == value.shape[:-3], "q, k, v batch dims must match."
  assert key.shape[-2] == value.shape[-2], "k, v num_kv_heads must match."
  assert key.shape[-3] == value.shape[-3], "k, v lengths must match."
  assert query.shape[-1] == key.shape[-1], "q, k depths must match."


def _as_bshd(x: torch.Tensor, heads: int) -> torch.Tensor:
  """[B,S,H*D] -> view [B,S,H,D];  [B,H,S,D] -> view [B,S,H,D] (what _reshape_data_for_flash,
  attention_flax.py:200-220, does with a transpose; here it is a stride change)."""
  if x.dim() == 3:
    b, s, n = x.shape
    if n % heads:
      raise ValueError(f"inner dim {n} is not divisible by heads={heads}")
    if x.stride(2) != 1:
      x = x.contiguous()
    return x.view(b, s, heads, n // heads) if x.is_contiguous() else x.unflatten(2, (heads, n // heads))
  if x.dim() == 4:
    if x.stride(3) != 1:
      x = x.contiguous()
    return x.permute(0, 2, 1, 3)
  raise ValueError(f"attention inputs must have rank 3 or 4, got {x.dim()}")


def _reject_unsupported(context) -> None:
  # The custom kernels of the reference raise NotImplementedError for what they cannot honour
  # (attention_flax.py:850-854, :1300-1304); these kernels are non-causal.
  if context.get("is_causal"):
    raise NotImplementedError("hip_flash is non-causal")


def _mask_bias(context, qv, kv):
  """context["attention_mask"] ([B,Skv] keep-mask or None) -> additive key bias for the kernels, or None."""
  mask = context.get("attention_mask")
  if mask is None:
    return None
  if tuple(mask.shape) != (qv.shape[0], kv.shape[1]):
    # the reference's additive bias would fail to broadcast against the [B,H,Sq,Skv] scores (:1550)
    raise ValueError(f"attention_mask must have shape [batch, kv_length] = {(qv.shape[0], kv.shape[1])}, got {tuple(mask.shape)}.")
  return ops.key_mask_bias(mask)


# From this many keys on at head dim 128 (half as many at head dim 64, where the multiply weighs twice as much), the
# registry entry folds the softmax scale into q before the call (see hip_flash_kernel): the pass over q costs what the
# multiply per logit costs at about 9,000 (4,000) keys.
FOLD_SCALE_MIN_KEYS = 16384


def _pad_head_dim(qv, kv, vv):
  """Head dims below 128 other than 64 are zero-padded to the next size the kernels take (64 or 128), as the
  reference's flash wrappers pad them to 128 (attention_flax.py:223-259, `_pad_data_for_flash`): zero columns of q and
  k add nothing to a logit, zero columns of v give output columns that the caller of this helper slices off.  Returns
  the (possibly padded) views and the original head dim.  One more pass over each tensor; gradients flow through the
  pad.  Head dims above 128 are left alone: the kernel entry rejects them."""
  d = qv.shape[-1]
  if d in (64, 128) or d > 128:
    return qv, kv, vv, d
  extra = (64 if d < 64 else 128) - d
  return tuple(torch.nn.functional.pad(t, (0, extra)) for t in (qv, kv, vv)) + (d,)


def _dense(t: torch.Tensor) -> torch.Tensor:
  """A view whose memory is dense in some axis order (the backward kernels write gradients with the operand's strides)."""
  return t if t.is_contiguous() or t.permute(0, 2, 1, 3).is_contiguous() else t.contiguous()


class _HipFlashAttention(torch.autograd.Function):
  """Forward + backward through the HIP kernels: the registry entry carries its own VJP, as the reference's kernels do
  (kernels/splash_attention/splash_attention_kernel.py:1166, :2067 define the custom_vjp the trainer differentiates
  through, trainers/wan_trainer.py:169).  Saved for the backward: q, k, v, out, lse -- the residuals the reference
  tags with `residual_checkpoint_name` for its remat policies; torch's checkpointing re-runs the forward instead, so
  the name is carried in the context and not used here."""

  @staticmethod
  def forward(ctx, q, k, v, scale, key_bias):
    out, lse = ops.flash_attention(q, k, v, scale=scale, return_lse=True, key_bias=key_bias)
    ctx.save_for_backward(q, k, v, out, lse)
    ctx.scale, ctx.key_bias = scale, key_bias
    return out

  @staticmethod
  def backward(ctx, dout):
    q, k, v, out, lse = ctx.saved_tensors
    dq, dk, dv = ops.flash_attention_backward(q, k, v, out, dout.to(torch.bfloat16), lse, scale=ctx.scale, key_bias=ctx.key_bias)
    return dq, dk, dv, None, None


def hip_flash_attention_autograd(q, k, v, scale: float, key_bias=None):
  """Differentiable attention on bf16 logical [B,S,H,D] views (torch autograd); key_bias as for ops.flash_attention."""
  return _HipFlashAttention.apply(_dense(q), _dense(k), _dense(v), float(scale), key_bias)


@register_kernel("hip_flash")
def hip_flash_kernel(q, k, v, context):
  """KERNEL_REGISTRY entry: fn(q, k, v, context) -> [B, Sq, H*D] in q's dtype.

  Unlike the reference's flash entries, which pass k * scale (attention_flax.py:1783), the scale goes
  to the kernel and is folded into the exp2 argument; `flash_block_sizes`, `mesh` and the axis names
  are accepted and ignored (one GPU, tiles fixed by the kernel).  Differentiable: when autograd is recording and an
  input requires a gradient, the call goes through `_HipFlashAttention` (forward with lse, HIP backward), in both
  input layouts and with a key mask.
  """
  _reject_unsupported(context)
  heads = context["heads"]
  qv, kv, vv = _as_bshd(q, heads), _as_bshd(k, heads), _as_bshd(v, heads)
  # LTX2 hands f32 q/k next to a v in the model dtype (norm dtype f32, attention_ltx2.py:415-432); the MFMA operands are
  # bf16.  Each such cast is one more pass over the tensor in HBM: `hip_norm_rope_ltx2` in front of this entry emits
  # bf16 q/k straight from the prologue kernel and leaves nothing to cast.
  cast = q.dtype != torch.bfloat16
  qv, kv, vv = (t if t.dtype == torch.bfloat16 else t.to(torch.bfloat16) for t in (qv, kv, vv))
  # [B,Skv] keep-mask (attention_flax.py:1926-1939): masked keys are excluded, as the flash wrappers do with
  # segment ids (:390-438); rows without a kept key return 0 (:1552-1554)
  bias = _mask_bias(context, qv, kv)
  qv, kv, vv, d0 = _pad_head_dim(qv, kv, vv)
  scale = context["scale"]
  if torch.is_grad_enabled() and (qv.requires_grad or kv.requires_grad or vv.requires_grad):
    out = hip_flash_attention_autograd(qv, kv, vv, scale, bias)
  else:
    c = scale * math.log2(math.e)
    if bias is None and kv.shape[1] * 128 >= FOLD_SCALE_MIN_KEYS * qv.shape[-1] and abs(c - 1.0) > 1e-6:
      # Long key sequences: q * (scale * log2 e), rounded to bf16 once, then scale = ln 2, on which the kernels drop the
      # multiply per logit (3.5 % of the launch at head dim 128, 7 % at 64) for one pass over q.  The reference's flash
      # wrappers round the same factors into their operands (k * scale and q * log2 e in bf16,
      # attention_flax.py:1783, :610).  Callers that apply the fused prologue with q_mul arrive here with scale = ln 2
      # already and skip this.
      qv, scale = qv * c, ops.FOLDED_SCALE
    out = ops.flash_attention(qv, kv, vv, scale=scale, key_bias=bias)
  b, s, h, d = out.shape
  out = out[..., :d0].reshape(b, s, h * d0)
  return out.to(q.dtype) if cast else out


@register_kernel("hip_flash_fp8")
def hip_flash_fp8_kernel(q, k, v, context):
  """fp8-e4m3 variant: per-tensor absmax quantisation of q, k, v on the device, then the fp8 kernel.  Forward only:
  called with inputs that require a gradient while autograd is recording, it raises instead of returning a result that
  would silently carry no gradient (train through `hip_flash`)."""
  _reject_unsupported(context)
  if torch.is_grad_enabled() and (q.requires_grad or k.requires_grad or v.requires_grad):
    raise NotImplementedError("hip_flash_fp8 has no backward pass: use hip_flash for training, or call it under torch.no_grad()")
  heads = context["heads"]
  qv, kv, vv, d0 = _pad_head_dim(*(_as_bshd(t, heads).to(torch.bfloat16) for t in (q, k, v)))
  qv, kv, vv = qv.contiguous(), kv.contiguous(), vv.contiguous()
  # the softmax scale rides on q's quantisation (one rounding either way) and the q and k scales are powers of two:
  # the kernel then applies the whole logit scale inside its MFMAs; the registry entry returns `out` only, so it asks
  # for the softmax without exponentials (P's e4m3 byte straight from the logit: a piecewise-linear exponential
  # within e4m3's own rounding noise).  Callers that need an lse to merge use ops.flash_attention_fp8(softmax="exp2").
  q8, sq = ops.quant_e4m3(qv, premul=context["scale"] * math.log2(math.e), pow2_scale=True)
  k8, sk = ops.quant_e4m3(kv, pow2_scale=True)
  v8, sv = ops.quant_e4m3(vv)
  # a [B,Skv] keep-mask goes in as an additive key bias (exact-exponential softmax), as for hip_flash
  out = ops.flash_attention_fp8(q8, k8, v8, sq, sk, sv, scale=ops.FOLDED_SCALE, softmax="byte_grid", key_bias=_mask_bias(context, qv, kv))
  b, s, h, d = out.shape
  return out[..., :d0].reshape(b, s, h * d0).to(q.dtype)



def _wants_grad(*ts) -> bool:
  return torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in ts)


class _HipNormRopeFullrow(torch.autograd.Function):
  """The Wan prologue with its HIP backward: saved for the backward are the inputs only (the row statistics are
  recomputed); the reference differentiates through these lines by JAX autodiff (attention_flax.py:2655-2677)."""

  @staticmethod
  def forward(ctx, q, k, wq, wk, cos, sin, heads, eps, out_layout, q_mul):
    q_out, k_out = ops.norm_rope_fullrow(q, k, wq, wk, cos, sin, heads, eps, out_layout, q_mul)
    ctx.save_for_backward(q, k, wq, wk, cos, sin)
    ctx.cfg = (heads, eps, q_mul)
    return q_out, k_out

  @staticmethod
  def backward(ctx, gq, gk):
    q, k, wq, wk, cos, sin = ctx.saved_tensors
    heads, eps, q_mul = ctx.cfg
    dq, dk, dwq, dwk = ops.norm_rope_fullrow_backward(q, k, wq, wk, cos, sin, heads, gq.to(torch.bfloat16),
                                                      gk.to(torch.bfloat16) if k is not None else None, eps, q_mul)
    return dq, dk, dwq.to(wq.dtype), (dwk.to(wk.dtype) if k is not None else None), None, None, None, None, None, None


class _HipNormRopeQkv(torch.autograd.Function):
  """The prologue over a fused q|k|v projection output with its HIP backward: the q | k blocks of the gradient buffer
  are written by mdattn_norm_rope_fullrow_bwd (which also returns their bias gradients), v's block is its output
  gradient (v only gains a bias, whose gradient is the token sum)."""

  @staticmethod
  def forward(ctx, qkv, bias, wq, wk, cos, sin, heads, eps, out_layout, q_mul):
    q_out, k_out, v_out = ops.norm_rope_qkv(qkv, wq, wk, cos, sin, heads, bias, eps, out_layout, q_mul)
    ctx.save_for_backward(qkv, bias, wq, wk, cos, sin)
    ctx.cfg = (heads, eps, q_mul)
    return q_out, k_out, v_out

  @staticmethod
  def backward(ctx, gq, gk, gv):
    qkv, bias, wq, wk, cos, sin = ctx.saved_tensors
    heads, eps, q_mul = ctx.cfg
    b, s, n3 = qkv.shape
    n = n3 // 3
    dqkv = torch.empty((b, s, n3), dtype=torch.bfloat16, device=qkv.device)
    res = ops.norm_rope_fullrow_backward(qkv[:, :, :n], qkv[:, :, n:2 * n], wq, wk, cos, sin, heads, gq.to(torch.bfloat16),
                                         gk.to(torch.bfloat16), eps, q_mul, bias=None if bias is None else bias[:2 * n].contiguous(),
                                         dq=dqkv[:, :, :n], dk=dqkv[:, :, n:2 * n])
    dqkv[:, :, 2 * n:].unflatten(2, (heads, n // heads)).copy_(gv)
    dbias = None
    if bias is not None:
      dbias = torch.cat([res[4], gv.float().sum(dim=(0, 1)).reshape(n)]).to(bias.dtype)
    return dqkv, dbias, res[2].to(wq.dtype), res[3].to(wk.dtype), None, None, None, None, None, None


class _HipNormRopePerhead(torch.autograd.Function):
  """The Flux prologue with its HIP backward (attention_flax.py:2989-3020)."""

  @staticmethod
  def forward(ctx, q, k, wq, wk, wq_txt, wk_txt, cos, sin, eps, n_txt, out_layout, q_mul):
    q_out, k_out = ops.norm_rope_perhead(q, k, wq, wk, cos, sin, eps, wq_txt, wk_txt, n_txt, out_layout, q_mul)
    ctx.save_for_backward(q, k, wq, wk, wq_txt, wk_txt, cos, sin)
    ctx.cfg = (eps, n_txt, q_mul)
    return q_out, k_out

  @staticmethod
  def backward(ctx, gq, gk):
    q, k, wq, wk, wq_txt, wk_txt, cos, sin = ctx.saved_tensors
    eps, n_txt, q_mul = ctx.cfg
    dq, dk, dwq, dwk, dwq_t, dwk_t = ops.norm_rope_perhead_backward(
        q, k, wq, wk, cos, sin, gq.to(torch.bfloat16), gk.to(torch.bfloat16) if k is not None else None, eps, wq_txt, wk_txt, n_txt, q_mul)
    cast = lambda g, w: None if g is None else g.to(w.dtype)
    return dq, dk, cast(dwq, wq), cast(dwk, wk), cast(dwq_t, wq_txt), cast(dwk_t, wk_txt), None, None, None, None, None, None


class _HipNormRopeRows(torch.autograd.Function):
  """The LTX-2 prologue of one tensor with its HIP backward (models/ltx2/attention_ltx2.py:556-585)."""

  @staticmethod
  def forward(ctx, x, w, cos, sin, heads, mode, eps):
    out = ops.norm_rope_rows(x, w, cos, sin, heads=heads, mode=mode, eps=eps)
    ctx.save_for_backward(x, w, cos, sin)
    ctx.cfg = (heads, mode, eps)
    return out

  @staticmethod
  def backward(ctx, g):
    x, w, cos, sin = ctx.saved_tensors
    heads, mode, eps = ctx.cfg
    dx, dw = ops.norm_rope_rows_backward(x, w, g.to(torch.bfloat16), cos, sin, heads=heads, mode=mode, eps=eps)
    return dx, dw, None, None, None, None, None


def _norm_rope_rows(x, w, cos, sin, heads, mode, eps):
  if _wants_grad(x, w):
    return _HipNormRopeRows.apply(x, w, cos, sin, heads, mode, eps)
  return ops.norm_rope_rows(x, w, cos, sin, heads=heads, mode=mode, eps=eps)


def hip_norm_rope_qkv(qkv, wq, wk, freqs_cis, heads: int, bias=None, eps: float = 1e-6, out_layout: str = "bshd",
                      q_mul: float = 1.0, inplace: bool = False):
  """The fused prologue over the output of ONE q|k|v projection `[B,S,3*H*D]` (the three projections of
  attention_flax.py:2653-2663 run as one GEMM): bias adds, norm_q / norm_k, head split and rotation in one launch;
  returns (q, k, v) logical [B,S,H,D] for `hip_flash`.  `bias`: the three Linear biases [3*H*D] when the GEMM ran
  without them.  Differentiable with respect to qkv, bias and the norm weights; `inplace=True` (the fused buffer
  itself becomes the three operands) is for inference only, since the backward needs the projection output."""
  b, s, n3 = qkv.shape
  cos, sin = _split_table(freqs_cis, s, n3 // 3 // heads)
  if _wants_grad(qkv, wq, wk, bias):
    if inplace:
      raise ValueError("inplace=True overwrites the projection output that the backward pass needs")
    return _HipNormRopeQkv.apply(qkv, bias, wq, wk, cos, sin, heads, eps, out_layout, q_mul)
  return ops.norm_rope_qkv(qkv, wq, wk, cos, sin, heads, bias, eps, out_layout, q_mul, inplace)


def hip_norm_rope_ltx2(query, key, norm_q_scale, norm_k_scale, heads: int, rotary_emb=None, k_rotary_emb=None,
                       rope_type: str = "interleaved", is_self_attention: bool = True, eps: float = 1e-6,
                       q_mul: float = 1.0):
  """Fused prologue of LTX2Attention.__call__ (models/ltx2/attention_ltx2.py:556-585).

  query/key [B,S,H*D] (bf16 or f32) are normalised over the full inner dim with the f32 scales; the query is rotated
  by `rotary_emb`, the key by `k_rotary_emb` if given, else by `rotary_emb` when this is self-attention, else not
  at all.  Tables are (cos, sin) as LTX2RotaryPosEmbed returns them: [B,S,H*D] (interleaved) or [B,H,S,D/2] (split).
  Returns (q, k) bf16 [B,S,H,D], ready for `hip_flash`.  `key` None (cached K/V): only the query is processed.
  `q_mul` (see hip_norm_rope) is folded into the f32 query scale on the host."""
  if rope_type not in ("interleaved", "split"):
    raise ValueError(f"{rope_type=} not supported. Choose between 'interleaved' and 'split'.")  # :145-146
  q_tab = rotary_emb
  k_tab = k_rotary_emb if k_rotary_emb is not None else (rotary_emb if is_self_attention else None)
  if rotary_emb is None:
    q_tab = k_tab = None

  def run(x, scale, tab):
    if tab is None:
      return _norm_rope_rows(x, scale, None, None, heads, "none", eps)
    cos, sin = (t.to(torch.float32).contiguous() for t in tab)
    return _norm_rope_rows(x, scale, cos, sin, heads, rope_type, eps)

  q = run(query, norm_q_scale if q_mul == 1.0 else norm_q_scale * q_mul, q_tab)
  k = run(key, norm_k_scale, k_tab) if key is not None else None
  return q, k



def _apply_attention(
    query,
    key,
    value,
    heads: int,
    dim_head: int,
    split_head_dim: bool,
    float32_qk_product: bool,
    attention_kernel: str,
    flash_min_seq_length: int,
    use_memory_efficient_attention: bool,
    scale: float,
    dtype,
    mesh,
    axis_names_q,
    axis_names_kv,
    flash_block_sizes,
    dpa_layer,
    mask_padding_tokens: bool = True,
    residual_checkpoint_name: str | None = None,
    attention_mask=None,
    use_base2_exp: bool = False,
    use_experimental_scheduler: bool = False,
    ulysses_shards: int = -1,
    ulysses_attention_chunks: int = 1,
    is_causal: bool = False,
):
  """Routes to an attention kernel through the module-level registry (attention_flax.py:1870-1968)."""
  _check_attention_inputs(query, key, value)
  seq_len_idx = 2 if query.ndim == 4 else 1

  can_use_flash_attention = True
  if attention_kernel in _FLASH_MIN_LENGTH_GATED:
    can_use_flash_attention = (
        query.shape[seq_len_idx] >= flash_min_seq_length
        and key.shape[seq_len_idx] >= flash_min_seq_length
        and value.shape[seq_len_idx] >= flash_min_seq_length
    )

  effective_attention_kernel = attention_kernel
  if attention_kernel == "dot_product" or use_memory_efficient_attention or not can_use_flash_attention:
    effective_attention_kernel = "dot_product"

  if attention_mask is not None:
    if attention_mask.ndim != 2:
      raise ValueError(f"attention_mask must have shape [batch, kv_length], got {tuple(attention_mask.shape)}.")
    attention_mask = attention_mask.to(torch.bool)

  context = {
      "heads": heads,
      "mesh": mesh,
      "axis_names_q": axis_names_q,
      "axis_names_kv": axis_names_kv,
      "flash_block_sizes": flash_block_sizes,
      "dtype": dtype,
      "mask_padding_tokens": mask_padding_tokens,
      "residual_checkpoint_name": residual_checkpoint_name,
      "attention_mask": attention_mask,
      "scale": scale,
      "use_base2_exp": use_base2_exp,
      "use_experimental_scheduler": use_experimental_scheduler,
      "ulysses_shards": ulysses_shards,
      "ulysses_attention_chunks": ulysses_attention_chunks,
      "dim_head": dim_head,
      "split_head_dim": split_head_dim,
      "float32_qk_product": float32_qk_product,
      "use_memory_efficient_attention": use_memory_efficient_attention,
      "dpa_layer": dpa_layer,
      "is_causal": is_causal,
  }

  if effective_attention_kernel in KERNEL_REGISTRY:
    return KERNEL_REGISTRY[effective_attention_kernel](query, key, value, context)

  raise ValueError(f"Unexpected attention kernel {effective_attention_kernel=}.")


class AttentionOp:
  """Same constructor arguments and `apply_attention` signature as NNXAttentionOp
  (attention_flax.py:2172-2273); `mesh`, axis names and block sizes are carried, not used."""

  def __init__(
      self,
      mesh=None,
      attention_kernel: str = "hip_flash",
      scale: float = 1.0,
      heads: int = 1,
      dim_head: int = 128,
      use_memory_efficient_attention: bool = False,
      split_head_dim: bool = True,
      float32_qk_product: bool = True,
      axis_names_q=("activation_batch", "activation_heads", "activation_length", "activation_kv"),
      axis_names_kv=("activation_batch", "activation_heads", "activation_kv_length", "activation_kv"),
      flash_min_seq_length: int = 0,
      flash_block_sizes=None,
      dtype=torch.float32,
      quant=None,
      mask_padding_tokens: bool = True,
      residual_checkpoint_name: str | None = None,
      use_base2_exp: bool = False,
      use_experimental_scheduler: bool = False,
      ulysses_shards: int = -1,
      ulysses_attention_chunks: int = 1,
  ):
    self.dpa_layer = None
    self.mesh = mesh
    self.scale = scale
    self.heads = heads
    self.dim_head = dim_head
    self.attention_kernel = attention_kernel
    self.use_memory_efficient_attention = use_memory_efficient_attention
    self.split_head_dim = split_head_dim
    self.float32_qk_product = float32_qk_product
    self.axis_names_q = axis_names_q
    self.axis_names_kv = axis_names_kv
    self.flash_min_seq_length = flash_min_seq_length
    self.flash_block_sizes = flash_block_sizes
    self.dtype = dtype
    self.quant = quant
    self.mask_padding_tokens = mask_padding_tokens
    self.residual_checkpoint_name = residual_checkpoint_name
    self.use_base2_exp = use_base2_exp
    self.use_experimental_scheduler = use_experimental_scheduler
    self.ulysses_shards = ulysses_shards
    self.ulysses_attention_chunks = ulysses_attention_chunks

  def apply_attention(self, query, key, value, attention_mask=None):
    return _apply_attention(
        query=query,
        key=key,
        value=value,
        heads=self.heads,
        dim_head=self.dim_head,
        split_head_dim=self.split_head_dim,
        float32_qk_product=self.float32_qk_product,
        attention_kernel=self.attention_kernel,
        flash_min_seq_length=self.flash_min_seq_length,
        use_memory_efficient_attention=self.use_memory_efficient_attention,
        scale=self.scale,
        dtype=self.dtype,
        mesh=self.mesh,
        axis_names_q=self.axis_names_q,
        axis_names_kv=self.axis_names_kv,
        flash_block_sizes=self.flash_block_sizes,
        dpa_layer=self.dpa_layer,
        mask_padding_tokens=self.mask_padding_tokens,
        residual_checkpoint_name=self.residual_checkpoint_name,
        attention_mask=attention_mask,
        use_base2_exp=self.use_base2_exp,
        use_experimental_scheduler=self.use_experimental_scheduler,
        ulysses_shards=self.ulysses_shards,
        ulysses_attention_chunks=self.ulysses_attention_chunks,
    )


def _split_table(freqs_cis, seq: int, d: int):
  """Accepts the reference's rotary tables and returns contiguous f32 (cos, sin) [S, D/2]:
  complex [1,1,S,D/2] (WanRotaryPosEmbed), (cos, sin) tuples with D or D/2 columns
  (FluxPosEmbed return_tuple, repeated pairwise), or the [S, D/2, 2, 2] matrix form."""
  if freqs_cis is None:
    return None, None
  if isinstance(freqs_cis, (tuple, list)):
    cos, sin = freqs_cis
    cos, sin = cos.reshape(seq, -1), sin.reshape(seq, -1)
    if cos.shape[1] == d:  # each angle repeated for both members of the pair
      cos, sin = cos[:, 0::2], sin[:, 0::2]
  elif torch.is_complex(freqs_cis):
    t = freqs_cis.reshape(seq, d // 2)
    cos, sin = t.real, t.imag
  else:
    t = freqs_cis.reshape(seq, d // 2, 2, 2)
    cos, sin = t[:, :, 0, 0], t[:, :, 1, 0]
  return cos.to(torch.float32).contiguous(), sin.to(torch.float32).contiguous()


def hip_norm_rope(q, k, wq, wk, freqs_cis, heads: int, eps: float = 1e-6, per_head: bool = False,
                  wq_txt=None, wk_txt=None, n_txt: int = 0, out_layout: str = "bshd", q_mul: float = 1.0):
  """The fused prologue the attention modules call in place of their inline norm + rope.

  per_head=False: FlaxWanAttention.__call__ lines attention_flax.py:2655-2677 (q, k are [B,S,H*D]).
  per_head=True : FlaxFluxAttention.__call__ lines :2989-3020 (q, k are [B,S,H,D] views).
  freqs_cis=None is the norm-only mode of the cross-attention (:2671).  Returns logical [B,S,H,D]
  views laid out as `out_layout`, ready for `hip_flash` with no transpose in between.  Differentiable with respect to
  q, k and the norm weights (torch autograd through the HIP backward kernels), so a trainer can keep the hook.
  `q_mul` is multiplied into the query before its single rounding: with q_mul=ops.folded_q_mul(D) and
  context["scale"]=ops.FOLDED_SCALE the softmax scale is carried by the prologue, where the reference carries it by
  two bf16 multiplies of k and q (:1783, :610), and the attention kernel saves its multiply per logit.
  """
  if per_head:
    b, s, h, d = q.shape
    cos, sin = _split_table(freqs_cis, s, d)
    if _wants_grad(q, k, wq, wk, wq_txt, wk_txt):
      return _HipNormRopePerhead.apply(q, k, wq, wk, wq_txt, wk_txt, cos, sin, eps, n_txt, out_layout, q_mul)
    return ops.norm_rope_perhead(q, k, wq, wk, cos, sin, eps, wq_txt, wk_txt, n_txt, out_layout, q_mul)
  b, s, n = q.shape
  cos, sin = _split_table(freqs_cis, s, n // heads)
  if _wants_grad(q, k, wq, wk):
    return _HipNormRopeFullrow.apply(q, k, wq, wk, cos, sin, heads, eps, out_layout, q_mul)
  return ops.norm_rope_fullrow(q, k, wq, wk, cos, sin, heads, eps, out_layout, q_mul)
