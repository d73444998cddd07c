"""Registers the HIP kernels with a live maxdiffusion + JAX (ROCm) install.

`install()` (1) registers the XLA-FFI targets exported by libmdattn_ffi.so with
``jax.ffi.register_ffi_target(..., platform="ROCM")`` and (2) adds ``hip_flash`` and ``hip_flash_fp8`` to
maxdiffusion's own KERNEL_REGISTRY (models/attention_flax.py:1589-1597), after which
``attention: hip_flash`` in any Wan / Flux / LTX config reaches the MI355X kernel through
the unchanged `_apply_attention` (models/attention_flax.py:1965-1966).

Every compute entry point of include/mdattn.h has one custom-call target here (FFI_TARGETS) and one wrapper below;
the operands, results and attributes of each `jax.ffi.ffi_call` follow the bind line of the same target in
csrc/ffi/mdattn_ffi.cc, in order.  Nothing here runs at import time: jax, jaxlib's FFI headers and maxdiffusion are
absent from the build image, so this module is exercised with them only where they exist
(tests/test_ffi_shim.py drives every wrapper through a recording stand-in for `jax.ffi`).
"""
from __future__ import annotations

import ctypes
import math
import os

from .build import FFI_LIB_PATH, build_ffi_library

# custom-call target (= the C-ABI entry point it ends in) -> handler symbol exported by libmdattn_ffi.so
FFI_TARGETS = {
    "mdattn_fwd_bf16": "MdattnFwdBf16",
    "mdattn_fwd_bf16_bias": "MdattnFwdBf16Bias",
    "mdattn_key_mask_bias": "MdattnKeyMaskBias",
    "mdattn_fwd_bf16_merge": "MdattnFwdBf16Merge",
    "mdattn_merge": "MdattnMerge",
    "mdattn_finalize": "MdattnFinalize",
    "mdattn_norm_rope_fullrow": "MdattnNormRopeFullrow",
    "mdattn_norm_rope_qkv": "MdattnNormRopeQkv",
    "mdattn_norm_rope_perhead": "MdattnNormRopePerhead",
    "mdattn_norm_rope_rows": "MdattnNormRopeRows",
    "mdattn_norm_rope_fullrow_bwd": "MdattnNormRopeFullrowBwd",
    "mdattn_norm_rope_perhead_bwd": "MdattnNormRopePerheadBwd",
    "mdattn_norm_rope_rows_bwd": "MdattnNormRopeRowsBwd",
    "mdattn_quant_e4m3": "MdattnQuantE4m3",
    "mdattn_fwd_fp8": "MdattnFwdFp8",
    "mdattn_fwd_fp8_bias": "MdattnFwdFp8Bias",
    "mdattn_bwd_bf16": "MdattnBwdBf16",
    "mdattn_bwd_bf16_bias": "MdattnBwdBf16Bias",
    "mdattn_bwd_bf16_static": "MdattnBwdBf16Static",
}
# entry points of mdattn.h that are host-side helpers, not kernels: no custom call
HOST_ONLY = ("mdattn_version", "mdattn_strerror", "mdattn_build_id", "mdattn_set_fwd_schedule",
             "mdattn_bwd_workspace_floats", "mdattn_bwd_static_max_floats", "mdattn_norm_rope_bwd_workspace_floats")

BWD_STATIC_MAX_FLOATS = 8 * 1024 * 1024  # MDATTN_BWD_STATIC_MAX_FLOATS of include/mdattn.h
NORM_ROPE_BWD_MAX_PARTIAL_ROWS = 1024    # mdattn_norm_rope_bwd_workspace_floats(rows, columns) = min(rows, 1024) * columns

FOLDED_SCALE = math.log(2.0)  # see ops.FOLDED_SCALE: scale * log2(e) == 1, the softmax scale rides on q
FOLD_SCALE_MIN_KEYS = 16384   # from this many keys on (head dim 128; half at 64), hip_flash_kernel folds the scale into q itself

_installed = False


def _require_jax():
  try:
    import jax  # noqa: F401
    import jax.ffi  # noqa: F401
    import jax.numpy as jnp  # noqa: F401
  except ImportError as e:  # pragma: no cover - jax is not in the build image
    raise RuntimeError("maxdiffusion_amd.jax_plugin needs jax with ROCm support") from e
  return jax, jnp


def register_ffi_targets():
  jax, _ = _require_jax()
  if not os.path.exists(FFI_LIB_PATH) and build_ffi_library() is None:
    raise RuntimeError("libmdattn_ffi.so is missing and jaxlib's FFI headers were not found to build it")
  lib = ctypes.CDLL(FFI_LIB_PATH)
  for target, symbol in FFI_TARGETS.items():
    jax.ffi.register_ffi_target(target, jax.ffi.pycapsule(getattr(lib, symbol)), platform="ROCM")


def _f32(x):
  import numpy as np

  return np.float32(x)


def _i64(x):
  import numpy as np

  return np.int64(x)


def _bshd_dims(x, layout: int):
  if layout == 0:
    b, s, h, d = x.shape
  else:
    b, h, s, d = x.shape
  return b, s, h, d


def hip_key_mask_bias(keep_mask, masked_value: float = -math.inf):
  """[B,Skv] bool keep-mask -> additive key bias f32 [B, Skv rounded up to 32] (masked keys and the padding get
  `masked_value`): the mask canonicalisation of models/attention_flax.py:1931-1939 for the flash-type kernels."""
  jax, jnp = _require_jax()
  if keep_mask.ndim != 2:
    raise ValueError(f"attention_mask must have shape [batch, kv_length], got {tuple(keep_mask.shape)}.")
  b, skv = keep_mask.shape
  call = jax.ffi.ffi_call("mdattn_key_mask_bias", jax.ShapeDtypeStruct((b, (skv + 31) // 32 * 32), jnp.float32), vmap_method="sequential")
  return call(keep_mask.astype(jnp.bool_), masked_value=_f32(masked_value))


def hip_flash_attention(q, k, v, scale: float, layout: int, keep_mask=None):
  """q [B,Sq,H,D] (layout 0) or [B,H,Sq,D] (layout 1) bf16 -> (out [B,Sq,H,D] bf16, lse [B,H,Sq] f32).

  keep_mask: optional [B,Skv] bool; masked keys are excluded, rows without a kept key return 0."""
  jax, jnp = _require_jax()
  b, sq, h, d = _bshd_dims(q, layout)
  results = (jax.ShapeDtypeStruct((b, sq, h, d), jnp.bfloat16), jax.ShapeDtypeStruct((b, h, sq), jnp.float32))
  if keep_mask is not None:
    skv = _bshd_dims(k, layout)[1]
    if tuple(keep_mask.shape) != (b, skv):
      raise ValueError(f"attention_mask must have shape [batch, kv_length] = {(b, skv)}, got {tuple(keep_mask.shape)}.")
    call = jax.ffi.ffi_call("mdattn_fwd_bf16_bias", results, vmap_method="sequential")
    return call(q, k, v, hip_key_mask_bias(keep_mask), scale=_f32(scale), layout=_i64(layout))
  call = jax.ffi.ffi_call("mdattn_fwd_bf16", results, vmap_method="sequential")
  return call(q, k, v, scale=_f32(scale), layout=_i64(layout))


def hip_quant_e4m3(x, premul: float = 1.0, pow2_scale: bool = False):
  """Per-tensor absmax quantisation of a bf16 array -> (float8_e4m3fn array of the same shape, f32[2]: [0] the
  de-quantisation scale of x * premul, [1] absmax(x))."""
  jax, jnp = _require_jax()
  call = jax.ffi.ffi_call("mdattn_quant_e4m3", (jax.ShapeDtypeStruct(x.shape, jnp.float8_e4m3fn), jax.ShapeDtypeStruct((2,), jnp.float32)),
                          vmap_method="sequential")
  return call(x.astype(jnp.bfloat16), premul=_f32(premul), pow2_scale=_i64(bool(pow2_scale)))


def hip_flash_attention_fp8(q, k, v, scale: float, layout: int, softmax: str = "byte_grid", keep_mask=None):
  """The fp8 configuration of the benchmark (Wan-14B self-attention in e4m3): quantises bf16 q, k, v per tensor (q carries scale * log2(e), q and k scales are powers of
  two) and runs the fp8-e4m3 kernel.  softmax "byte_grid" (fastest; use `out`) or "exp2" (exact lse, mergeable);
  keep_mask [B,Skv] bool: masked keys are excluded (exact exponentials).
  Returns (out [B,Sq,H,D] bf16, lse [B,H,Sq] f32)."""
  jax, jnp = _require_jax()
  modes = {"exp2": 0, "byte_grid": 1}
  if softmax not in modes:
    raise ValueError(f"softmax={softmax!r} not supported. Choose between 'exp2' and 'byte_grid'.")
  b, sq, h, d = _bshd_dims(q, layout)
  q8, qs = hip_quant_e4m3(q, premul=scale * math.log2(math.e), pow2_scale=True)
  k8, ks = hip_quant_e4m3(k, pow2_scale=True)
  v8, vs = hip_quant_e4m3(v)
  results = (jax.ShapeDtypeStruct((b, sq, h, d), jnp.bfloat16), jax.ShapeDtypeStruct((b, h, sq), jnp.float32))
  if keep_mask is not None:
    skv = _bshd_dims(k, layout)[1]
    if tuple(keep_mask.shape) != (b, skv):
      raise ValueError(f"attention_mask must have shape [batch, kv_length] = {(b, skv)}, got {tuple(keep_mask.shape)}.")
    call = jax.ffi.ffi_call("mdattn_fwd_fp8_bias", results, vmap_method="sequential")
    return call(q8, k8, v8, qs, ks, vs, hip_key_mask_bias(keep_mask), scale=_f32(FOLDED_SCALE), layout=_i64(layout))
  call = jax.ffi.ffi_call("mdattn_fwd_fp8", results, vmap_method="sequential")
  return call(q8, k8, v8, qs, ks, vs, scale=_f32(FOLDED_SCALE), layout=_i64(layout), softmax_mode=_i64(modes[softmax]))


def hip_ring_step(q, k_chunk, v_chunk, o_run, lse_run, scale: float, layout: int = 0):
  """One ring hop in one custom call: attention of q against the visiting K/V chunk merged into the carry
  (o_run f32 [B,Sq,H,D], lse_run f32 [B,H,Sq]; start from zeros and -1e30).  The body of the scan step in
  kernels/splash_attention/ring_attention_kernel.py:1045-1073; the carry is donated and updated in place."""
  jax, jnp = _require_jax()
  call = jax.ffi.ffi_call(
      "mdattn_fwd_bf16_merge",
      (jax.ShapeDtypeStruct(o_run.shape, jnp.float32), jax.ShapeDtypeStruct(lse_run.shape, jnp.float32)),
      input_output_aliases={3: 0, 4: 1},
      vmap_method="sequential",
  )
  return call(q, k_chunk, v_chunk, o_run, lse_run, scale=_f32(scale), layout=_i64(layout))


def hip_merge(o_run, lse_run, o_cur, lse_cur):
  """LSE-space merge of a normalised partial (o_cur bf16|f32 [B,S,H,D], lse_cur) into the donated carry
  (kernels/splash_attention/ring_attention_kernel.py:1062-1073)."""
  jax, jnp = _require_jax()
  call = jax.ffi.ffi_call(
      "mdattn_merge",
      (jax.ShapeDtypeStruct(o_run.shape, jnp.float32), jax.ShapeDtypeStruct(lse_run.shape, jnp.float32)),
      input_output_aliases={0: 0, 1: 1},
      vmap_method="sequential",
  )
  return call(o_run, lse_run, o_cur, lse_cur)


def hip_finalize(o_run):
  """f32 carry -> bf16 (the `.astype(q.dtype)` of ring_attention_kernel.py:1130)."""
  jax, jnp = _require_jax()
  call = jax.ffi.ffi_call("mdattn_finalize", jax.ShapeDtypeStruct(o_run.shape, jnp.bfloat16), vmap_method="sequential")
  return call(o_run)


def hip_flash_attention_vjp(q, k, v, scale: float, static_scratch: bool = False, keep_mask=None, layout: int = 0,
                            residual_checkpoint_name: str | None = None):
  """Differentiable attention: jax.custom_vjp around the forward and backward custom calls (what
  kernels/splash_attention/splash_attention_kernel.py:1166, :2067 do for the Pallas kernels), on [B,S,H,D] (layout 0) or
  [B,H,S,D] (layout 1) bf16 arrays; returns out [B,Sq,H,D].  keep_mask: a [B,Skv] key padding mask, honoured by the
  forward and the backward alike.  residual_checkpoint_name: the saved (out, lse) are tagged with
  jax.ad_checkpoint.checkpoint_name, as the reference's wrappers tag their residuals for the remat policies
  (models/attention_flax.py:1941-1962).  static_scratch: the backward whose scratch is a static device array of the
  library (no workspace result); used only when the shape fits that array (decided here, at trace time), and it assumes
  that XLA runs the custom calls of one GPU on one stream: two such calls overlapping on one GPU would race on the array."""
  jax, jnp = _require_jax()
  bias = hip_key_mask_bias(keep_mask) if keep_mask is not None else None
  if keep_mask is not None:
    skv = _bshd_dims(k, layout)[1]
    if tuple(keep_mask.shape) != (q.shape[0], skv):
      raise ValueError(f"attention_mask must have shape [batch, kv_length] = {(q.shape[0], skv)}, got {tuple(keep_mask.shape)}.")
  b, sq, h, d = _bshd_dims(q, layout)
  results = (jax.ShapeDtypeStruct((b, sq, h, d), jnp.bfloat16), jax.ShapeDtypeStruct((b, h, sq), jnp.float32))
  nws = 2 * b * h * ((sq + 31) // 32 * 32)  # mdattn_bwd_workspace_floats
  use_static = static_scratch and bias is None and nws <= BWD_STATIC_MAX_FLOATS
  # the backward custom calls take [B,S,H,D] operands: layout 1 inputs are transposed for them (XLA fuses the copies
  # into the producers where it can); the forward reads either layout in place
  to_bshd = (lambda x: x) if layout == 0 else (lambda x: x.transpose(0, 2, 1, 3))

  def forward(q, k, v):
    if bias is None:
      call = jax.ffi.ffi_call("mdattn_fwd_bf16", results, vmap_method="sequential")
      return call(q, k, v, scale=_f32(scale), layout=_i64(layout))
    call = jax.ffi.ffi_call("mdattn_fwd_bf16_bias", results, vmap_method="sequential")
    return call(q, k, v, bias, scale=_f32(scale), layout=_i64(layout))

  @jax.custom_vjp
  def attn(q, k, v):
    return forward(q, k, v)[0]

  def fwd(q, k, v):
    out, lse = forward(q, k, v)
    if residual_checkpoint_name is not None:
      from jax.ad_checkpoint import checkpoint_name

      out, lse = checkpoint_name(out, residual_checkpoint_name), checkpoint_name(lse, residual_checkpoint_name + "_lse")
    return out, (q, k, v, out, lse)

  def bwd(res, dout):
    q, k, v, out, lse = res
    q, k, v = to_bshd(q), to_bshd(k), to_bshd(v)
    grads = (jax.ShapeDtypeStruct(q.shape, jnp.bfloat16), jax.ShapeDtypeStruct(k.shape, jnp.bfloat16), jax.ShapeDtypeStruct(v.shape, jnp.bfloat16))
    if use_static:
      call = jax.ffi.ffi_call("mdattn_bwd_bf16_static", grads, vmap_method="sequential")
      dq, dk, dv = call(q, k, v, out, dout.astype(jnp.bfloat16), lse, scale=_f32(scale))
    else:
      results_b = grads + (jax.ShapeDtypeStruct((nws,), jnp.float32),)
      if bias is not None:
        call = jax.ffi.ffi_call("mdattn_bwd_bf16_bias", results_b, vmap_method="sequential")
        dq, dk, dv, _ = call(q, k, v, out, dout.astype(jnp.bfloat16), lse, bias, scale=_f32(scale))
      else:
        call = jax.ffi.ffi_call("mdattn_bwd_bf16", results_b, vmap_method="sequential")
        dq, dk, dv, _ = call(q, k, v, out, dout.astype(jnp.bfloat16), lse, scale=_f32(scale))
    return to_bshd(dq), to_bshd(dk), to_bshd(dv)  # the transposition is its own inverse: back to the inputs' layout

  attn.defvjp(fwd, bwd)
  return attn(q, k, v)


def _partial_rows_floats(rows: int, columns: int) -> int:
  return min(rows, NORM_ROPE_BWD_MAX_PARTIAL_ROWS) * columns


def hip_norm_rope_fullrow(q, k, wq, wk, cos, sin, heads: int, eps: float = 1e-6, q_mul: float = 1.0):
  """q, k [B,S,H*D] bf16 (k may be None: cached text K/V); cos/sin f32 [S,D/2] or None (norm only) -> (q_out, k_out)
  [B,S,H,D] bf16.  `q_mul` is multiplied into q_out before its rounding: D**-0.5 * log2(e) here and scale = ln 2 in
  hip_flash_attention carry the softmax scale in the prologue.  FlaxWanAttention.__call__, attention_flax.py:2655-2677.
  Differentiable with respect to q, k, wq, wk (jax.custom_vjp around mdattn_norm_rope_fullrow_bwd; the reference
  differentiates through these lines by autodiff)."""
  jax, jnp = _require_jax()
  b, s, n = q.shape
  d = n // heads
  rope, has_k = cos is not None, k is not None
  dummy = jnp.zeros((8,), jnp.float32)
  cos_, sin_ = (cos, sin) if rope else (dummy, dummy)
  attrs = dict(eps=_f32(eps), q_mul=_f32(q_mul), heads=_i64(heads), rope=_i64(rope), has_k=_i64(has_k))

  def forward(q, k, wq, wk):
    out = jax.ShapeDtypeStruct((b, s, heads, d), jnp.bfloat16)
    k_out = out if has_k else jax.ShapeDtypeStruct((8,), jnp.bfloat16)
    call = jax.ffi.ffi_call("mdattn_norm_rope_fullrow", (out, k_out), vmap_method="sequential")
    return call(q, k, wq, wk, cos_, sin_, **attrs)

  @jax.custom_vjp
  def prologue(q, k, wq, wk):
    return forward(q, k, wq, wk)

  def fwd(q, k, wq, wk):
    return forward(q, k, wq, wk), (q, k, wq, wk)

  def bwd(res, g):
    q, k, wq, wk = res
    gq, gk = g
    cols = n * (2 if has_k else 1)
    small = jax.ShapeDtypeStruct((8,), jnp.bfloat16)
    small_f = jax.ShapeDtypeStruct((8,), jnp.float32)
    results = (jax.ShapeDtypeStruct(q.shape, jnp.bfloat16), jax.ShapeDtypeStruct(q.shape, jnp.bfloat16) if has_k else small,
               jax.ShapeDtypeStruct((n,), jnp.float32), jax.ShapeDtypeStruct((n,), jnp.float32) if has_k else small_f, small_f,
               jax.ShapeDtypeStruct((_partial_rows_floats(b * s, cols),), jnp.float32))
    call = jax.ffi.ffi_call("mdattn_norm_rope_fullrow_bwd", results, vmap_method="sequential")
    dq, dk, dwq, dwk, _, _ = call(q, k, gq.astype(jnp.bfloat16), gk.astype(jnp.bfloat16) if has_k else gq.astype(jnp.bfloat16), wq, wk,
                                  cos_, sin_, wq, has_bias=_i64(0), **attrs)
    # without k the stand-in operands (q, wq) receive zero cotangents
    return dq, (dk if has_k else jnp.zeros(k.shape, k.dtype)), dwq.astype(wq.dtype), (dwk.astype(wk.dtype) if has_k else jnp.zeros(wk.shape, wk.dtype))

  prologue.defvjp(fwd, bwd)
  q_out, k_res = prologue(q, k if has_k else q, wq, wk if has_k else wq)
  return q_out, (k_res if has_k else None)


def hip_norm_rope_qkv(qkv, wq, wk, cos, sin, heads: int, bias=None, eps: float = 1e-6, q_mul: float = 1.0):
  """The prologue over the output of one fused q|k|v projection: qkv bf16 [B,S,3*H*D] (column blocks q | k | v);
  bias bf16 [3*H*D] or None (the Linear biases, when the GEMM ran without them) -> (q, k, v) [B,S,H,D] bf16.  Without
  a bias v is a slice of the fused buffer (XLA fuses the reshape; nothing is copied by the custom call).  One launch in
  place of the three bias adds, norm_q / norm_k, _unflatten_heads and _apply_rope of attention_flax.py:2653-2677.
  Differentiable with respect to qkv, wq, wk and bias: the backward runs mdattn_norm_rope_fullrow_bwd on the q | k
  blocks (with their biases) and passes v's gradient through (its bias gradient is the token sum)."""
  jax, jnp = _require_jax()
  b, s, n3 = qkv.shape
  n = n3 // 3
  d = n // heads
  rope, has_bias = cos is not None, bias is not None
  dummy = jnp.zeros((8,), jnp.float32)
  cos_, sin_ = (cos, sin) if rope else (dummy, dummy)

  def forward(qkv, wq, wk, bias_):
    out = jax.ShapeDtypeStruct((b, s, heads, d), jnp.bfloat16)
    v_out = out if has_bias else jax.ShapeDtypeStruct((8,), jnp.bfloat16)
    call = jax.ffi.ffi_call("mdattn_norm_rope_qkv", (out, out, v_out), vmap_method="sequential")
    q_out, k_out, v_res = call(qkv, bias_, wq, wk, cos_, sin_, eps=_f32(eps), q_mul=_f32(q_mul), heads=_i64(heads),
                               rope=_i64(rope), has_bias=_i64(has_bias), has_v=_i64(has_bias))
    return q_out, k_out, (v_res if has_bias else qkv[:, :, 2 * n:].reshape(b, s, heads, d))

  @jax.custom_vjp
  def prologue(qkv, wq, wk, bias_):
    return forward(qkv, wq, wk, bias_)

  def fwd(qkv, wq, wk, bias_):
    return forward(qkv, wq, wk, bias_), (qkv, wq, wk, bias_)

  def bwd(res, g):
    qkv, wq, wk, bias_ = res
    gq, gk, gv = g
    cols = 2 * n * (2 if has_bias else 1)
    rows = jax.ShapeDtypeStruct((b, s, n), jnp.bfloat16)
    vec = jax.ShapeDtypeStruct((n,), jnp.float32)
    results = (rows, rows, vec, vec, jax.ShapeDtypeStruct((2 * n,) if has_bias else (8,), jnp.float32),
               jax.ShapeDtypeStruct((_partial_rows_floats(b * s, cols),), jnp.float32))
    call = jax.ffi.ffi_call("mdattn_norm_rope_fullrow_bwd", results, vmap_method="sequential")
    dq, dk, dwq, dwk, dbias_qk, _ = call(qkv[:, :, :n], qkv[:, :, n:2 * n], gq.astype(jnp.bfloat16), gk.astype(jnp.bfloat16), wq, wk,
                                         cos_, sin_, bias_[:2 * n] if has_bias else wq, eps=_f32(eps), q_mul=_f32(q_mul),
                                         heads=_i64(heads), rope=_i64(rope), has_k=_i64(1), has_bias=_i64(has_bias))
    gv_rows = gv.astype(jnp.bfloat16).reshape(b, s, n)
    dqkv = jnp.concatenate([dq, dk, gv_rows], axis=2)
    if has_bias:
      dbias = jnp.concatenate([dbias_qk, gv.astype(jnp.float32).sum(axis=(0, 1)).reshape(n)]).astype(bias_.dtype)
    else:
      dbias = jnp.zeros(bias_.shape, bias_.dtype)  # the stand-in operand (wq) receives a zero cotangent
    return dqkv, dwq.astype(wq.dtype), dwk.astype(wk.dtype), dbias

  prologue.defvjp(fwd, bwd)
  return prologue(qkv, wq, wk, bias if has_bias else wq)


def hip_norm_rope_perhead(q, k, wq, wk, cos, sin, eps: float = 1e-6, wq_txt=None, wk_txt=None, n_txt: int = 0, q_mul: float = 1.0):
  """q, k [B,S,H,D] bf16 (k may be None); per-head RMSNorm with weights [D]; tokens [0, n_txt) take wq_txt / wk_txt
  (FlaxFluxAttention's encoder_*_norm on the text tokens of the joint sequence, attention_flax.py:3002-3003);
  cos/sin f32 [S,D/2] or None -> (q_out, k_out) [B,S,H,D] bf16.  FlaxFluxAttention.__call__, :2989-3020.
  Differentiable with respect to q, k and the four weights (jax.custom_vjp around mdattn_norm_rope_perhead_bwd)."""
  jax, jnp = _require_jax()
  rope, has_k = cos is not None, k is not None
  if n_txt and (wq_txt is None or (has_k and wk_txt is None)):
    raise ValueError("n_txt > 0 needs the text-token norm weights wq_txt (and wk_txt with k)")
  dummy = jnp.zeros((8,), jnp.float32)
  cos_, sin_ = (cos, sin) if rope else (dummy, dummy)
  d = q.shape[-1]
  attrs = dict(eps=_f32(eps), q_mul=_f32(q_mul), n_txt=_i64(n_txt), rope=_i64(rope), has_k=_i64(has_k))

  def forward(q, k, wq, wk, wqt, wkt):
    out = jax.ShapeDtypeStruct(q.shape, jnp.bfloat16)
    k_out = out if has_k else jax.ShapeDtypeStruct((8,), jnp.bfloat16)
    call = jax.ffi.ffi_call("mdattn_norm_rope_perhead", (out, k_out), vmap_method="sequential")
    return call(q, k, wq, wk, wqt, wkt, cos_, sin_, **attrs)

  @jax.custom_vjp
  def prologue(q, k, wq, wk, wqt, wkt):
    return forward(q, k, wq, wk, wqt, wkt)

  def fwd(q, k, wq, wk, wqt, wkt):
    return forward(q, k, wq, wk, wqt, wkt), (q, k, wq, wk, wqt, wkt)

  def bwd(res, g):
    q, k, wq, wk, wqt, wkt = res
    gq, gk = g
    b, s, h, _ = q.shape
    act, vec = jax.ShapeDtypeStruct(q.shape, jnp.bfloat16), jax.ShapeDtypeStruct((d,), jnp.float32)
    small, small_f = jax.ShapeDtypeStruct((8,), jnp.bfloat16), jax.ShapeDtypeStruct((8,), jnp.float32)
    results = (act, act if has_k else small, vec, vec if has_k else small_f, vec if n_txt else small_f,
               vec if (n_txt and has_k) else small_f, jax.ShapeDtypeStruct((_partial_rows_floats(b * s * h, 4 * d),), jnp.float32))
    call = jax.ffi.ffi_call("mdattn_norm_rope_perhead_bwd", results, vmap_method="sequential")
    gq = gq.astype(jnp.bfloat16)
    dq, dk, dwq, dwk, dwqt, dwkt, _ = call(q, k, gq, gk.astype(jnp.bfloat16) if has_k else gq, wq, wk, wqt, wkt, cos_, sin_, **attrs)
    zero = lambda x: jnp.zeros(x.shape, x.dtype)
    return (dq, dk if has_k else zero(k), dwq.astype(wq.dtype), dwk.astype(wk.dtype) if has_k else zero(wk),
            dwqt.astype(wqt.dtype) if n_txt else zero(wqt), dwkt.astype(wkt.dtype) if (n_txt and has_k) else zero(wkt))

  prologue.defvjp(fwd, bwd)
  q_out, k_res = prologue(q, k if has_k else q, wq, wk if has_k else wq, wq_txt if n_txt else wq, wk_txt if (n_txt and has_k) else wq)
  return q_out, (k_res if has_k else None)


def hip_norm_rope_ltx2(query, key, norm_q_scale, norm_k_scale, heads: int, rotary_emb=None, k_rotary_emb=None,
                       rope_type: str = "interleaved", is_self_attention: bool = True, eps: float = 1e-6, q_mul: float = 1.0):
  """Fused prologue of LTX2Attention.__call__ (models/ltx2/attention_ltx2.py:556-585): see attention_op.hip_norm_rope_ltx2.
  query/key [B,S,H*D] -> bf16 [B,S,H,D]; tables (cos, sin) as LTX2RotaryPosEmbed returns them; `q_mul` is folded into
  the f32 query scale."""
  jax, jnp = _require_jax()
  if rope_type not in ("interleaved", "split"):
    raise ValueError(f"{rope_type=} not supported. Choose between 'interleaved' and 'split'.")
  q_tab = rotary_emb
  k_tab = k_rotary_emb if k_rotary_emb is not None else (rotary_emb if is_self_attention else None)
  if rotary_emb is None:
    q_tab = k_tab = None
  dummy = jnp.zeros((8,), jnp.float32)

  def run(x, scale, tab):
    b, s, n = x.shape
    mode = 0 if tab is None else (1 if rope_type == "interleaved" else 2)
    cos, sin = (dummy, dummy) if tab is None else (tab[0].astype(jnp.float32), tab[1].astype(jnp.float32))
    attrs = dict(eps=_f32(eps), heads=_i64(heads), mode=_i64(mode))

    def forward(x, w):
      out = jax.ShapeDtypeStruct((b, s, heads, n // heads), jnp.bfloat16)
      return jax.ffi.ffi_call("mdattn_norm_rope_rows", out, vmap_method="sequential")(x, w, cos, sin, **attrs)

    @jax.custom_vjp
    def prologue(x, w):
      return forward(x, w)

    def fwd(x, w):
      return forward(x, w), (x, w)

    def bwd(res, g):
      x, w = res
      results = (jax.ShapeDtypeStruct(x.shape, x.dtype), jax.ShapeDtypeStruct((n,), jnp.float32),
                 jax.ShapeDtypeStruct((_partial_rows_floats(b * s, n),), jnp.float32))
      dx, dw, _ = jax.ffi.ffi_call("mdattn_norm_rope_rows_bwd", results, vmap_method="sequential")(x, g.astype(jnp.bfloat16), w, cos, sin, **attrs)
      return dx, dw

    prologue.defvjp(fwd, bwd)
    return prologue(x, scale.astype(jnp.float32))

  q_scale = norm_q_scale if q_mul == 1.0 else norm_q_scale * q_mul
  return run(query, q_scale, q_tab), (run(key, norm_k_scale, k_tab) if key is not None else None)


def _as_rank4(q, k, v, heads: int):
  """Registry inputs are rank 3 [B,S,H*D] (a free reshape to [B,S,H,D]: layout 0) or rank 4 [B,H,S,D] (layout 1)."""
  if q.ndim == 3:
    b, sq, n = q.shape
    d = n // heads
    return q.reshape(b, sq, heads, d), k.reshape(b, k.shape[1], heads, d), v.reshape(b, v.shape[1], heads, d), 0
  return q, k, v, 1


def _pad_head_dim(q4, k4, v4):
  """Head dims below 128 other than 64: zero-padded to the next size the kernels take (64 or 128), as the reference's
  flash wrappers pad to 128 (attention_flax.py:223-259); returns the arrays and the original head dim, to which the
  caller slices the output.  jnp.pad and the slice are differentiable, so the custom_vjp inside sees padded shapes."""
  _, jnp = _require_jax()
  d = q4.shape[-1]
  if d in (64, 128) or d > 128:
    return q4, k4, v4, d
  extra = (64 if d < 64 else 128) - d
  widths = ((0, 0), (0, 0), (0, 0), (0, extra))
  return jnp.pad(q4, widths), jnp.pad(k4, widths), jnp.pad(v4, widths), d


def hip_flash_kernel(q, k, v, context):
  """The KERNEL_REGISTRY entry `hip_flash`: fn(q, k, v, context) -> [B, Sq, H*D] in q's dtype.  The function is a
  jax.custom_vjp (forward custom call with lse, backward custom calls): the trainer differentiates straight through
  `apply_attention` (trainers/wan_trainer.py:169), as it does through the reference's own kernels
  (kernels/splash_attention/splash_attention_kernel.py:1166, :2067).  Both input layouts, the key mask and
  context["residual_checkpoint_name"] are honoured.  f32 inputs (LTX-2's q, k) are cast to bf16 by XLA, one more pass
  over each; `hip_norm_rope_ltx2` in front of this entry emits bf16 and leaves nothing to cast."""
  _, jnp = _require_jax()
  if context.get("is_causal"):
    raise NotImplementedError("hip_flash is non-causal")
  q4, k4, v4, layout = _as_rank4(q, k, v, context["heads"])
  q4, k4, v4, d0 = _pad_head_dim(q4, k4, v4)
  dt = q.dtype
  scale, mask = context["scale"], context.get("attention_mask")
  q4 = q4.astype(jnp.bfloat16)
  c = scale * math.log2(math.e)
  if mask is None and k4.shape[2 if layout else 1] * 128 >= FOLD_SCALE_MIN_KEYS * k4.shape[-1] and abs(c - 1.0) > 1e-6:
    # long key sequences: q * (scale * log2 e) in bf16 (XLA fuses the multiply into q's producer) and scale = ln 2, on
    # which forward and backward kernels drop the multiply per logit; the reference rounds the same factors into its
    # operands (attention_flax.py:1783, :610).  Autodiff scales dq back through the multiply.
    q4, scale = q4 * c, FOLDED_SCALE
  out = hip_flash_attention_vjp(q4, k4.astype(jnp.bfloat16), v4.astype(jnp.bfloat16), scale,
                                keep_mask=mask, layout=layout,
                                residual_checkpoint_name=context.get("residual_checkpoint_name"))
  b, sq, h, d = out.shape
  return out[..., :d0].reshape(b, sq, h * d0).astype(dt)


def hip_flash_fp8_kernel(q, k, v, context):
  """The KERNEL_REGISTRY entry `hip_flash_fp8` (the benchmark's fp8 configuration): per-tensor e4m3 q, k, v on the device, then the
  fp8 kernel; a [B,Skv] attention_mask is honoured like hip_flash honours it."""
  _, jnp = _require_jax()
  if context.get("is_causal"):
    raise NotImplementedError("hip_flash is non-causal")
  q4, k4, v4, layout = _as_rank4(q, k, v, context["heads"])
  q4, k4, v4, d0 = _pad_head_dim(q4, k4, v4)
  dt = q.dtype
  out, _ = hip_flash_attention_fp8(q4.astype(jnp.bfloat16), k4.astype(jnp.bfloat16), v4.astype(jnp.bfloat16), context["scale"], layout,
                                   keep_mask=context.get("attention_mask"))
  b, sq, h, d = out.shape
  return out[..., :d0].reshape(b, sq, h * d0).astype(dt)


def install():
  """Idempotent: FFI targets + maxdiffusion KERNEL_REGISTRY['hip_flash'] and ['hip_flash_fp8']."""
  global _installed
  if _installed:
    return
  register_ffi_targets()
  from maxdiffusion.models import attention_flax  # type: ignore

  attention_flax.register_kernel("hip_flash")(hip_flash_kernel)
  attention_flax.register_kernel("hip_flash_fp8")(hip_flash_fp8_kernel)
  _installed = True
