"""Registers the HIP kernels with a live maxdiffusion + JAX (ROCm) install.

`install()` (1) registers the XLA-FFI targets exported by libmdattn_ffi.so with
``jax.ffi.register_ffi_target(..., platform="ROCM")`` and (2) adds ``hip_flash`` to
maxdiffusion's own KERNEL_REGISTRY (models/attention_flax.py:1589-1597), after which
``attention: hip_flash`` in any Wan / Flux / LTX config reaches the MI355X kernel through
the unchanged `_apply_attention` (models/attention_flax.py:1965-1966).

Nothing here runs at import time: jax, jaxlib's FFI headers and maxdiffusion are absent from
the build image, so this module is exercised only where they exist.
"""
from __future__ import annotations

import ctypes
import os

from .build import FFI_LIB_PATH, build_ffi_library

FFI_TARGETS = {
    "mdattn_fwd_bf16": "MdattnFwdBf16",
    "mdattn_fwd_bf16_bias": "MdattnFwdBf16Bias",
    "mdattn_bwd_bf16": "MdattnBwdBf16",
    "mdattn_norm_rope_fullrow": "MdattnNormRopeFullrow",
    "mdattn_norm_rope_perhead": "MdattnNormRopePerhead",
    "mdattn_norm_rope_rows": "MdattnNormRopeRows",
    "mdattn_merge": "MdattnMerge",
    "mdattn_fwd_bf16_merge": "MdattnFwdBf16Merge",
}

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


def hip_flash_attention(q, k, v, scale: float, layout: int, keep_mask=None):
  """q [B,Sq,H,D] (layout 0) or [B,H,Sq,D] (layout 1) bf16 -> (out [B,Sq,H,D] bf16, lse [B,H,Sq] f32).

  keep_mask: optional [B,Skv] bool; masked keys are excluded (the bias is built with jnp: a [B,Skv] select)."""
  jax, jnp = _require_jax()
  if layout == 0:
    b, sq, h, d = q.shape
  else:
    b, h, sq, d = q.shape
  call = jax.ffi.ffi_call(
      "mdattn_fwd_bf16",
      (jax.ShapeDtypeStruct((b, sq, h, d), jnp.bfloat16), jax.ShapeDtypeStruct((b, h, sq), jnp.float32)),
      vmap_method="sequential",
  )
  import numpy as np

  if keep_mask is not None:
    skv = k.shape[1] if layout == 0 else k.shape[2]
    pad = (-skv) % 32
    bias = jnp.where(keep_mask, 0.0, -jnp.inf).astype(jnp.float32)
    bias = jnp.pad(bias, ((0, 0), (0, pad)), constant_values=-jnp.inf)
    call = jax.ffi.ffi_call(
        "mdattn_fwd_bf16_bias",
        (jax.ShapeDtypeStruct((b, sq, h, d), jnp.bfloat16), jax.ShapeDtypeStruct((b, h, sq), jnp.float32)),
        vmap_method="sequential",
    )
    return call(q, k, v, bias, scale=np.float32(scale), layout=np.int64(layout))
  return call(q, k, v, scale=np.float32(scale), layout=np.int64(layout))


def hip_ring_step(q, k_chunk, v_chunk, o_run, lse_run, scale: float, layout: int = 0):
  """One ring hop in one custom call: attention of q against the visiting K/V chunk merged into the carry
  (o_run f32 [B,Sq,H,D], lse_run f32 [B,H,Sq]; start from zeros and -1e30).  The body of the scan step in
  kernels/splash_attention/ring_attention_kernel.py:1045-1073; the carry is donated and updated in place."""
  jax, jnp = _require_jax()
  import numpy as np

  call = jax.ffi.ffi_call(
      "mdattn_fwd_bf16_merge",
      (jax.ShapeDtypeStruct(o_run.shape, jnp.float32), jax.ShapeDtypeStruct(lse_run.shape, jnp.float32)),
      input_output_aliases={3: 0, 4: 1},
      vmap_method="sequential",
  )
  return call(q, k_chunk, v_chunk, o_run, lse_run, scale=np.float32(scale), layout=np.int64(layout))


def hip_flash_attention_vjp(q, k, v, scale: float):
  """Differentiable attention on [B,S,H,D] bf16 arrays: jax.custom_vjp around the forward and backward custom calls
  (what kernels/splash_attention/splash_attention_kernel.py:1277-1600 does for the Pallas kernel)."""
  jax, jnp = _require_jax()
  import numpy as np

  @jax.custom_vjp
  def attn(q, k, v):
    return hip_flash_attention(q, k, v, scale, 0)[0]

  def fwd(q, k, v):
    out, lse = hip_flash_attention(q, k, v, scale, 0)
    return out, (q, k, v, out, lse)

  def bwd(res, dout):
    q, k, v, out, lse = res
    b, sq, h, d = q.shape
    nws = 2 * b * h * ((sq + 31) // 32 * 32)  # mdattn_bwd_workspace_floats
    call = jax.ffi.ffi_call(
        "mdattn_bwd_bf16",
        (jax.ShapeDtypeStruct(q.shape, jnp.bfloat16), jax.ShapeDtypeStruct(k.shape, jnp.bfloat16),
         jax.ShapeDtypeStruct(v.shape, jnp.bfloat16), jax.ShapeDtypeStruct((nws,), jnp.float32)),
        vmap_method="sequential",
    )
    dq, dk, dv, _ = call(q, k, v, out, dout.astype(jnp.bfloat16), lse, scale=np.float32(scale))
    return dq, dk, dv

  attn.defvjp(fwd, bwd)
  return attn(q, k, v)


def hip_norm_rope_fullrow(q, k, wq, wk, cos, sin, heads: int, eps: float = 1e-6, q_mul: float = 1.0):
  """q, k [B,S,H*D] bf16; cos/sin f32 [S,D/2] or None -> (q_out, k_out) [B,S,H,D] bf16.  `q_mul` is multiplied into
  q_out before its rounding: D**-0.5 * log2(e) here and scale = ln 2 in hip_flash_attention carry the softmax scale
  in the prologue."""
  jax, jnp = _require_jax()
  import numpy as np

  b, s, n = q.shape
  d = n // heads
  rope = cos is not None
  if not rope:
    cos = sin = jnp.zeros((1, 1), jnp.float32)
  out = jax.ShapeDtypeStruct((b, s, heads, d), jnp.bfloat16)
  call = jax.ffi.ffi_call("mdattn_norm_rope_fullrow", (out, out), vmap_method="sequential")
  return call(q, k, wq, wk, cos, sin, eps=np.float32(eps), q_mul=np.float32(q_mul), heads=np.int64(heads), rope=np.int64(rope))


def hip_norm_rope_ltx2(query, key, norm_q_scale, norm_k_scale, heads: int, rotary_emb=None, k_rotary_emb=None,
                       rope_type: str = "interleaved", is_self_attention: bool = True, eps: float = 1e-6):
  """Fused prologue of LTX2Attention.__call__ (models/ltx2/attention_ltx2.py:556-585): see attention_op.hip_norm_rope_ltx2.
  query/key [B,S,H*D] -> bf16 [B,S,H,D]; tables (cos, sin) as LTX2RotaryPosEmbed returns them."""
  jax, jnp = _require_jax()
  import numpy as np

  if rope_type not in ("interleaved", "split"):
    raise ValueError(f"{rope_type=} not supported. Choose between 'interleaved' and 'split'.")
  q_tab = rotary_emb
  k_tab = k_rotary_emb if k_rotary_emb is not None else (rotary_emb if is_self_attention else None)
  if rotary_emb is None:
    q_tab = k_tab = None
  dummy = jnp.zeros((1,), jnp.float32)

  def run(x, scale, tab):
    b, s, n = x.shape
    out = jax.ShapeDtypeStruct((b, s, heads, n // heads), jnp.bfloat16)
    mode = 0 if tab is None else (1 if rope_type == "interleaved" else 2)
    cos, sin = (dummy, dummy) if tab is None else (tab[0].astype(jnp.float32), tab[1].astype(jnp.float32))
    call = jax.ffi.ffi_call("mdattn_norm_rope_rows", out, vmap_method="sequential")
    return call(x, scale.astype(jnp.float32), cos, sin, eps=np.float32(eps), heads=np.int64(heads), mode=np.int64(mode))

  return run(query, norm_q_scale, q_tab), (run(key, norm_k_scale, k_tab) if key is not None else None)


def hip_flash_kernel(q, k, v, context):
  """The KERNEL_REGISTRY entry: fn(q, k, v, context) -> [B, Sq, H*D] in q's dtype."""
  _, jnp = _require_jax()
  if context.get("is_causal"):
    raise NotImplementedError("hip_flash is non-causal")
  heads = context["heads"]
  if q.ndim == 3:
    b, sq, n = q.shape
    d = n // heads
    q4 = q.reshape(b, sq, heads, d)
    k4 = k.reshape(b, k.shape[1], heads, d)
    v4 = v.reshape(b, v.shape[1], heads, d)
    layout = 0
  else:
    q4, k4, v4, layout = q, k, v, 1
  dt = q.dtype
  out, _ = hip_flash_attention(q4.astype(jnp.bfloat16), k4.astype(jnp.bfloat16), v4.astype(jnp.bfloat16), context["scale"], layout,
                               keep_mask=context.get("attention_mask"))
  b, sq, h, d = out.shape
  return out.reshape(b, sq, h * d).astype(dt)


def install():
  """Idempotent: FFI targets + maxdiffusion KERNEL_REGISTRY['hip_flash']."""
  global _installed
  if _installed:
    return
  register_ffi_targets()
  from maxdiffusion.models import attention_flax  # type: ignore

  attention_flax.register_kernel("hip_flash")(hip_flash_kernel)
  _installed = True
