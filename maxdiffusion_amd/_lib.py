"""ctypes binding of libmdattn.so (the C ABI declared in include/mdattn.h).

There is no fallback: when the library is missing or a call fails this module raises.
"""
from __future__ import annotations

import ctypes
import os

from .build import LIB_PATH

E_OK, E_BADARG, E_UNSUPPORTED, E_ALIGN, E_LAUNCH, E_TOOBIG = 0, -1, -2, -3, -4, -5


class Strides(ctypes.Structure):
  _fields_ = [("batch", ctypes.c_int64), ("seq", ctypes.c_int64), ("head", ctypes.c_int64)]


class MdattnError(RuntimeError):

  def __init__(self, code: int, where: str, text: str):
    super().__init__(f"{where}: mdattn error {code}: {text}")
    self.code = code


_P = ctypes.c_void_p
_I = ctypes.c_int
_L = ctypes.c_int64
_F = ctypes.c_float
_S = ctypes.POINTER(Strides)

# symbol -> argtypes; every symbol include/mdattn.h declares
SIGNATURES = {
    "mdattn_version": ([], _I),
    "mdattn_strerror": ([_I], ctypes.c_char_p),
    "mdattn_build_id": ([], ctypes.c_char_p),
    "mdattn_set_fwd_schedule": ([_I], _I),
    "mdattn_norm_rope_fullrow": ([_P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _F, _F, _L, _L, _S], _I),
    "mdattn_norm_rope_qkv": ([_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _F, _F, _L, _L, _S], _I),
    "mdattn_norm_rope_perhead": ([_P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _P, _P, _I, _I, _I, _I, _F, _F, _S, _S], _I),
    "mdattn_norm_rope_rows": ([_P, _P, _I, _P, _P, _P, _P, _I, _I, _I, _I, _I, _F, _L, _L, _S], _I),
    "mdattn_norm_rope_bwd_workspace_floats": ([_L, _L], _L),
    "mdattn_norm_rope_fullrow_bwd": ([_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _F, _F, _L, _L, _L, _L, _S, _P, _L], _I),
    "mdattn_norm_rope_perhead_bwd": ([_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _F, _F, _S, _S, _S, _P, _L], _I),
    "mdattn_norm_rope_rows_bwd": ([_P, _P, _I, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _F, _L, _L, _L, _L, _S, _P, _L], _I),
    "mdattn_fwd_bf16": ([_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _S, _S, _S, _S, _F], _I),
    "mdattn_fwd_bf16_bias": ([_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _S, _S, _S, _S, _F, _P, _L], _I),
    "mdattn_key_mask_bias": ([_P, _P, _P, _I, _I, _L, _F], _I),
    "mdattn_bwd_workspace_floats": ([_I, _I, _I], _L),
    "mdattn_bwd_bf16": ([_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _L, _I, _I, _I, _I, _I, _S, _S, _S, _S, _F], _I),
    "mdattn_bwd_bf16_bias": ([_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _L, _I, _I, _I, _I, _I, _S, _S, _S, _S, _F, _P, _L], _I),
    "mdattn_bwd_static_max_floats": ([], _L),
    "mdattn_bwd_bf16_static": ([_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _S, _S, _S, _S, _F], _I),
    "mdattn_quant_e4m3": ([_P, _P, _P, _P, _L, _F, _I], _I),
    "mdattn_fwd_fp8": ([_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _S, _S, _S, _S, _F, _P, _P, _P, _I], _I),
    "mdattn_fwd_fp8_bias": ([_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _S, _S, _S, _S, _F, _P, _P, _P, _P, _L], _I),
    "mdattn_merge": ([_P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _S, _S], _I),
    "mdattn_fwd_bf16_merge": ([_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _S, _S, _S, _S, _F], _I),
    "mdattn_finalize": ([_P, _P, _P, _L], _I),
}

_lib = None


def load() -> ctypes.CDLL:
  """Load libmdattn.so once; raise if it has not been built."""
  global _lib
  if _lib is None:
    if not os.path.exists(LIB_PATH):
      raise RuntimeError(
          f"{LIB_PATH} is missing: build it with `python -m maxdiffusion_amd.build` "
          "(there is no non-HIP fallback for this path)")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (argtypes, restype) in SIGNATURES.items():
      fn = getattr(lib, name)
      fn.argtypes = argtypes
      fn.restype = restype
    from . import build

    if os.path.isdir(build.CSRC) and lib.mdattn_build_id().decode() != build.source_id():
      raise RuntimeError(
          f"{LIB_PATH} was built from other sources than the ones in {build.CSRC} (build id "
          f"{lib.mdattn_build_id().decode()}, sources {build.source_id()}): rebuild with `python -m maxdiffusion_amd.build`")
    _lib = lib
  return _lib


def strerror(code: int) -> str:
  return load().mdattn_strerror(code).decode()


def check(code: int, where: str) -> None:
  if code != E_OK:
    raise MdattnError(code, where, strerror(code))
