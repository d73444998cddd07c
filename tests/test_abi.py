"""The C-ABI library loads on a machine without a GPU, exports every symbol include/mdattn.h
declares, and rejects malformed requests on the host (no kernel launch, no GPU needed)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mdattn.h")


def declared_symbols():
  text = open(HEADER).read()
  text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
  return sorted(set(re.findall(r"\b(mdattn_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
  assert declared_symbols() == sorted([
      "mdattn_version", "mdattn_strerror", "mdattn_norm_rope_fullrow", "mdattn_norm_rope_perhead", "mdattn_fwd_bf16",
      "mdattn_quant_e4m3", "mdattn_fwd_fp8", "mdattn_merge", "mdattn_finalize", "mdattn_fwd_bf16_bias", "mdattn_key_mask_bias", "mdattn_norm_rope_rows", "mdattn_bwd_bf16", "mdattn_bwd_workspace_floats",
      "mdattn_fwd_bf16_merge", "mdattn_bwd_bf16_static", "mdattn_bwd_static_max_floats",
      "mdattn_build_id", "mdattn_set_fwd_schedule", "mdattn_norm_rope_qkv", "mdattn_bwd_bf16_bias", "mdattn_fwd_fp8_bias",
      "mdattn_norm_rope_bwd_workspace_floats", "mdattn_norm_rope_fullrow_bwd", "mdattn_norm_rope_perhead_bwd", "mdattn_norm_rope_rows_bwd",
  ])


def test_library_exports_every_declared_symbol(lib):
  from maxdiffusion_amd import _lib

  for name in declared_symbols():
    assert hasattr(lib, name), f"libmdattn.so does not export {name}"
    assert name in _lib.SIGNATURES, f"ctypes binding lacks {name}"
  assert sorted(_lib.SIGNATURES) == declared_symbols()


def test_version_and_strerror(lib):
  text = open(HEADER).read()
  want = int(re.search(r"#define MDATTN_VERSION (\d+)", text).group(1))
  assert lib.mdattn_version() == want
  for code in (0, -1, -2, -3, -4, -5, -99):
    assert len(lib.mdattn_strerror(code)) > 0
  assert lib.mdattn_strerror(0) == b"ok"


def test_build_id_and_schedule_hook(lib):
  from maxdiffusion_amd import _lib, build

  assert lib.mdattn_build_id().decode() == build.source_id()  # the library in the tree was built from the tree
  assert lib.mdattn_set_fwd_schedule(3) == 0 and lib.mdattn_set_fwd_schedule(0) == 3
  assert lib.mdattn_set_fwd_schedule(99) == _lib.E_BADARG and lib.mdattn_set_fwd_schedule(-1) == _lib.E_BADARG
  assert lib.mdattn_set_fwd_schedule(0) == 0


def test_header_is_plain_c_and_a_c_program_links_against_the_library(lib, tmp_path):
  """The boundary is a C ABI: include/mdattn.h compiles as C99 and as C++11 with the host compilers (no HIP, no torch
  type in it), and a C program that calls the host-only entry points links against libmdattn.so and runs."""
  import shutil
  import subprocess

  from maxdiffusion_amd import build

  gcc, gxx = shutil.which("gcc"), shutil.which("g++")
  if not gcc or not gxx:
    pytest.skip("no host C / C++ compiler")
  inc = os.path.dirname(HEADER)
  src = tmp_path / "abi.c"
  src.write_text(
      '#include <stdio.h>\n#include <string.h>\n#include "mdattn.h"\n'
      "int main(void) {\n"
      "  mdattn_strides s; memset(&s, 0, sizeof s);\n"
      "  if (mdattn_version() != MDATTN_VERSION) return 2;\n"
      '  if (strcmp(mdattn_strerror(MDATTN_OK), "ok") != 0) return 3;\n'
      "  /* a null operand is refused on the host: no kernel is launched */\n"
      "  if (mdattn_fwd_bf16(0, 0, 0, 0, 0, 0, 1, 1, 1, 1, 128, &s, &s, &s, &s, 1.0f) != MDATTN_E_BADARG) return 4;\n"
      '  printf("%s\\n", mdattn_build_id());\n'
      "  return 0;\n}\n")
  subprocess.run([gcc, "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-fsyntax-only", f"-I{inc}", str(src)], check=True)
  cxx = tmp_path / "abi.cc"
  cxx.write_text('#include "mdattn.h"\nint main() { return mdattn_version() == MDATTN_VERSION ? 0 : 1; }\n')
  subprocess.run([gxx, "-std=c++11", "-Wall", "-Wextra", "-pedantic", "-Werror", "-fsyntax-only", f"-I{inc}", str(cxx)], check=True)
  exe = tmp_path / "abi"
  libdir = os.path.dirname(build.LIB_PATH)
  subprocess.run([gcc, "-std=c99", f"-I{inc}", str(src), "-o", str(exe), f"-L{libdir}", "-l:libmdattn.so", f"-Wl,-rpath,{libdir}"], check=True)
  r = subprocess.run([str(exe)], capture_output=True, text=True)
  assert r.returncode == 0, (r.returncode, r.stderr)
  assert r.stdout.strip() == build.source_id()


def test_stale_library_is_refused(monkeypatch):
  from maxdiffusion_amd import _lib, build

  monkeypatch.setattr(_lib, "_lib", None)
  monkeypatch.setattr(build, "source_id", lambda: "0123456789abcdef")
  with pytest.raises(RuntimeError, match="built from other sources"):
    _lib.load()
  assert not build.library_is_current()


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
  from maxdiffusion_amd import _lib

  monkeypatch.setattr(_lib, "_lib", None)
  monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libmdattn.so"))
  with pytest.raises(RuntimeError, match="no non-HIP fallback"):
    _lib.load()


def _st(b, s, h):
  from maxdiffusion_amd._lib import Strides

  return ctypes.byref(Strides(b, s, h))


def test_bad_arguments_are_rejected_on_the_host(lib):
  from maxdiffusion_amd import _lib

  P = ctypes.c_void_p
  fake = P(0x1000)  # aligned, never dereferenced: every call below must fail validation first
  odd = P(0x1004)
  st = _st(128 * 8 * 4, 128 * 4, 128)
  f = lib.mdattn_fwd_bf16
  assert f(None, None, fake, fake, fake, None, 1, 4, 8, 8, 128, st, st, st, st, 0.1) == _lib.E_BADARG
  assert f(None, fake, fake, fake, fake, None, 1, 4, 0, 8, 128, st, st, st, st, 0.1) == _lib.E_BADARG
  assert f(None, fake, fake, fake, fake, None, 1, 4, 8, 8, 128, st, st, st, st, 0.0) == _lib.E_BADARG
  assert f(None, fake, fake, fake, fake, None, 1, 4, 8, 8, 128, st, st, st, st, float("nan")) == _lib.E_BADARG
  assert f(None, fake, fake, fake, fake, None, 1, 4, 8, 8, 32, st, st, st, st, 0.1) == _lib.E_UNSUPPORTED
  assert f(None, odd, fake, fake, fake, None, 1, 4, 8, 8, 128, st, st, st, st, 0.1) == _lib.E_ALIGN
  assert f(None, fake, fake, fake, fake, None, 1, 4, 8, 8, 128, _st(0, 516, 129), st, st, st, 0.1) == _lib.E_ALIGN
  assert f(None, fake, fake, fake, fake, None, 1, 4, 8, 8, 128, None, st, st, st, 0.1) == _lib.E_BADARG

  g = lib.mdattn_norm_rope_fullrow
  assert g(None, None, None, fake, None, fake, None, None, None, 1, 8, 4, 128, 1e-6, 1.0, 0, 512, st) == _lib.E_BADARG
  assert g(None, fake, fake, fake, None, fake, fake, None, None, 1, 8, 4, 128, 1e-6, 1.0, 0, 512, st) == _lib.E_BADARG  # k_in without k_out
  assert g(None, fake, None, fake, None, fake, None, fake, None, 1, 8, 4, 128, 1e-6, 1.0, 0, 512, st) == _lib.E_BADARG  # cos without sin
  assert g(None, fake, None, fake, None, fake, None, None, None, 1, 8, 80, 128, 1e-6, 1.0, 0, 10240, st) == _lib.E_UNSUPPORTED  # H*D > 8192
  assert g(None, fake, None, fake, None, fake, None, None, None, 1, 8, 4, 128, 1e-6, 1.0, 0, 100, st) == _lib.E_BADARG  # row stride < H*D
  assert g(None, fake, None, odd, None, fake, None, None, None, 1, 8, 4, 128, 1e-6, 1.0, 0, 512, st) == _lib.E_ALIGN
  assert g(None, fake, None, fake, None, fake, None, None, None, 1, 8, 4, 128, 1e-6, 0.0, 0, 512, st) == _lib.E_BADARG  # q_mul must be > 0

  p = lib.mdattn_norm_rope_perhead
  assert p(None, fake, None, fake, None, fake, None, None, None, 0, None, None, 1, 8, 4, 96, 1e-6, 1.0, st, st) == _lib.E_UNSUPPORTED
  assert p(None, fake, None, fake, None, fake, None, None, None, 9, None, None, 1, 8, 4, 128, 1e-6, 1.0, st, st) == _lib.E_BADARG  # n_txt > S
  assert p(None, fake, None, fake, None, None, None, None, None, 0, None, None, 1, 8, 4, 128, 1e-6, 1.0, st, st) == _lib.E_BADARG

  m = lib.mdattn_merge
  assert m(None, fake, fake, fake, None, 0, 1, 4, 8, 128, st, st) == _lib.E_BADARG
  assert m(None, fake, fake, fake, fake, 0, 1, 4, 8, 100, st, st) == _lib.E_UNSUPPORTED
  assert m(None, fake, P(0x1002), fake, fake, 0, 1, 4, 8, 128, st, st) == _lib.E_ALIGN

  fm = lib.mdattn_fwd_bf16_merge
  assert fm(None, fake, fake, fake, None, fake, 1, 4, 8, 8, 128, st, st, st, st, 0.1) == _lib.E_BADARG  # no carry
  assert fm(None, fake, fake, fake, fake, None, 1, 4, 8, 8, 128, st, st, st, st, 0.1) == _lib.E_BADARG  # no lse carry
  assert fm(None, fake, fake, fake, odd, fake, 1, 4, 8, 8, 128, st, st, st, st, 0.1) == _lib.E_ALIGN
  assert fm(None, fake, fake, fake, fake, P(0x1002), 1, 4, 8, 8, 128, st, st, st, st, 0.1) == _lib.E_ALIGN
  assert fm(None, fake, fake, fake, fake, fake, 1, 4, 8, 8, 32, st, st, st, st, 0.1) == _lib.E_UNSUPPORTED
  assert fm(None, fake, fake, fake, fake, fake, 1, 4, 8, 0, 128, st, st, st, st, 0.1) == _lib.E_BADARG

  assert lib.mdattn_finalize(None, fake, fake, 12) == _lib.E_UNSUPPORTED
  assert lib.mdattn_finalize(None, fake, None, 16) == _lib.E_BADARG
  assert lib.mdattn_quant_e4m3(None, fake, fake, fake, 24, 1.0, 0) == _lib.E_UNSUPPORTED
  assert lib.mdattn_quant_e4m3(None, fake, fake, None, 32, 1.0, 0) == _lib.E_BADARG
  assert lib.mdattn_quant_e4m3(None, fake, fake, fake, 32, 0.0, 1) == _lib.E_BADARG
  with pytest.raises(_lib.MdattnError, match="mdattn error -1"):
    _lib.check(_lib.E_BADARG, "unit test")
