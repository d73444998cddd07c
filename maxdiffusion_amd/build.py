"""Builds libmdattn.so (hand-written HIP for gfx950) in-tree with hipcc.

`python -m maxdiffusion_amd.build` or `build_library()`.  hipcc cross-compiles without a GPU.
The XLA-FFI shim (csrc/ffi/mdattn_ffi.cc) is built only where jaxlib's FFI headers exist.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
INCLUDE = os.path.join(os.path.dirname(PKG_DIR), "include")
LIB_PATH = os.path.join(PKG_DIR, "libmdattn.so")
FFI_LIB_PATH = os.path.join(PKG_DIR, "libmdattn_ffi.so")

SOURCES = ["mdattn_api.hip", "norm_rope.hip", "norm_rope_bwd.hip", "attn_fwd_bf16.hip", "attn_fwd_fp8.hip", "attn_bwd_bf16.hip", "merge_quant.hip", "probes.hip",
           # the bodies of the XLA custom-call handlers on plain structs (no XLA header): part of the library
           os.path.join("ffi", "mdattn_marshal.cc")]

# -packed-fp32-ops: keep the compiler from forming v_pk_{add,mul,fma}_f32 out of scalar float code.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # MFMA results that the vector ALU reads next (attention logits) stay in architectural VGPRs
    # instead of bouncing through AGPRs with v_accvgpr_read/write
    "-mllvm", "-amdgpu-mfma-vgpr-form",
    "-Wno-unused-command-line-argument",
    # the direct global->LDS loads are inline assembly that writes M0 and lists it as clobbered; clang remarks that
    # M0 is a reserved register.  The statement really does overwrite it, so the compiler is told.
    "-Wno-inline-asm",
]


def _hipcc() -> str:
  exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
  if not os.path.exists(exe):
    raise RuntimeError("hipcc not found: libmdattn.so cannot be built on this machine")
  return exe


def _filter(stderr: str) -> str:
  """hipcc's stderr without the resource-usage remarks (and their source excerpts) and the host pass's complaint
  about the target feature it does not know."""
  import re

  keep, in_remark = [], False
  for l in stderr.splitlines():
    if "remark:" in l:
      in_remark = True
      continue
    if in_remark and re.match(r"^\s*(\d+\s*)?\|", l):
      continue
    in_remark = False
    if "packed-fp32-ops" in l or "-Rpass-analysis" in l or re.match(r"^\d+ (warning|remark)s? generated", l):
      continue
    keep.append(l)
  return "\n".join(keep)


def _resource_table(stderr: str) -> list[tuple[str, dict]]:
  """Kernel name -> registers, scratch and occupancy from hipcc's kernel-resource-usage remarks."""
  import re

  rows, cur = [], None
  for line in stderr.splitlines():
    m = re.search(r"remark: Function Name: (\S+)", line)
    if m:
      cur = {}
      rows.append((m.group(1), cur))
      continue
    m = re.search(r"remark:\s+(VGPRs|AGPRs|ScratchSize \[bytes/lane\]|Occupancy \[waves/SIMD\]|LDS Size \[bytes/block\]): (\d+)", line)
    if m and cur is not None:
      cur[m.group(1).split(" ")[0]] = int(m.group(2))
  return rows


def _demangled(names: list[str]) -> dict[str, str]:
  exe = shutil.which("llvm-cxxfilt") or shutil.which("c++filt") or "/opt/rocm/lib/llvm/bin/llvm-cxxfilt"
  if not names or not os.path.exists(exe):
    return {n: n for n in names}
  out = subprocess.run([exe, *names], capture_output=True, text=True).stdout.splitlines()
  return dict(zip(names, out)) if len(out) == len(names) else {n: n for n in names}


def source_id() -> str:
  """Hash of everything libmdattn.so is compiled from (sources, headers, flags); compiled into the library as
  mdattn_build_id() so that a library built from other sources than the ones beside it is recognised."""
  import hashlib

  h = hashlib.sha256(" ".join(HIPCC_FLAGS).encode())
  files = [os.path.join(CSRC, f) for f in sorted(os.listdir(CSRC)) if f.endswith((".hip", ".h"))]
  for path in files + [os.path.join(CSRC, "ffi", "mdattn_marshal.cc"), os.path.join(INCLUDE, "mdattn.h"), os.path.join(INCLUDE, "mdattn_marshal.h")]:
    h.update(os.path.basename(path).encode())
    with open(path, "rb") as f:
      h.update(f.read())
  return h.hexdigest()[:16]


def built_library_id(path: str | None = None) -> str | None:
  """The source id a built library carries, read from the file (nothing is loaded), or None."""
  path = path or LIB_PATH
  marker = b"mdattn-build-id:"
  try:
    with open(path, "rb") as f:
      data = f.read()
  except OSError:
    return None
  i = data.find(marker)
  if i < 0:
    return None
  j = data.find(b"\0", i)
  return data[i + len(marker):j].decode(errors="replace")


def library_is_current() -> bool:
  """True when libmdattn.so exists and was built from the sources in this tree."""
  return built_library_id() == source_id()


def ensure_built(verbose: bool = True) -> str:
  """What tests, smoke() and bench.py call: loads what is built, builds only when nothing is built or the library
  was compiled from other sources than the ones in the tree."""
  if not library_is_current():
    build_library(verbose)
  return LIB_PATH


def build_library(verbose: bool = True) -> str:
  """Compile every HIP source into maxdiffusion_amd/libmdattn.so.  Always recompiles."""
  # Linked under another name and moved into place: a process that has the previous library mapped keeps its own
  # file, and a later dlopen of the path finds the new one instead of the handle it already holds.
  tmp = LIB_PATH + f".{os.getpid()}.tmp"
  cmd = [_hipcc(), *HIPCC_FLAGS, "-Rpass-analysis=kernel-resource-usage", f'-DMDATTN_BUILD_ID="{source_id()}"',
         f"-I{INCLUDE}", f"-I{CSRC}", "-o", tmp, *[os.path.join(CSRC, s) for s in SOURCES]]
  if verbose:
    print("[maxdiffusion_amd.build]", " ".join(cmd), flush=True)
  r = subprocess.run(cmd, capture_output=True, text=True)
  err = _filter(r.stderr)
  if r.returncode != 0:
    if os.path.exists(tmp):
      os.remove(tmp)
    raise RuntimeError(f"hipcc failed ({r.returncode}):\n{r.stdout}\n{err}")
  os.replace(tmp, LIB_PATH)
  if verbose and err.strip():
    print(err, file=sys.stderr)
  if verbose:  # registers, spills and occupancy of every kernel: a spill in a hot loop shows here, not in a test
    rows = _resource_table(r.stderr)
    names = _demangled([n for n, _ in rows])
    for n, d in rows:
      short = names[n].replace("(anonymous namespace)::", "").split("(")[0].replace("void ", "").replace("mdattn::", "")
      spill = "  <-- spills" if d.get("ScratchSize", 0) else ""
      print(f"[maxdiffusion_amd.build]   {short:<46} vgpr {d.get('VGPRs', 0):>3} agpr {d.get('AGPRs', 0):>3} "
            f"scratch {d.get('ScratchSize', 0):>3} B  lds {d.get('LDS', 0):>6} B  waves/SIMD {d.get('Occupancy', 0)}{spill}", flush=True)
  return LIB_PATH


def xla_ffi_include_dir() -> str | None:
  try:
    import jax.ffi  # type: ignore

    return jax.ffi.include_dir()
  except Exception:  # jax / jaxlib absent: the FFI shim is not buildable here
    return None


def build_ffi_library(verbose: bool = True) -> str | None:
  """Compile the XLA-FFI handlers against jaxlib's headers; returns None when they are absent."""
  inc = xla_ffi_include_dir()
  if inc is None:
    return None
  cmd = [_hipcc(), *HIPCC_FLAGS, f"-I{INCLUDE}", f"-I{inc}", "-o", FFI_LIB_PATH,
         os.path.join(CSRC, "ffi", "mdattn_ffi.cc"), f"-L{PKG_DIR}", "-lmdattn", f"-Wl,-rpath,{PKG_DIR}"]
  if verbose:
    print("[maxdiffusion_amd.build]", " ".join(cmd), flush=True)
  r = subprocess.run(cmd, capture_output=True, text=True)
  if r.returncode != 0:
    raise RuntimeError(f"hipcc failed on the FFI shim ({r.returncode}):\n{_filter(r.stderr)}")
  return FFI_LIB_PATH


if __name__ == "__main__":
  print(build_library())
  print(build_ffi_library() or "XLA FFI headers not found: libmdattn_ffi.so skipped")
