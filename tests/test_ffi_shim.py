"""The JAX boundary without JAX: (1) the XLA-FFI shim type-checks against a stand-in for jaxlib's header and its bind
lines, the marshalling layer (include/mdattn_marshal.h, part of libmdattn.so) and the Python wrappers of jax_plugin.py
agree target by target; (2) every compute entry point of include/mdattn.h has exactly one custom-call target;
(3) the marshalling layer rejects wrong ranks, dtypes, shapes and missing donations on the host, naming the argument.
The GPU half (handler bodies against the torch-side operators, bit for bit) is tests/test_gpu_ffi_marshal.py."""
import ctypes
import os
import re
import shutil
import subprocess
import sys
import types

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SHIM = os.path.join(ROOT, "maxdiffusion_amd", "csrc", "ffi", "mdattn_ffi.cc")
STUB = os.path.join(ROOT, "tests", "xla_ffi_stub")
INCLUDE = os.path.join(ROOT, "include")


def _entry_points(header):
  text = re.sub(r"/\*.*?\*/", "", open(os.path.join(INCLUDE, header)).read(), flags=re.S)
  return sorted(set(re.findall(r"\b(mdattn_[a-z0-9_]+)\s*\(", text)))


def _bind_lines():
  """handler symbol -> (impl function, #Arg, #Ret, [(attr type, attr name), ...]) parsed from the shim."""
  text = open(SHIM).read()
  out = {}
  for m in re.finditer(r"XLA_FFI_DEFINE_HANDLER_SYMBOL\((\w+),\s*(\w+),\s*(.*?)\);", text, flags=re.S):
    sym, impl, bind = m.groups()
    out[sym] = (impl, len(re.findall(r"\.Arg<", bind)), len(re.findall(r"\.Ret<", bind)), re.findall(r'\.Attr<(\w+)>\("(\w+)"\)', bind))
  return out


def _hipcc():
  exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
  if not os.path.exists(exe):
    pytest.skip("hipcc not found")
  return exe


def test_shim_type_checks_against_the_header_stand_in(tmp_path):
  cmd = [_hipcc(), "-std=c++17", "-fsyntax-only", "-Wno-unused-command-line-argument", f"-I{INCLUDE}", f"-I{STUB}"]
  r = subprocess.run(cmd + [SHIM], capture_output=True, text=True)
  assert r.returncode == 0, r.stderr
  # the check is real: a bind line that drifts from its handler (one attribute dropped) no longer compiles
  broken = tmp_path / "mdattn_ffi_broken.cc"
  text = open(SHIM).read()
  assert text.count('.Attr<int64_t>("softmax_mode")') == 1
  broken.write_text(text.replace('.Attr<int64_t>("softmax_mode")', ""))
  r = subprocess.run(cmd + [str(broken)], capture_output=True, text=True)
  assert r.returncode != 0 and "MdattnFwdFp8" in r.stderr
  # ... and so does a call into the marshalling layer with a wrong argument list
  broken.write_text(text.replace("mdattn_xla_finalize(s, &a, &o, m.text, sizeof m.text)", "mdattn_xla_finalize(s, &a, &o, 1.0f, m.text, sizeof m.text)"))
  r = subprocess.run(cmd + [str(broken)], capture_output=True, text=True)
  assert r.returncode != 0


def test_every_compute_entry_point_has_exactly_one_custom_call_target(lib):
  from maxdiffusion_amd import jax_plugin

  declared = _entry_points("mdattn.h")
  assert sorted(set(declared) - set(jax_plugin.HOST_ONLY)) == sorted(jax_plugin.FFI_TARGETS)
  assert set(jax_plugin.HOST_ONLY) <= set(declared)
  binds = _bind_lines()
  assert sorted(binds) == sorted(jax_plugin.FFI_TARGETS.values())
  marshal = _entry_points("mdattn_marshal.h")
  assert marshal == sorted("mdattn_xla_" + t[len("mdattn_"):] for t in jax_plugin.FFI_TARGETS)
  shim = open(SHIM).read()
  for target in jax_plugin.FFI_TARGETS:
    fn = "mdattn_xla_" + target[len("mdattn_"):]
    assert hasattr(lib, fn), f"libmdattn.so does not export {fn}"
    assert shim.count(fn + "(") == 1, f"the shim must call {fn} exactly once"


# ----------------------------------------------------------------------------- jax_plugin against the bind lines
class _FakeArray:
  """Just enough of a jax Array for the wrappers: shape, dtype, ndim, astype, reshape, scalar multiply."""

  def __init__(self, shape, dtype):
    self.shape, self.dtype = tuple(shape), dtype

  ndim = property(lambda self: len(self.shape))

  def astype(self, dtype):
    return _FakeArray(self.shape, dtype)

  def reshape(self, *shape):
    shape = shape[0] if len(shape) == 1 and isinstance(shape[0], (tuple, list)) else shape
    assert int(np.prod(shape)) == int(np.prod(self.shape)), (shape, self.shape)
    return _FakeArray(shape, self.dtype)

  def __mul__(self, other):
    return _FakeArray(self.shape, self.dtype)

  def transpose(self, *axes):
    return _FakeArray(tuple(self.shape[a] for a in axes), self.dtype)

  def __getitem__(self, idx):  # slicing of the last axis only: x[:, :, a:b], x[a:b]
    sl = idx[-1] if isinstance(idx, tuple) else idx
    a, b = sl.start or 0, self.shape[-1] if sl.stop is None else sl.stop
    return _FakeArray(self.shape[:-1] + (b - a,), self.dtype)

  def sum(self, axis):
    axes = (axis,) if isinstance(axis, int) else tuple(axis)
    return _FakeArray(tuple(n for i, n in enumerate(self.shape) if i not in axes), self.dtype)


@pytest.fixture
def fake_jax(monkeypatch):
  """A recording stand-in for jax / jax.ffi / jax.numpy: every ffi_call is logged as (target, result specs, aliases,
  operands, attributes) and returns arrays of the declared result shapes."""
  calls = []
  jax = types.ModuleType("jax")
  jnp = types.ModuleType("jax.numpy")
  ffi = types.ModuleType("jax.ffi")
  for name in ("bfloat16", "float32", "bool_", "float8_e4m3fn"):
    setattr(jnp, name, name)
  jnp.zeros = lambda shape, dtype: _FakeArray(shape, dtype)

  def concatenate(parts, axis=0):
    shape = list(parts[0].shape)
    shape[axis] = sum(x.shape[axis] for x in parts)
    return _FakeArray(shape, parts[0].dtype)

  jnp.concatenate = concatenate
  jnp.pad = lambda x, widths: _FakeArray(tuple(n + lo + hi for n, (lo, hi) in zip(x.shape, widths)), x.dtype)
  jax.ShapeDtypeStruct = lambda shape, dtype: _FakeArray(shape, dtype)

  def ffi_call(target, results, **kw):
    def run(*operands, **attrs):
      calls.append({"target": target, "results": results, "kw": kw, "operands": operands, "attrs": attrs})
      return tuple(_FakeArray(r.shape, r.dtype) for r in results) if isinstance(results, tuple) else _FakeArray(results.shape, results.dtype)

    return run

  ffi.ffi_call = ffi_call

  class _CustomVjp:
    def __init__(self, f):
      self.f = f

    def defvjp(self, fwd, bwd):
      self.fwd, self.bwd = fwd, bwd

    def __call__(self, *a):  # run forward AND backward so that both custom calls are recorded
      out, res = self.fwd(*a)
      cot = self.bwd(res, out)
      calls.append({"primals": tuple(x.shape for x in a), "cotangents": tuple(x.shape for x in cot)})
      return out

  jax.custom_vjp = _CustomVjp
  adc = types.ModuleType("jax.ad_checkpoint")

  def checkpoint_name(x, name):
    calls.append({"checkpoint_name": name, "shape": x.shape})
    return x

  adc.checkpoint_name = checkpoint_name
  jax.ffi, jax.numpy, jax.ad_checkpoint = ffi, jnp, adc
  for name, mod in (("jax", jax), ("jax.ffi", ffi), ("jax.numpy", jnp), ("jax.ad_checkpoint", adc)):
    monkeypatch.setitem(sys.modules, name, mod)
  return calls


def test_python_wrappers_follow_the_bind_lines(fake_jax):
  from maxdiffusion_amd import jax_plugin as P

  bf, f32 = "bfloat16", "float32"
  B, S, Skv, H, D = 2, 40, 60, 3, 128
  q, k, v = _FakeArray((B, S, H, D), bf), _FakeArray((B, Skv, H, D), bf), _FakeArray((B, Skv, H, D), bf)
  q3, w = _FakeArray((B, S, H * D), bf), _FakeArray((H * D,), bf)
  wd, tab = _FakeArray((D,), bf), _FakeArray((S, D // 2), f32)
  o_run, l_run = _FakeArray((B, S, H, D), f32), _FakeArray((B, H, S), f32)
  mask = _FakeArray((B, Skv), "bool_")
  P.hip_flash_attention(q, k, v, 0.1, 0)
  P.hip_flash_attention(q, k, v, 0.1, 0, keep_mask=mask)                       # key_mask_bias + fwd_bf16_bias
  P.hip_flash_attention_fp8(q, k, v, 0.1, 0, softmax="exp2")                   # 3 x quant_e4m3 + fwd_fp8
  P.hip_flash_attention_fp8(q, k, v, 0.1, 0, keep_mask=mask)                   # ... + key_mask_bias + fwd_fp8_bias
  P.hip_ring_step(q, k, v, o_run, l_run, 0.1)
  P.hip_merge(o_run, l_run, q, l_run)
  P.hip_finalize(o_run)
  P.hip_flash_attention_vjp(q, k, v, 0.1)                                      # fwd_bf16 + bwd_bf16
  P.hip_flash_attention_vjp(q, k, v, 0.1, static_scratch=True)                 # fwd_bf16 + bwd_bf16_static
  P.hip_flash_attention_vjp(q, k, v, 0.1, keep_mask=mask)                      # key_mask_bias + fwd_bf16_bias + bwd_bf16_bias
  P.hip_norm_rope_fullrow(q3, q3, w, w, tab, tab, H)
  P.hip_norm_rope_fullrow(q3, None, w, None, None, None, H)                    # norm only, cached K/V
  P.hip_norm_rope_perhead(q, q, wd, wd, tab, tab, wq_txt=wd, wk_txt=wd, n_txt=7)
  qkv, b3 = _FakeArray((B, S, 3 * H * D), bf), _FakeArray((3 * H * D,), bf)
  assert [t.shape for t in P.hip_norm_rope_qkv(qkv, w, w, tab, tab, H, bias=b3)] == [(B, S, H, D)] * 3
  assert [t.shape for t in P.hip_norm_rope_qkv(qkv, w, w, None, None, H)] == [(B, S, H, D)] * 3   # v sliced from the fused buffer
  P.hip_norm_rope_ltx2(q3, q3, _FakeArray((H * D,), f32), _FakeArray((H * D,), f32), H,
                       rotary_emb=(_FakeArray((B, S, H * D), f32), _FakeArray((B, S, H * D), f32)))
  binds = _bind_lines()
  seen = set()
  for c in fake_jax:
    if "target" not in c:
      continue
    impl, n_arg, n_ret, attrs = binds[P.FFI_TARGETS[c["target"]]]
    seen.add(c["target"])
    n_results = len(c["results"]) if isinstance(c["results"], tuple) else 1
    assert len(c["operands"]) == n_arg, (c["target"], len(c["operands"]), n_arg)
    assert n_results == n_ret, (c["target"], n_results, n_ret)
    assert sorted(c["attrs"]) == sorted(name for _, name in attrs), (c["target"], sorted(c["attrs"]))
    for typ, name in attrs:  # XLA decodes attributes by exact type: float -> np.float32, int64_t -> np.int64
      want = np.float32 if typ == "float" else np.int64
      assert type(c["attrs"][name]) is want, (c["target"], name, type(c["attrs"][name]))
    for i, o in c["kw"].get("input_output_aliases", {}).items():
      assert c["operands"][i].shape == c["results"][o].shape
  assert seen == set(P.FFI_TARGETS), sorted(set(P.FFI_TARGETS) - seen)
  # the text-token weights of Flux's double blocks reach the custom call (operands 4 and 5) with n_txt
  ph = [c for c in fake_jax if c.get("target") == "mdattn_norm_rope_perhead"][0]
  assert ph["attrs"]["n_txt"] == 7 and ph["operands"][4] is wd and ph["operands"][5] is wd
  # the registry entries: rank-3 [B,S,H*D] in, [B,Sq,H*D] out, both names
  ctx = {"heads": H, "scale": 0.1, "attention_mask": None, "is_causal": False}
  k3 = _FakeArray((B, Skv, H * D), bf)
  for fn in (P.hip_flash_kernel, P.hip_flash_fp8_kernel):
    out = fn(q3, k3, k3, ctx)
    assert out.shape == (B, S, H * D)
  assert P.hip_flash_fp8_kernel(q3, k3, k3, dict(ctx, attention_mask=mask)).shape == (B, S, H * D)
  with pytest.raises(NotImplementedError):
    P.hip_flash_kernel(q3, k3, k3, dict(ctx, is_causal=True))
  with pytest.raises(ValueError, match=r"\[batch, kv_length\]"):
    P.hip_flash_attention(q, k, v, 0.1, 0, keep_mask=_FakeArray((B, 40), "bool_"))


def test_registered_entry_is_differentiable(fake_jax):
  """The function `install()` registers as `hip_flash` is a custom_vjp: forward custom call with lse, backward custom
  calls, in both input layouts, with a key mask, with the residuals tagged by context["residual_checkpoint_name"];
  the prologue hooks are custom_vjps too; the static-scratch backward is used only for shapes that fit its array."""
  from maxdiffusion_amd import jax_plugin as P

  bf = "bfloat16"
  B, S, Skv, H, D = 2, 40, 60, 3, 128
  ctx = {"heads": H, "scale": 0.1, "attention_mask": None, "is_causal": False, "residual_checkpoint_name": "attn_res"}
  targets = lambda: [c["target"] for c in fake_jax if "target" in c]
  # rank 3 ([B,S,H*D], layout 0)
  q3, k3 = _FakeArray((B, S, H * D), bf), _FakeArray((B, Skv, H * D), bf)
  assert P.hip_flash_kernel(q3, k3, k3, ctx).shape == (B, S, H * D)
  assert targets() == ["mdattn_fwd_bf16", "mdattn_bwd_bf16"]      # the fake custom_vjp runs fwd and bwd
  assert [c["checkpoint_name"] for c in fake_jax if "checkpoint_name" in c] == ["attn_res", "attn_res_lse"]
  fwd, bwd = [c for c in fake_jax if "target" in c]
  assert fwd["attrs"]["layout"] == 0 and [r.shape for r in bwd["results"][:3]] == [(B, S, H, D), (B, Skv, H, D), (B, Skv, H, D)]
  # rank 4 ([B,H,S,D], layout 1): the forward reads it in place, the backward's operands are transposed to [B,S,H,D]
  fake_jax.clear()
  q4, k4 = _FakeArray((B, H, S, D), bf), _FakeArray((B, H, Skv, D), bf)
  assert P.hip_flash_kernel(q4, k4, k4, ctx).shape == (B, S, H * D)
  fwd, bwd = [c for c in fake_jax if "target" in c]
  assert fwd["attrs"]["layout"] == 1 and fwd["operands"][0].shape == (B, H, S, D)
  assert [o.shape for o in bwd["operands"][:3]] == [(B, S, H, D), (B, Skv, H, D), (B, Skv, H, D)]
  # with a key mask: the biased forward and the biased backward
  fake_jax.clear()
  P.hip_flash_kernel(q3, k3, k3, dict(ctx, attention_mask=_FakeArray((B, Skv), "bool_")))
  assert targets() == ["mdattn_key_mask_bias", "mdattn_fwd_bf16_bias", "mdattn_bwd_bf16_bias"]
  # head dims below 128 other than 64 are zero-padded to 64 / 128 around the custom calls (the reference pads to 128,
  # attention_flax.py:223-259) and the output is cut back: rank 3 and rank 4, both registry names
  for d, padded in ((40, 64), (80, 128), (64, 64)):
    fake_jax.clear()
    qd, kd = _FakeArray((B, S, H * d), bf), _FakeArray((B, Skv, H * d), bf)
    assert P.hip_flash_kernel(qd, kd, kd, ctx).shape == (B, S, H * d)
    fwd, bwd = [c for c in fake_jax if "target" in c]
    assert fwd["operands"][0].shape == (B, S, H, padded) and bwd["operands"][1].shape == (B, Skv, H, padded)
    assert P.hip_flash_kernel(_FakeArray((B, H, S, d), bf), _FakeArray((B, H, Skv, d), bf), _FakeArray((B, H, Skv, d), bf), ctx).shape == (B, S, H * d)
    assert P.hip_flash_fp8_kernel(qd, kd, kd, ctx).shape == (B, S, H * d)
  # long key sequences: the entry multiplies q by scale * log2(e) itself and hands the kernels scale = ln 2 (forward
  # and backward then run without a multiply per logit); not with a key mask, not when the caller's scale is ln 2 already
  long_k = _FakeArray((B, P.FOLD_SCALE_MIN_KEYS, H * D), bf)
  for c, want in ((ctx, P.FOLDED_SCALE), (dict(ctx, scale=P.FOLDED_SCALE), P.FOLDED_SCALE),
                  (dict(ctx, attention_mask=_FakeArray((B, P.FOLD_SCALE_MIN_KEYS), "bool_")), 0.1)):
    fake_jax.clear()
    P.hip_flash_kernel(q3, long_k, long_k, c)
    scales = {float(x["attrs"]["scale"]) for x in fake_jax if "target" in x and "scale" in x["attrs"]}
    assert scales == {float(np.float32(want))}, (scales, want)
  fake_jax.clear()
  P.hip_flash_kernel(q3, k3, k3, ctx)  # 60 keys: the caller's scale goes through
  assert {float(x["attrs"]["scale"]) for x in fake_jax if "target" in x} == {float(np.float32(0.1))}
  # the static-scratch backward only where 2*B*H*ceil32(Sq) fits its array; beyond, the workspace form
  fake_jax.clear()
  P.hip_flash_attention_vjp(_FakeArray((B, S, H, D), bf), _FakeArray((B, Skv, H, D), bf), _FakeArray((B, Skv, H, D), bf), 0.1, static_scratch=True)
  big = _FakeArray((1, 1 << 21, 4, D), bf)  # 2 * 4 * 2^21 = 16 Mi floats > 8 Mi
  P.hip_flash_attention_vjp(big, big, big, 0.1, static_scratch=True)
  assert targets() == ["mdattn_fwd_bf16", "mdattn_bwd_bf16_static", "mdattn_fwd_bf16", "mdattn_bwd_bf16"]
  m = re.search(r"#define MDATTN_BWD_STATIC_MAX_FLOATS \(([\d\s*]+)\)", open(os.path.join(INCLUDE, "mdattn.h")).read())
  assert P.BWD_STATIC_MAX_FLOATS == eval(m.group(1))  # digits, blanks and '*' only
  # the prologue hooks: forward and backward custom calls, workspace result sized min(rows, 1024) * columns
  fake_jax.clear()
  w, tab = _FakeArray((H * D,), bf), _FakeArray((S, D // 2), "float32")
  P.hip_norm_rope_fullrow(q3, q3, w, w, tab, tab, H)
  assert targets() == ["mdattn_norm_rope_fullrow", "mdattn_norm_rope_fullrow_bwd"]
  ws = [c for c in fake_jax if c.get("target") == "mdattn_norm_rope_fullrow_bwd"][0]["results"][-1]
  assert ws.shape == (min(B * S, P.NORM_ROPE_BWD_MAX_PARTIAL_ROWS) * 2 * H * D,)
  # every custom_vjp returns one cotangent per primal, of the primal's shape
  for c in fake_jax:
    if "cotangents" in c:
      assert c["cotangents"] == c["primals"], c
  # the fused-projection form: its backward is the full-row backward on the q | k column blocks with their biases; the
  # cotangent of the fused buffer is [dq | dk | gv], the bias's [dbias_q | dbias_k | sum of gv]
  fake_jax.clear()
  N = H * D
  qkv, b3 = _FakeArray((B, S, 3 * N), bf), _FakeArray((3 * N,), bf)
  assert [t.shape for t in P.hip_norm_rope_qkv(qkv, w, w, tab, tab, H, bias=b3)] == [(B, S, H, D)] * 3
  assert targets() == ["mdattn_norm_rope_qkv", "mdattn_norm_rope_fullrow_bwd"]
  bwd = [c for c in fake_jax if c.get("target") == "mdattn_norm_rope_fullrow_bwd"][0]
  assert [o.shape for o in bwd["operands"][:4]] == [(B, S, N), (B, S, N), (B, S, H, D), (B, S, H, D)]
  assert bwd["operands"][8].shape == (2 * N,) and bwd["attrs"]["has_bias"] == 1 and bwd["attrs"]["has_k"] == 1
  assert [r.shape for r in bwd["results"]] == [(B, S, N), (B, S, N), (N,), (N,), (2 * N,), (min(B * S, 1024) * 4 * N,)]
  vjp = [c for c in fake_jax if "cotangents" in c][0]
  assert vjp["cotangents"] == ((B, S, 3 * N), (N,), (N,), (3 * N,)) == vjp["primals"]
  fake_jax.clear()
  P.hip_norm_rope_qkv(qkv, w, w, None, None, H)                      # no bias, norm only: v is a slice, workspace 2N columns
  bwd = [c for c in fake_jax if c.get("target") == "mdattn_norm_rope_fullrow_bwd"][0]
  assert bwd["attrs"]["has_bias"] == 0 and bwd["attrs"]["rope"] == 0 and bwd["results"][-1].shape == (min(B * S, 1024) * 2 * N,)


def test_install_registers_both_kernel_names(fake_jax, monkeypatch, tmp_path):
  from maxdiffusion_amd import jax_plugin as P

  registered, registry = [], {}
  sys.modules["jax.ffi"].register_ffi_target = lambda name, capsule, platform: registered.append((name, platform))
  sys.modules["jax.ffi"].pycapsule = lambda fn: fn
  md = types.ModuleType("maxdiffusion")
  mdm = types.ModuleType("maxdiffusion.models")
  af = types.ModuleType("maxdiffusion.models.attention_flax")
  af.register_kernel = lambda name: (lambda f: registry.setdefault(name, f))
  mdm.attention_flax = af
  for name, mod in (("maxdiffusion", md), ("maxdiffusion.models", mdm), ("maxdiffusion.models.attention_flax", af)):
    monkeypatch.setitem(sys.modules, name, mod)
  fake_lib = types.SimpleNamespace(**{s: s for s in P.FFI_TARGETS.values()})
  monkeypatch.setattr(P.ctypes, "CDLL", lambda path: fake_lib)
  lib_file = tmp_path / "libmdattn_ffi.so"
  lib_file.write_bytes(b"")
  monkeypatch.setattr(P, "FFI_LIB_PATH", str(lib_file))
  monkeypatch.setattr(P, "_installed", False)
  P.install()
  assert sorted(n for n, _ in registered) == sorted(P.FFI_TARGETS) and {p for _, p in registered} == {"ROCM"}
  assert registry == {"hip_flash": P.hip_flash_kernel, "hip_flash_fp8": P.hip_flash_fp8_kernel}


# ----------------------------------------------------------------------------- marshalling layer, host side
class Buffer(ctypes.Structure):
  _fields_ = [("data", ctypes.c_void_p), ("dtype", ctypes.c_int32), ("rank", ctypes.c_int32), ("dims", ctypes.POINTER(ctypes.c_int64))]


BF16, F32, U8, F8 = 1, 2, 3, 4


def buf(shape, dtype, ptr=0x10000):
  dims = (ctypes.c_int64 * max(len(shape), 1))(*shape)
  b = Buffer(ptr, dtype, len(shape), dims)
  b._keep = dims
  return b


def call(lib, name, *args):
  """Calls mdattn_xla_<name>(NULL stream, buffers..., attributes..., err, len); returns (code, message)."""
  fn = getattr(lib, "mdattn_xla_" + name)
  fn.restype = ctypes.c_int
  err = ctypes.create_string_buffer(512)
  conv = [ctypes.byref(a) if isinstance(a, Buffer) else a for a in args]
  rc = fn(None, *conv, err, 512)
  return rc, err.value.decode()


def test_marshalling_rejects_bad_buffers_by_name(lib):
  from maxdiffusion_amd import _lib

  f, i = ctypes.c_float, ctypes.c_int64
  B, S, Skv, H, D = 2, 40, 60, 3, 128
  q, k, v = buf((B, S, H, D), BF16), buf((B, Skv, H, D), BF16), buf((B, Skv, H, D), BF16)
  out, lse = buf((B, S, H, D), BF16), buf((B, H, S), F32)
  q3, wN, wD, tabh = buf((B, S, H * D), BF16), buf((H * D,), BF16), buf((D,), BF16), buf((S, D // 2), F32)
  fN, fD = buf((H * D,), F32), buf((D,), F32)
  cases = [
      (("fwd_bf16", buf((B, S, H * D), BF16), k, v, out, lse, f(0.1), i(0)), "rank-4"),
      (("fwd_bf16", buf((B, S, H, D), F32), k, v, out, lse, f(0.1), i(0)), "q must be bf16, got f32"),
      (("fwd_bf16", q, buf((B, Skv, H + 1, D), BF16), v, out, lse, f(0.1), i(0)), "does not match q"),
      (("fwd_bf16", q, k, buf((B, Skv + 1, H, D), BF16), out, lse, f(0.1), i(0)), "k and v must have the same shape"),
      (("fwd_bf16", q, k, v, buf((B, H, S, D), BF16), lse, f(0.1), i(0)), "out must be [B,Sq,H,D]"),
      (("fwd_bf16", q, k, v, out, buf((B, S, H), F32), f(0.1), i(0)), "lse must be [B,H,Sq]"),
      (("fwd_bf16", q, k, v, out, lse, f(0.1), i(2)), "layout must be 0"),
      (("fwd_bf16", buf((B, S, H, D), BF16, ptr=0), k, v, out, lse, f(0.1), i(0)), "q is missing"),
      (("fwd_bf16_bias", q, k, v, buf((B, 32), F32), out, lse, f(0.1), i(0)), "key_bias must be [B, Skv rounded up to 32] = [2,64]"),
      (("key_mask_bias", buf((B, Skv), F32), buf((B, 64), F32), f(-1e4)), "keep must be u8"),
      (("key_mask_bias", buf((B, 1, Skv), U8), buf((B, 64), F32), f(-1e4)), "[batch, kv_length]"),
      (("key_mask_bias", buf((B, Skv), U8), buf((B, Skv), F32), f(-1e4)), "bias must be [B, Skv rounded up to 32]"),
      (("fwd_bf16_merge", q, k, v, buf((B, S, H, D), F32), lse, buf((B, S, H, D), F32, ptr=0x20000), lse, f(0.1), i(0)), "o_run must be donated"),
      (("fwd_bf16_merge", q, k, v, out, lse, out, lse, f(0.1), i(0)), "o_run must be f32"),
      (("merge", buf((B, S, H, D), F32), lse, buf((B, S, H, D), U8), lse, buf((B, S, H, D), F32), lse), "o_cur must be bf16 or f32"),
      (("finalize", buf((B, S, H, D), F32), buf((B, S, H), BF16)), "same number of elements"),
      (("norm_rope_fullrow", buf((B, S, H * D), BF16), buf((B, S, H * D), BF16), buf((H * D,), BF16), buf((H * D,), BF16),
        buf((S, D // 2), F32), buf((S, D // 2), F32), out, out, f(1e-6), f(1.0), i(H + 2), i(1), i(1)), "q must be [B,S,H*D] with H = heads"),
      (("norm_rope_fullrow", buf((B, S, H * D), BF16), buf((B, S, H * D), BF16), buf((H * D,), BF16), buf((H * D,), BF16),
        buf((S, D), F32), buf((S, D // 2), F32), out, out, f(1e-6), f(1.0), i(H), i(1), i(1)), "cos must hold"),
      (("norm_rope_fullrow", buf((B, S, H * D), BF16), buf((B, S, H * D), BF16), buf((D,), BF16), buf((H * D,), BF16),
        buf((S, D // 2), F32), buf((S, D // 2), F32), out, out, f(1e-6), f(1.0), i(H), i(1), i(1)), "wq must hold 384"),
      (("norm_rope_perhead", q, q, buf((D,), BF16), buf((D,), BF16), buf((D,), BF16), buf((D,), BF16), buf((S, D // 2), F32),
        buf((S, D // 2), F32), out, out, f(1e-6), f(1.0), i(S + 1), i(1), i(1)), "n_txt"),
      (("norm_rope_qkv", buf((B, S, 3 * H * D), BF16), buf((3 * H * D,), BF16), buf((H * D,), BF16), buf((H * D,), BF16),
        buf((S, D // 2), F32), buf((S, D // 2), F32), out, out, out, f(1e-6), f(1.0), i(H), i(1), i(1), i(0)), "has_v must be set"),
      (("norm_rope_qkv", buf((B, S, 3 * H * D), BF16), buf((H * D,), BF16), buf((H * D,), BF16), buf((H * D,), BF16),
        buf((S, D // 2), F32), buf((S, D // 2), F32), out, out, out, f(1e-6), f(1.0), i(H), i(1), i(1), i(1)), "bias must hold 1152"),
      (("norm_rope_qkv", buf((B, S, 2 * H * D), BF16), buf((3 * H * D,), BF16), buf((H * D,), BF16), buf((H * D,), BF16),
        buf((S, D // 2), F32), buf((S, D // 2), F32), out, out, out, f(1e-6), f(1.0), i(H), i(1), i(0), i(0)), "qkv must be [B,S,3*H*D]"),
      (("norm_rope_perhead", q, q, buf((D,), BF16), buf((D,), BF16), buf((2 * D,), BF16), buf((D,), BF16), buf((S, D // 2), F32),
        buf((S, D // 2), F32), out, out, f(1e-6), f(1.0), i(5), i(1), i(1)), "wq_txt must hold 128"),
      (("norm_rope_rows", buf((B, S, H * D), BF16), buf((H * D,), F32), buf((B, S, H * D), F32), buf((B, S, H * D), F32), out,
        f(1e-6), i(H), i(3)), "mode must be"),
      (("norm_rope_rows", buf((B, S, H * D), BF16), buf((H * D,), BF16), buf((B, S, H * D), F32), buf((B, S, H * D), F32), out,
        f(1e-6), i(H), i(1)), "w must be f32"),
      (("norm_rope_fullrow_bwd", q3, q3, out, out, wN, wN, tabh, tabh, wN, q3, q3, fN, fN, fN, buf((10,), F32), f(1e-6), f(1.0), i(H), i(1), i(1), i(0)),
       "workspace must hold at least 768"),
      (("norm_rope_fullrow_bwd", q3, q3, buf((B, H, S, D), BF16), out, wN, wN, tabh, tabh, wN, q3, q3, fN, fN, fN, buf((768,), F32), f(1e-6), f(1.0), i(H), i(1), i(1), i(0)),
       "gq must be [B,S,H,D]"),
      (("norm_rope_fullrow_bwd", q3, q3, out, out, wN, wN, tabh, tabh, wN, q3, q3, buf((H * D,), BF16), fN, fN, buf((768,), F32), f(1e-6), f(1.0), i(H), i(1), i(1), i(0)),
       "dwq must be f32"),
      (("norm_rope_fullrow_bwd", q3, q3, out, out, wN, wN, tabh, tabh, wN, q3, q3, fN, fN, fN, buf((768,), F32), f(1e-6), f(1.0), i(H), i(1), i(0), i(1)),
       "has_bias needs has_k"),
      (("norm_rope_perhead_bwd", q, q, out, out, wD, wD, wD, wD, tabh, tabh, out, out, fD, fD, fD, buf((2 * D,), F32), buf((4 * D,), F32), f(1e-6), f(1.0), i(5), i(1), i(1)),
       "dwk_txt must hold 128"),
      (("norm_rope_rows_bwd", q3, out, buf((H * D,), F32), tabh, tabh, buf((B, S, H * D), F32), fN, buf((H * D,), F32), f(1e-6), i(H), i(0)),
       "dx must have x's dtype and shape"),
      (("quant_e4m3", q, buf((B, S, H, D), BF16), buf((2,), F32), f(1.0), i(0)), "x8 must be a u8 or f8e4m3fn"),
      (("quant_e4m3", q, buf((B, S, H, D), F8), buf((1,), F32), f(1.0), i(0)), "scale_out must hold 2"),
      (("fwd_fp8", q, k, v, buf((2,), F32), buf((2,), F32), buf((2,), F32), out, lse, f(0.1), i(0), i(0)), "q8, k8, v8 must be u8 or f8e4m3fn"),
      (("fwd_fp8", buf((B, S, H, D), F8), buf((B, Skv, H, D), F8), buf((B, Skv, H, D), U8), buf((2,), F32), buf((2,), F32), buf((2,), F32),
        out, lse, f(0.1), i(0), i(5)), "softmax_mode"),
      (("bwd_bf16", q, k, v, out, out, lse, out, k, k, buf((10,), F32), f(0.1)), "workspace must hold at least 768"),
      (("bwd_bf16", q, k, v, out, out, lse, out, out, k, buf((768,), F32), f(0.1)), "dk must be [B,Sq,H,D] = [2,60,3,128]"),
      (("bwd_bf16_static", q, k, v, out, buf((B, S, H, D), F32), lse, out, k, k, f(0.1)), "dout must be bf16"),
  ]
  for args, needle in cases:
    rc, msg = call(lib, *args)
    assert rc == _lib.E_BADARG, (args[0], rc, msg)
    assert msg.startswith("mdattn_" + args[0] + ": ") and needle in msg, (args[0], msg)


def test_marshalling_hands_well_formed_requests_to_the_c_abi(lib):
  """Well-formed buffers pass the marshalling layer and reach the C ABI, whose own validation then objects to what
  only it checks: a misaligned pointer (MDATTN_E_ALIGN), an unsupported head dim.  No kernel is launched."""
  from maxdiffusion_amd import _lib

  f, i = ctypes.c_float, ctypes.c_int64
  B, S, Skv, H, D = 2, 40, 60, 3, 128
  odd = 0x10004
  k, v = buf((B, H, Skv, D), BF16), buf((B, H, Skv, D), BF16)
  out, lse = buf((B, S, H, D), BF16), buf((B, H, S), F32)
  rc, msg = call(lib, "fwd_bf16", buf((B, H, S, D), BF16, ptr=odd), k, v, out, lse, f(0.1), i(1))
  assert rc == _lib.E_ALIGN and "aligned" in msg
  q32 = buf((B, S, H, 32), BF16)
  rc, msg = call(lib, "fwd_bf16", q32, buf((B, Skv, H, 32), BF16), buf((B, Skv, H, 32), BF16), buf((B, S, H, 32), BF16), lse, f(0.1), i(0))
  assert rc == _lib.E_UNSUPPORTED and msg.startswith("mdattn_fwd_bf16: unsupported")
  rc, msg = call(lib, "finalize", buf((B, S, H, D), F32, ptr=odd), buf((B, S, H, D), BF16))
  assert rc == _lib.E_ALIGN
  rc, msg = call(lib, "quant_e4m3", buf((3, 5), BF16), buf((3, 5), F8), buf((2,), F32), f(1.0), i(1))
  assert rc == _lib.E_UNSUPPORTED  # 15 elements: the quantiser wants a multiple of 16
  rc, msg = call(lib, "fwd_fp8", buf((B, S, H, D), F8, ptr=odd), buf((B, Skv, H, D), F8), buf((B, Skv, H, D), U8), buf((2,), F32),
                 buf((2,), F32), buf((2,), F32), out, lse, f(0.1), i(0), i(1))
  assert rc == _lib.E_ALIGN
  # a message buffer is optional
  fn = lib.mdattn_xla_finalize
  fn.restype = ctypes.c_int
  assert fn(None, ctypes.byref(buf((4, 4), F32)), ctypes.byref(buf((4, 5), BF16)), None, 0) == _lib.E_BADARG
