// XLA FFI bind lines: the only file that sees xla/ffi/api/ffi.h.  Each handler converts its ffi::AnyBuffer arguments
// to mdattn_buffer (pointer, element type, dimensions) and calls the handler body of the same name in
// mdattn_marshal.h, which lives in libmdattn.so and holds every check and the call into the C ABI.
// Built only where jaxlib's headers (jax.ffi.include_dir()) are present.  Handlers enqueue on XLA's stream, never
// synchronise, never allocate.
//
// Registered from Python (maxdiffusion_amd/jax_plugin.py) with
//   jax.ffi.register_ffi_target(name, jax.ffi.pycapsule(lib.<Symbol>), platform="ROCM")
#include <hip/hip_runtime.h>

#include <cstdint>
#include <string>

#include "mdattn_marshal.h"
#include "xla/ffi/api/ffi.h"

namespace ffi = xla::ffi;

namespace {

using Buf = ffi::AnyBuffer;
using Res = ffi::Result<ffi::AnyBuffer>;

int Dtype(ffi::DataType t) {
  switch (t) {
    case ffi::DataType::BF16: return MDATTN_DT_BF16;
    case ffi::DataType::F32: return MDATTN_DT_F32;
    case ffi::DataType::U8:
    case ffi::DataType::S8:
    case ffi::DataType::PRED: return MDATTN_DT_U8;
    case ffi::DataType::F8E4M3FN: return MDATTN_DT_F8E4M3FN;
    default: return MDATTN_DT_OTHER;
  }
}
mdattn_buffer In(const Buf& b) {
  const auto d = b.dimensions();
  return mdattn_buffer{b.untyped_data(), Dtype(b.element_type()), (int32_t)d.size(), d.begin()};
}
mdattn_buffer Out(Res& r) {
  const auto d = r->dimensions();
  return mdattn_buffer{r->untyped_data(), Dtype(r->element_type()), (int32_t)d.size(), d.begin()};
}
struct Msg {
  char text[512] = {0};
  // argument errors stay InvalidArgument; a launch the runtime rejected, a request no kernel is built for and a request
  // beyond the static scratch are not the caller's arguments being wrong, and say so
  ffi::Error done(int rc) const {
    switch (rc) {
      case MDATTN_OK: return ffi::Error::Success();
      case MDATTN_E_LAUNCH: return ffi::Error::Internal(std::string(text));
      case MDATTN_E_UNSUPPORTED: return ffi::Error(ffi::ErrorCode::kUnimplemented, std::string(text));
      case MDATTN_E_TOOBIG: return ffi::Error(ffi::ErrorCode::kResourceExhausted, std::string(text));
      default: return ffi::Error::InvalidArgument(std::string(text));
    }
  }
};

ffi::Error FwdBf16(hipStream_t s, Buf q, Buf k, Buf v, Res out, Res lse, float scale, int64_t layout) {
  Msg m;
  const mdattn_buffer a = In(q), b = In(k), c = In(v), o = Out(out), l = Out(lse);
  return m.done(mdattn_xla_fwd_bf16(s, &a, &b, &c, &o, &l, scale, layout, m.text, sizeof m.text));
}
ffi::Error FwdBf16Bias(hipStream_t s, Buf q, Buf k, Buf v, Buf key_bias, Res out, Res lse, float scale, int64_t layout) {
  Msg m;
  const mdattn_buffer a = In(q), b = In(k), c = In(v), kb = In(key_bias), o = Out(out), l = Out(lse);
  return m.done(mdattn_xla_fwd_bf16_bias(s, &a, &b, &c, &kb, &o, &l, scale, layout, m.text, sizeof m.text));
}
ffi::Error KeyMaskBias(hipStream_t s, Buf keep, Res bias, float masked_value) {
  Msg m;
  const mdattn_buffer a = In(keep), o = Out(bias);
  return m.done(mdattn_xla_key_mask_bias(s, &a, &o, masked_value, m.text, sizeof m.text));
}
ffi::Error FwdBf16Merge(hipStream_t s, Buf q, Buf k, Buf v, Buf o_run_in, Buf lse_run_in, Res o_run, Res lse_run, float scale,
                        int64_t layout) {
  Msg m;
  const mdattn_buffer a = In(q), b = In(k), c = In(v), oi = In(o_run_in), li = In(lse_run_in), o = Out(o_run), l = Out(lse_run);
  return m.done(mdattn_xla_fwd_bf16_merge(s, &a, &b, &c, &oi, &li, &o, &l, scale, layout, m.text, sizeof m.text));
}
ffi::Error Merge(hipStream_t s, Buf o_run_in, Buf lse_run_in, Buf o_cur, Buf lse_cur, Res o_run, Res lse_run) {
  Msg m;
  const mdattn_buffer oi = In(o_run_in), li = In(lse_run_in), oc = In(o_cur), lc = In(lse_cur), o = Out(o_run), l = Out(lse_run);
  return m.done(mdattn_xla_merge(s, &oi, &li, &oc, &lc, &o, &l, m.text, sizeof m.text));
}
ffi::Error Finalize(hipStream_t s, Buf o_run, Res out) {
  Msg m;
  const mdattn_buffer a = In(o_run), o = Out(out);
  return m.done(mdattn_xla_finalize(s, &a, &o, m.text, sizeof m.text));
}
ffi::Error NormRopeFullrow(hipStream_t s, Buf q, Buf k, Buf wq, Buf wk, Buf cos, Buf sin, Res q_out, Res k_out, float eps, float q_mul,
                           int64_t heads, int64_t rope, int64_t has_k) {
  Msg m;
  const mdattn_buffer a = In(q), b = In(k), c = In(wq), d = In(wk), e = In(cos), f = In(sin), qo = Out(q_out), ko = Out(k_out);
  return m.done(mdattn_xla_norm_rope_fullrow(s, &a, &b, &c, &d, &e, &f, &qo, &ko, eps, q_mul, heads, rope, has_k, m.text, sizeof m.text));
}
ffi::Error NormRopeQkv(hipStream_t s, Buf qkv, Buf bias, Buf wq, Buf wk, Buf cos, Buf sin, Res q_out, Res k_out, Res v_out, float eps,
                       float q_mul, int64_t heads, int64_t rope, int64_t has_bias, int64_t has_v) {
  Msg m;
  const mdattn_buffer a = In(qkv), b = In(bias), c = In(wq), d = In(wk), e = In(cos), f = In(sin), qo = Out(q_out), ko = Out(k_out),
                      vo = Out(v_out);
  return m.done(mdattn_xla_norm_rope_qkv(s, &a, &b, &c, &d, &e, &f, &qo, &ko, &vo, eps, q_mul, heads, rope, has_bias, has_v, m.text,
                                         sizeof m.text));
}
ffi::Error NormRopePerhead(hipStream_t s, Buf q, Buf k, Buf wq, Buf wk, Buf wq_txt, Buf wk_txt, Buf cos, Buf sin, Res q_out, Res k_out,
                           float eps, float q_mul, int64_t n_txt, int64_t rope, int64_t has_k) {
  Msg m;
  const mdattn_buffer a = In(q), b = In(k), c = In(wq), d = In(wk), ct = In(wq_txt), dt = In(wk_txt), e = In(cos), f = In(sin),
                      qo = Out(q_out), ko = Out(k_out);
  return m.done(mdattn_xla_norm_rope_perhead(s, &a, &b, &c, &d, &ct, &dt, &e, &f, &qo, &ko, eps, q_mul, n_txt, rope, has_k, m.text,
                                             sizeof m.text));
}
ffi::Error NormRopeRows(hipStream_t s, Buf x, Buf w, Buf cos, Buf sin, Res x_out, float eps, int64_t heads, int64_t mode) {
  Msg m;
  const mdattn_buffer a = In(x), b = In(w), c = In(cos), d = In(sin), o = Out(x_out);
  return m.done(mdattn_xla_norm_rope_rows(s, &a, &b, &c, &d, &o, eps, heads, mode, m.text, sizeof m.text));
}
ffi::Error NormRopeFullrowBwd(hipStream_t s, Buf q, Buf k, Buf gq, Buf gk, Buf wq, Buf wk, Buf cos, Buf sin, Buf bias, Res dq, Res dk,
                              Res dwq, Res dwk, Res dbias, Res workspace, float eps, float q_mul, int64_t heads, int64_t rope,
                              int64_t has_k, int64_t has_bias) {
  Msg m;
  const mdattn_buffer a = In(q), b = In(k), c = In(gq), d = In(gk), e = In(wq), f = In(wk), g = In(cos), h = In(sin), i = In(bias),
                      o0 = Out(dq), o1 = Out(dk), o2 = Out(dwq), o3 = Out(dwk), o4 = Out(dbias), ws = Out(workspace);
  return m.done(mdattn_xla_norm_rope_fullrow_bwd(s, &a, &b, &c, &d, &e, &f, &g, &h, &i, &o0, &o1, &o2, &o3, &o4, &ws, eps, q_mul, heads, rope,
                                                 has_k, has_bias, m.text, sizeof m.text));
}
ffi::Error NormRopePerheadBwd(hipStream_t s, Buf q, Buf k, Buf gq, Buf gk, Buf wq, Buf wk, Buf wq_txt, Buf wk_txt, Buf cos, Buf sin, Res dq,
                              Res dk, Res dwq, Res dwk, Res dwq_txt, Res dwk_txt, Res workspace, float eps, float q_mul, int64_t n_txt,
                              int64_t rope, int64_t has_k) {
  Msg m;
  const mdattn_buffer a = In(q), b = In(k), c = In(gq), d = In(gk), e = In(wq), f = In(wk), et = In(wq_txt), ft = In(wk_txt), g = In(cos),
                      h = In(sin), o0 = Out(dq), o1 = Out(dk), o2 = Out(dwq), o3 = Out(dwk), o4 = Out(dwq_txt), o5 = Out(dwk_txt),
                      ws = Out(workspace);
  return m.done(mdattn_xla_norm_rope_perhead_bwd(s, &a, &b, &c, &d, &e, &f, &et, &ft, &g, &h, &o0, &o1, &o2, &o3, &o4, &o5, &ws, eps, q_mul,
                                                 n_txt, rope, has_k, m.text, sizeof m.text));
}
ffi::Error NormRopeRowsBwd(hipStream_t s, Buf x, Buf g, Buf w, Buf cos, Buf sin, Res dx, Res dw, Res workspace, float eps, int64_t heads,
                           int64_t mode) {
  Msg m;
  const mdattn_buffer a = In(x), b = In(g), c = In(w), d = In(cos), e = In(sin), o0 = Out(dx), o1 = Out(dw), ws = Out(workspace);
  return m.done(mdattn_xla_norm_rope_rows_bwd(s, &a, &b, &c, &d, &e, &o0, &o1, &ws, eps, heads, mode, m.text, sizeof m.text));
}
ffi::Error QuantE4m3(hipStream_t s, Buf x, Res x8, Res scale_out, float premul, int64_t pow2_scale) {
  Msg m;
  const mdattn_buffer a = In(x), o = Out(x8), sc = Out(scale_out);
  return m.done(mdattn_xla_quant_e4m3(s, &a, &o, &sc, premul, pow2_scale, m.text, sizeof m.text));
}
ffi::Error FwdFp8(hipStream_t s, Buf q8, Buf k8, Buf v8, Buf q_scale, Buf k_scale, Buf v_scale, Res out, Res lse, float scale,
                  int64_t layout, int64_t softmax_mode) {
  Msg m;
  const mdattn_buffer a = In(q8), b = In(k8), c = In(v8), qs = In(q_scale), ks = In(k_scale), vs = In(v_scale), o = Out(out), l = Out(lse);
  return m.done(mdattn_xla_fwd_fp8(s, &a, &b, &c, &qs, &ks, &vs, &o, &l, scale, layout, softmax_mode, m.text, sizeof m.text));
}
ffi::Error FwdFp8Bias(hipStream_t s, Buf q8, Buf k8, Buf v8, Buf q_scale, Buf k_scale, Buf v_scale, Buf key_bias, Res out, Res lse,
                      float scale, int64_t layout) {
  Msg m;
  const mdattn_buffer a = In(q8), b = In(k8), c = In(v8), qs = In(q_scale), ks = In(k_scale), vs = In(v_scale), kb = In(key_bias),
                      o = Out(out), l = Out(lse);
  return m.done(mdattn_xla_fwd_fp8_bias(s, &a, &b, &c, &qs, &ks, &vs, &kb, &o, &l, scale, layout, m.text, sizeof m.text));
}
ffi::Error BwdBf16(hipStream_t s, Buf q, Buf k, Buf v, Buf out, Buf dout, Buf lse, Res dq, Res dk, Res dv, Res workspace, float scale) {
  Msg m;
  const mdattn_buffer a = In(q), b = In(k), c = In(v), o = In(out), d = In(dout), l = In(lse), gq = Out(dq), gk = Out(dk), gv = Out(dv),
                      ws = Out(workspace);
  return m.done(mdattn_xla_bwd_bf16(s, &a, &b, &c, &o, &d, &l, &gq, &gk, &gv, &ws, scale, m.text, sizeof m.text));
}
ffi::Error BwdBf16Bias(hipStream_t s, Buf q, Buf k, Buf v, Buf out, Buf dout, Buf lse, Buf key_bias, Res dq, Res dk, Res dv, Res workspace,
                       float scale) {
  Msg m;
  const mdattn_buffer a = In(q), b = In(k), c = In(v), o = In(out), d = In(dout), l = In(lse), kb = In(key_bias), gq = Out(dq),
                      gk = Out(dk), gv = Out(dv), ws = Out(workspace);
  return m.done(mdattn_xla_bwd_bf16_bias(s, &a, &b, &c, &o, &d, &l, &kb, &gq, &gk, &gv, &ws, scale, m.text, sizeof m.text));
}
ffi::Error BwdBf16Static(hipStream_t s, Buf q, Buf k, Buf v, Buf out, Buf dout, Buf lse, Res dq, Res dk, Res dv, float scale) {
  Msg m;
  const mdattn_buffer a = In(q), b = In(k), c = In(v), o = In(out), d = In(dout), l = In(lse), gq = Out(dq), gk = Out(dk), gv = Out(dv);
  return m.done(mdattn_xla_bwd_bf16_static(s, &a, &b, &c, &o, &d, &l, &gq, &gk, &gv, scale, m.text, sizeof m.text));
}

}  // namespace

#define MDATTN_BIND ffi::Ffi::Bind().Ctx<ffi::PlatformStream<hipStream_t>>()

XLA_FFI_DEFINE_HANDLER_SYMBOL(MdattnFwdBf16, FwdBf16,
                              MDATTN_BIND.Arg<Buf>().Arg<Buf>().Arg<Buf>().Ret<Buf>().Ret<Buf>()
                                  .Attr<float>("scale").Attr<int64_t>("layout"));
XLA_FFI_DEFINE_HANDLER_SYMBOL(MdattnFwdBf16Bias, FwdBf16Bias,
                              MDATTN_BIND.Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Ret<Buf>().Ret<Buf>()
                                  .Attr<float>("scale").Attr<int64_t>("layout"));
XLA_FFI_DEFINE_HANDLER_SYMBOL(MdattnKeyMaskBias, KeyMaskBias,
                              MDATTN_BIND.Arg<Buf>().Ret<Buf>().Attr<float>("masked_value"));
XLA_FFI_DEFINE_HANDLER_SYMBOL(MdattnFwdBf16Merge, FwdBf16Merge,
                              MDATTN_BIND.Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Ret<Buf>().Ret<Buf>()
                                  .Attr<float>("scale").Attr<int64_t>("layout"));
XLA_FFI_DEFINE_HANDLER_SYMBOL(MdattnMerge, Merge,
                              MDATTN_BIND.Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Ret<Buf>().Ret<Buf>());
XLA_FFI_DEFINE_HANDLER_SYMBOL(MdattnFinalize, Finalize, MDATTN_BIND.Arg<Buf>().Ret<Buf>());
XLA_FFI_DEFINE_HANDLER_SYMBOL(MdattnNormRopeFullrow, NormRopeFullrow,
                              MDATTN_BIND.Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Ret<Buf>().Ret<Buf>()
                                  .Attr<float>("eps").Attr<float>("q_mul").Attr<int64_t>("heads").Attr<int64_t>("rope")
                                  .Attr<int64_t>("has_k"));
XLA_FFI_DEFINE_HANDLER_SYMBOL(MdattnNormRopeQkv, NormRopeQkv,
                              MDATTN_BIND.Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>()
                                  .Ret<Buf>().Ret<Buf>().Ret<Buf>()
                                  .Attr<float>("eps").Attr<float>("q_mul").Attr<int64_t>("heads").Attr<int64_t>("rope")
                                  .Attr<int64_t>("has_bias").Attr<int64_t>("has_v"));
XLA_FFI_DEFINE_HANDLER_SYMBOL(MdattnNormRopePerhead, NormRopePerhead,
                              MDATTN_BIND.Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>()
                                  .Ret<Buf>().Ret<Buf>()
                                  .Attr<float>("eps").Attr<float>("q_mul").Attr<int64_t>("n_txt").Attr<int64_t>("rope")
                                  .Attr<int64_t>("has_k"));
XLA_FFI_DEFINE_HANDLER_SYMBOL(MdattnNormRopeRows, NormRopeRows,
                              MDATTN_BIND.Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Ret<Buf>()
                                  .Attr<float>("eps").Attr<int64_t>("heads").Attr<int64_t>("mode"));
XLA_FFI_DEFINE_HANDLER_SYMBOL(MdattnNormRopeFullrowBwd, NormRopeFullrowBwd,
                              MDATTN_BIND.Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>()
                                  .Ret<Buf>().Ret<Buf>().Ret<Buf>().Ret<Buf>().Ret<Buf>().Ret<Buf>()
                                  .Attr<float>("eps").Attr<float>("q_mul").Attr<int64_t>("heads").Attr<int64_t>("rope")
                                  .Attr<int64_t>("has_k").Attr<int64_t>("has_bias"));
XLA_FFI_DEFINE_HANDLER_SYMBOL(MdattnNormRopePerheadBwd, NormRopePerheadBwd,
                              MDATTN_BIND.Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>()
                                  .Arg<Buf>().Ret<Buf>().Ret<Buf>().Ret<Buf>().Ret<Buf>().Ret<Buf>().Ret<Buf>().Ret<Buf>()
                                  .Attr<float>("eps").Attr<float>("q_mul").Attr<int64_t>("n_txt").Attr<int64_t>("rope")
                                  .Attr<int64_t>("has_k"));
XLA_FFI_DEFINE_HANDLER_SYMBOL(MdattnNormRopeRowsBwd, NormRopeRowsBwd,
                              MDATTN_BIND.Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Ret<Buf>().Ret<Buf>().Ret<Buf>()
                                  .Attr<float>("eps").Attr<int64_t>("heads").Attr<int64_t>("mode"));
XLA_FFI_DEFINE_HANDLER_SYMBOL(MdattnQuantE4m3, QuantE4m3,
                              MDATTN_BIND.Arg<Buf>().Ret<Buf>().Ret<Buf>().Attr<float>("premul").Attr<int64_t>("pow2_scale"));
XLA_FFI_DEFINE_HANDLER_SYMBOL(MdattnFwdFp8, FwdFp8,
                              MDATTN_BIND.Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Ret<Buf>().Ret<Buf>()
                                  .Attr<float>("scale").Attr<int64_t>("layout").Attr<int64_t>("softmax_mode"));
XLA_FFI_DEFINE_HANDLER_SYMBOL(MdattnFwdFp8Bias, FwdFp8Bias,
                              MDATTN_BIND.Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>()
                                  .Ret<Buf>().Ret<Buf>().Attr<float>("scale").Attr<int64_t>("layout"));
XLA_FFI_DEFINE_HANDLER_SYMBOL(MdattnBwdBf16, BwdBf16,
                              MDATTN_BIND.Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>()
                                  .Ret<Buf>().Ret<Buf>().Ret<Buf>().Ret<Buf>().Attr<float>("scale"));
XLA_FFI_DEFINE_HANDLER_SYMBOL(MdattnBwdBf16Bias, BwdBf16Bias,
                              MDATTN_BIND.Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>()
                                  .Ret<Buf>().Ret<Buf>().Ret<Buf>().Ret<Buf>().Attr<float>("scale"));
XLA_FFI_DEFINE_HANDLER_SYMBOL(MdattnBwdBf16Static, BwdBf16Static,
                              MDATTN_BIND.Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>()
                                  .Ret<Buf>().Ret<Buf>().Ret<Buf>().Attr<float>("scale"));
