// XLA FFI handlers: a mechanical shim from XLA custom-call buffers to the C ABI of mdattn.h.
// Built only where jaxlib's headers (jax.ffi.include_dir()) are present; all logic lives in
// libmdattn.so.  Handlers enqueue on XLA's stream, never synchronise, never allocate.
//
// Registered from Python (maxdiffusion_amd/jax_plugin.py) with
//   jax.ffi.register_ffi_target(name, jax.ffi.pycapsule(lib.<Symbol>), platform="ROCM")
#include <hip/hip_runtime.h>

#include <cstdint>
#include <string>

#include "mdattn.h"
#include "xla/ffi/api/ffi.h"

namespace ffi = xla::ffi;

namespace {

ffi::Error ToError(int rc, const char* where) {
  if (rc == MDATTN_OK) return ffi::Error::Success();
  return ffi::Error::InvalidArgument(std::string(where) + ": " + mdattn_strerror(rc));
}

// layout 0: [B,S,H,D]   layout 1: [B,H,S,D]; returns logical (B,S,H,D) and element strides
bool Describe(ffi::Span<const int64_t> dims, int64_t layout, int64_t* B, int64_t* S, int64_t* H, int64_t* D,
              mdattn_strides* st) {
  if (dims.size() != 4) return false;
  *B = dims[0];
  *D = dims[3];
  if (layout == 0) {
    *S = dims[1]; *H = dims[2];
    st->batch = dims[1] * dims[2] * dims[3]; st->seq = dims[2] * dims[3]; st->head = dims[3];
  } else {
    *H = dims[1]; *S = dims[2];
    st->batch = dims[1] * dims[2] * dims[3]; st->head = dims[2] * dims[3]; st->seq = dims[3];
  }
  return true;
}

ffi::Error FwdBf16Impl(hipStream_t stream, ffi::AnyBuffer q, ffi::AnyBuffer k, ffi::AnyBuffer v,
                       ffi::Result<ffi::AnyBuffer> out, ffi::Result<ffi::AnyBuffer> lse, float scale, int64_t layout) {
  if (q.element_type() != ffi::BF16 || k.element_type() != ffi::BF16 || v.element_type() != ffi::BF16 ||
      out->element_type() != ffi::BF16 || lse->element_type() != ffi::F32)
    return ffi::Error::InvalidArgument("mdattn_fwd_bf16: q, k, v, out must be bf16 and lse f32");
  int64_t B, Sq, H, D, Bk, Skv, Hk, Dk, Bo, So, Ho, Do;
  mdattn_strides sq, sk, sv, so;
  if (!Describe(q.dimensions(), layout, &B, &Sq, &H, &D, &sq) || !Describe(k.dimensions(), layout, &Bk, &Skv, &Hk, &Dk, &sk) ||
      !Describe(v.dimensions(), layout, &Bk, &Skv, &Hk, &Dk, &sv) || !Describe(out->dimensions(), 0, &Bo, &So, &Ho, &Do, &so))
    return ffi::Error::InvalidArgument("mdattn_fwd_bf16: rank-4 buffers expected");
  if (Bk != B || Hk != H || Dk != D || Bo != B || So != Sq || Ho != H || Do != D)
    return ffi::Error::InvalidArgument("mdattn_fwd_bf16: inconsistent shapes");
  return ToError(mdattn_fwd_bf16(stream, q.untyped_data(), k.untyped_data(), v.untyped_data(), out->untyped_data(),
                                 static_cast<float*>(lse->untyped_data()), (int)B, (int)H, (int)Sq, (int)Skv, (int)D,
                                 &sq, &sk, &sv, &so, scale),
                 "mdattn_fwd_bf16");
}

// key_bias: f32 [B, P] with P a multiple of 32 and >= Skv rounded up to 32 (0 keeps a key, -inf excludes it)
ffi::Error FwdBf16BiasImpl(hipStream_t stream, ffi::AnyBuffer q, ffi::AnyBuffer k, ffi::AnyBuffer v, ffi::AnyBuffer key_bias,
                           ffi::Result<ffi::AnyBuffer> out, ffi::Result<ffi::AnyBuffer> lse, float scale, int64_t layout) {
  if (q.element_type() != ffi::BF16 || k.element_type() != ffi::BF16 || v.element_type() != ffi::BF16 ||
      out->element_type() != ffi::BF16 || lse->element_type() != ffi::F32 || key_bias.element_type() != ffi::F32)
    return ffi::Error::InvalidArgument("mdattn_fwd_bf16_bias: q, k, v, out must be bf16, key_bias and lse f32");
  int64_t B, Sq, H, D, Bk, Skv, Hk, Dk, Bo, So, Ho, Do;
  mdattn_strides sq, sk, sv, so;
  if (!Describe(q.dimensions(), layout, &B, &Sq, &H, &D, &sq) || !Describe(k.dimensions(), layout, &Bk, &Skv, &Hk, &Dk, &sk) ||
      !Describe(v.dimensions(), layout, &Bk, &Skv, &Hk, &Dk, &sv) || !Describe(out->dimensions(), 0, &Bo, &So, &Ho, &Do, &so))
    return ffi::Error::InvalidArgument("mdattn_fwd_bf16_bias: rank-4 buffers expected");
  auto bd = key_bias.dimensions();
  if (Bk != B || Hk != H || Dk != D || Bo != B || So != Sq || Ho != H || Do != D || bd.size() != 2 || bd[0] != B)
    return ffi::Error::InvalidArgument("mdattn_fwd_bf16_bias: inconsistent shapes");
  return ToError(mdattn_fwd_bf16_bias(stream, q.untyped_data(), k.untyped_data(), v.untyped_data(), out->untyped_data(),
                                      static_cast<float*>(lse->untyped_data()), (int)B, (int)H, (int)Sq, (int)Skv, (int)D,
                                      &sq, &sk, &sv, &so, scale, static_cast<const float*>(key_bias.untyped_data()), bd[1]),
                 "mdattn_fwd_bf16_bias");
}

ffi::Error NormRopeFullrowImpl(hipStream_t stream, ffi::AnyBuffer q, ffi::AnyBuffer k, ffi::AnyBuffer wq, ffi::AnyBuffer wk,
                               ffi::AnyBuffer cos, ffi::AnyBuffer sin, ffi::Result<ffi::AnyBuffer> q_out,
                               ffi::Result<ffi::AnyBuffer> k_out, float eps, float q_mul, int64_t heads, int64_t rope) {
  auto d = q.dimensions();
  if (d.size() != 3 || heads <= 0 || d[2] % heads) return ffi::Error::InvalidArgument("mdattn_norm_rope_fullrow: q must be [B,S,H*D]");
  const int64_t B = d[0], S = d[1], N = d[2], D = N / heads;
  mdattn_strides so{S * N, N, D};  // q_out/k_out are [B,S,H,D]
  return ToError(mdattn_norm_rope_fullrow(stream, q.untyped_data(), k.untyped_data(), q_out->untyped_data(), k_out->untyped_data(),
                                          wq.untyped_data(), wk.untyped_data(),
                                          rope ? static_cast<const float*>(cos.untyped_data()) : nullptr,
                                          rope ? static_cast<const float*>(sin.untyped_data()) : nullptr,
                                          (int)B, (int)S, (int)heads, (int)D, eps, q_mul, S * N, N, &so),
                 "mdattn_norm_rope_fullrow");
}

ffi::Error NormRopePerheadImpl(hipStream_t stream, ffi::AnyBuffer q, ffi::AnyBuffer k, ffi::AnyBuffer wq, ffi::AnyBuffer wk,
                               ffi::AnyBuffer cos, ffi::AnyBuffer sin, ffi::Result<ffi::AnyBuffer> q_out,
                               ffi::Result<ffi::AnyBuffer> k_out, float eps, float q_mul, int64_t rope) {
  int64_t B, S, H, D;
  mdattn_strides si;
  if (!Describe(q.dimensions(), 0, &B, &S, &H, &D, &si)) return ffi::Error::InvalidArgument("mdattn_norm_rope_perhead: q must be [B,S,H,D]");
  return ToError(mdattn_norm_rope_perhead(stream, q.untyped_data(), k.untyped_data(), q_out->untyped_data(), k_out->untyped_data(),
                                          wq.untyped_data(), wk.untyped_data(), nullptr, nullptr, 0,
                                          rope ? static_cast<const float*>(cos.untyped_data()) : nullptr,
                                          rope ? static_cast<const float*>(sin.untyped_data()) : nullptr,
                                          (int)B, (int)S, (int)H, (int)D, eps, q_mul, &si, &si),
                 "mdattn_norm_rope_perhead");
}

// q, out, dout, dq [B,Sq,H,D]; k, v, dk, dv [B,Skv,H,D] (layout 0); lse f32 [B,H,Sq]; workspace f32 [>= mdattn_bwd_workspace_floats]
ffi::Error BwdBf16Impl(hipStream_t stream, ffi::AnyBuffer q, ffi::AnyBuffer k, ffi::AnyBuffer v, ffi::AnyBuffer out,
                       ffi::AnyBuffer dout, ffi::AnyBuffer lse, ffi::Result<ffi::AnyBuffer> dq, ffi::Result<ffi::AnyBuffer> dk,
                       ffi::Result<ffi::AnyBuffer> dv, ffi::Result<ffi::AnyBuffer> workspace, float scale) {
  int64_t B, Sq, H, D, Bk, Skv, Hk, Dk;
  mdattn_strides sq, sk;
  if (!Describe(q.dimensions(), 0, &B, &Sq, &H, &D, &sq) || !Describe(k.dimensions(), 0, &Bk, &Skv, &Hk, &Dk, &sk))
    return ffi::Error::InvalidArgument("mdattn_bwd_bf16: rank-4 [B,S,H,D] buffers expected");
  if (Bk != B || Hk != H || Dk != D) return ffi::Error::InvalidArgument("mdattn_bwd_bf16: inconsistent shapes");
  return ToError(mdattn_bwd_bf16(stream, q.untyped_data(), k.untyped_data(), v.untyped_data(), out.untyped_data(),
                                 dout.untyped_data(), static_cast<const float*>(lse.untyped_data()), dq->untyped_data(),
                                 dk->untyped_data(), dv->untyped_data(), static_cast<float*>(workspace->untyped_data()),
                                 (int64_t)workspace->element_count(), (int)B, (int)H, (int)Sq, (int)Skv, (int)D, &sq, &sk, &sk, &sq, scale),
                 "mdattn_bwd_bf16");
}

// x [B,S,H*D] bf16 or f32; w f32 [H*D]; cos/sin f32 [B,S,H*D] (mode 1) or [B,H,S,D/2] (mode 2), ignored for mode 0
ffi::Error NormRopeRowsImpl(hipStream_t stream, ffi::AnyBuffer x, ffi::AnyBuffer w, ffi::AnyBuffer cos, ffi::AnyBuffer sin,
                            ffi::Result<ffi::AnyBuffer> x_out, float eps, int64_t heads, int64_t mode) {
  auto d = x.dimensions();
  if (d.size() != 3 || heads <= 0 || d[2] % heads) return ffi::Error::InvalidArgument("mdattn_norm_rope_rows: x must be [B,S,H*D]");
  if (x.element_type() != ffi::BF16 && x.element_type() != ffi::F32) return ffi::Error::InvalidArgument("mdattn_norm_rope_rows: x must be bf16 or f32");
  const int64_t B = d[0], S = d[1], N = d[2], D = N / heads;
  mdattn_strides so{S * N, N, D};  // x_out is [B,S,H,D]
  return ToError(mdattn_norm_rope_rows(stream, x.untyped_data(), x.element_type() == ffi::F32, x_out->untyped_data(),
                                       static_cast<const float*>(w.untyped_data()),
                                       mode ? static_cast<const float*>(cos.untyped_data()) : nullptr,
                                       mode ? static_cast<const float*>(sin.untyped_data()) : nullptr, (int)mode,
                                       (int)B, (int)S, (int)heads, (int)D, eps, q_mul, S * N, N, &so),
                 "mdattn_norm_rope_rows");
}

// o_run / lse_run are donated by the caller (input_output_aliases) and updated in place.
ffi::Error MergeImpl(hipStream_t stream, ffi::AnyBuffer o_run_in, ffi::AnyBuffer lse_run_in, ffi::AnyBuffer o_cur,
                     ffi::AnyBuffer lse_cur, ffi::Result<ffi::AnyBuffer> o_run, ffi::Result<ffi::AnyBuffer> lse_run) {
  if (o_run->untyped_data() != o_run_in.untyped_data() || lse_run->untyped_data() != lse_run_in.untyped_data())
    return ffi::Error::InvalidArgument("mdattn_merge: o_run and lse_run must alias their outputs (input_output_aliases={0:0,1:1})");
  int64_t B, S, H, D;
  mdattn_strides st;
  if (!Describe(o_cur.dimensions(), 0, &B, &S, &H, &D, &st)) return ffi::Error::InvalidArgument("mdattn_merge: o_cur must be [B,S,H,D]");
  return ToError(mdattn_merge(stream, static_cast<float*>(o_run->untyped_data()), static_cast<float*>(lse_run->untyped_data()),
                              o_cur.untyped_data(), static_cast<const float*>(lse_cur.untyped_data()),
                              o_cur.element_type() == ffi::F32, (int)B, (int)H, (int)S, (int)D, &st, &st),
                 "mdattn_merge");
}

// One ring hop: attention of q against the visiting K/V chunk, merged into the donated (o_run, lse_run) in one launch.
ffi::Error FwdBf16MergeImpl(hipStream_t stream, ffi::AnyBuffer q, ffi::AnyBuffer k, ffi::AnyBuffer v,
                            ffi::AnyBuffer o_run_in, ffi::AnyBuffer lse_run_in, ffi::Result<ffi::AnyBuffer> o_run,
                            ffi::Result<ffi::AnyBuffer> lse_run, float scale, int64_t layout) {
  if (o_run->untyped_data() != o_run_in.untyped_data() || lse_run->untyped_data() != lse_run_in.untyped_data())
    return ffi::Error::InvalidArgument("mdattn_fwd_bf16_merge: o_run and lse_run must alias their outputs (input_output_aliases={3:0,4:1})");
  if (q.element_type() != ffi::BF16 || k.element_type() != ffi::BF16 || v.element_type() != ffi::BF16 ||
      o_run->element_type() != ffi::F32 || lse_run->element_type() != ffi::F32)
    return ffi::Error::InvalidArgument("mdattn_fwd_bf16_merge: q, k, v must be bf16, o_run and lse_run f32");
  int64_t B, Sq, H, D, Bk, Skv, Hk, Dk, Bo, So, Ho, Do;
  mdattn_strides sq, sk, sv, so;
  if (!Describe(q.dimensions(), layout, &B, &Sq, &H, &D, &sq) || !Describe(k.dimensions(), layout, &Bk, &Skv, &Hk, &Dk, &sk) ||
      !Describe(v.dimensions(), layout, &Bk, &Skv, &Hk, &Dk, &sv) || !Describe(o_run->dimensions(), 0, &Bo, &So, &Ho, &Do, &so))
    return ffi::Error::InvalidArgument("mdattn_fwd_bf16_merge: rank-4 buffers expected");
  if (Bk != B || Hk != H || Dk != D || Bo != B || So != Sq || Ho != H || Do != D)
    return ffi::Error::InvalidArgument("mdattn_fwd_bf16_merge: inconsistent shapes");
  return ToError(mdattn_fwd_bf16_merge(stream, q.untyped_data(), k.untyped_data(), v.untyped_data(),
                                       static_cast<float*>(o_run->untyped_data()), static_cast<float*>(lse_run->untyped_data()),
                                       (int)B, (int)H, (int)Sq, (int)Skv, (int)D, &sq, &sk, &sv, &so, scale),
                 "mdattn_fwd_bf16_merge");
}

}  // namespace

XLA_FFI_DEFINE_HANDLER_SYMBOL(MdattnFwdBf16, FwdBf16Impl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>()
                                  .Attr<float>("scale").Attr<int64_t>("layout"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(MdattnFwdBf16Bias, FwdBf16BiasImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>()
                                  .Attr<float>("scale").Attr<int64_t>("layout"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(MdattnNormRopeFullrow, NormRopeFullrowImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>()
                                  .Attr<float>("eps").Attr<float>("q_mul").Attr<int64_t>("heads").Attr<int64_t>("rope"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(MdattnBwdBf16, BwdBf16Impl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>()
                                  .Attr<float>("scale"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(MdattnNormRopeRows, NormRopeRowsImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Attr<float>("eps").Attr<int64_t>("heads").Attr<int64_t>("mode"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(MdattnNormRopePerhead, NormRopePerheadImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>()
                                  .Attr<float>("eps").Attr<float>("q_mul").Attr<int64_t>("rope"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(MdattnMerge, MergeImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>());

XLA_FFI_DEFINE_HANDLER_SYMBOL(MdattnFwdBf16Merge, FwdBf16MergeImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>()
                                  .Attr<float>("scale").Attr<int64_t>("layout"));
