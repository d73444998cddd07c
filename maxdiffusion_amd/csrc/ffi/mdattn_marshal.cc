// Bodies of the XLA custom-call handlers on plain structs (include/mdattn_marshal.h): shape and dtype checks, the
// translation of dense row-major buffers into the pointers, sizes and strides of the C ABI, the call.  No XLA header,
// no HIP call: this file is part of libmdattn.so and is tested through ctypes on machines without jaxlib or a GPU.
#include "mdattn_marshal.h"

#include <cstdarg>
#include <cstdio>

namespace {

struct Err {
  char* buf;
  int len;
  const char* where;
  // formats "<where>: <message>" into the caller's buffer and returns `code`
  int fail(int code, const char* fmt, ...) const {
    if (buf && len > 0) {
      int n = snprintf(buf, (size_t)len, "%s: ", where);
      if (n < 0) n = 0;
      if (n < len) {
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(buf + n, (size_t)(len - n), fmt, ap);
        va_end(ap);
      }
      buf[len - 1] = 0;
    }
    return code;
  }
  // turns a C-ABI return code into the handler's: adds the library's own text
  int from(int rc) const {
    if (rc != MDATTN_OK) return fail(rc, "%s", mdattn_strerror(rc));
    if (buf && len > 0) buf[0] = 0;
    return rc;
  }
};

const char* dt_name(int dt) {
  switch (dt) {
    case MDATTN_DT_BF16: return "bf16";
    case MDATTN_DT_F32: return "f32";
    case MDATTN_DT_U8: return "u8";
    case MDATTN_DT_F8E4M3FN: return "f8e4m3fn";
    default: return "another dtype";
  }
}

bool ok_buffer(const mdattn_buffer* b) {
  if (!b || !b->data || b->rank < 0 || (b->rank > 0 && !b->dims)) return false;
  for (int i = 0; i < b->rank; ++i)
    if (b->dims[i] <= 0) return false;
  return true;
}
int64_t count(const mdattn_buffer* b) {
  int64_t n = 1;
  for (int i = 0; i < b->rank; ++i) n *= b->dims[i];
  return n;
}
bool is_fp8(const mdattn_buffer* b) { return b->dtype == MDATTN_DT_U8 || b->dtype == MDATTN_DT_F8E4M3FN; }
bool fits_int(int64_t x) { return x > 0 && x <= 0x7FFFFFFF; }

// A rank-4 attention operand: logical (B, S, H, D) and element strides of a dense buffer in `layout`.
struct View4 {
  int64_t B, S, H, D;
  mdattn_strides st;
};
bool describe(const mdattn_buffer* b, int64_t layout, View4* v) {
  if (b->rank != 4) return false;
  const int64_t* d = b->dims;
  v->B = d[0];
  v->D = d[3];
  v->st.batch = d[1] * d[2] * d[3];
  if (layout == 0) {
    v->S = d[1]; v->H = d[2];
    v->st.seq = d[2] * d[3]; v->st.head = d[3];
  } else {
    v->H = d[1]; v->S = d[2];
    v->st.head = d[2] * d[3]; v->st.seq = d[3];
  }
  return fits_int(v->B) && fits_int(v->S) && fits_int(v->H) && fits_int(v->D);
}

#define CHECK_BUF(e, b, name) \
  if (!ok_buffer(b)) return (e).fail(MDATTN_E_BADARG, "%s is missing, empty or has a null pointer", name)
#define CHECK_DT(e, b, name, want) \
  if ((b)->dtype != (want)) return (e).fail(MDATTN_E_BADARG, "%s must be %s, got %s", name, dt_name(want), dt_name((b)->dtype))

// q, k, v in `layout`, out [B,Sq,H,D], lse [B,H,Sq]: the checks every forward handler shares
int check_qkv(const Err& e, const mdattn_buffer* q, const mdattn_buffer* k, const mdattn_buffer* v, int64_t layout, bool fp8,
              View4* vq, View4* vk, View4* vv) {
  CHECK_BUF(e, q, "q"); CHECK_BUF(e, k, "k"); CHECK_BUF(e, v, "v");
  if (layout != 0 && layout != 1) return e.fail(MDATTN_E_BADARG, "layout must be 0 ([B,S,H,D]) or 1 ([B,H,S,D]), got %lld", (long long)layout);
  if (fp8) {
    if (!is_fp8(q) || !is_fp8(k) || !is_fp8(v)) return e.fail(MDATTN_E_BADARG, "q8, k8, v8 must be u8 or f8e4m3fn buffers");
  } else {
    CHECK_DT(e, q, "q", MDATTN_DT_BF16); CHECK_DT(e, k, "k", MDATTN_DT_BF16); CHECK_DT(e, v, "v", MDATTN_DT_BF16);
  }
  if (!describe(q, layout, vq) || !describe(k, layout, vk) || !describe(v, layout, vv))
    return e.fail(MDATTN_E_BADARG, "q, k, v must be rank-4 buffers");
  if (vk->B != vq->B || vk->H != vq->H || vk->D != vq->D)
    return e.fail(MDATTN_E_BADARG, "k [B=%lld,S=%lld,H=%lld,D=%lld] does not match q [B=%lld,S=%lld,H=%lld,D=%lld] in batch, heads or depth",
                  (long long)vk->B, (long long)vk->S, (long long)vk->H, (long long)vk->D, (long long)vq->B, (long long)vq->S, (long long)vq->H, (long long)vq->D);
  if (vv->B != vk->B || vv->S != vk->S || vv->H != vk->H || vv->D != vk->D) return e.fail(MDATTN_E_BADARG, "k and v must have the same shape");
  return MDATTN_OK;
}
int check_out_bshd(const Err& e, const mdattn_buffer* out, const char* name, int want_dt, const View4& vq, View4* vo) {
  CHECK_BUF(e, out, name);
  CHECK_DT(e, out, name, want_dt);
  if (!describe(out, 0, vo) || vo->B != vq.B || vo->S != vq.S || vo->H != vq.H || vo->D != vq.D)
    return e.fail(MDATTN_E_BADARG, "%s must be [B,Sq,H,D] = [%lld,%lld,%lld,%lld]", name, (long long)vq.B, (long long)vq.S, (long long)vq.H, (long long)vq.D);
  return MDATTN_OK;
}
int check_lse(const Err& e, const mdattn_buffer* lse, const char* name, const View4& vq) {
  CHECK_BUF(e, lse, name);
  CHECK_DT(e, lse, name, MDATTN_DT_F32);
  if (lse->rank != 3 || lse->dims[0] != vq.B || lse->dims[1] != vq.H || lse->dims[2] != vq.S)
    return e.fail(MDATTN_E_BADARG, "%s must be [B,H,Sq] = [%lld,%lld,%lld]", name, (long long)vq.B, (long long)vq.H, (long long)vq.S);
  return MDATTN_OK;
}
int check_alias(const Err& e, const mdattn_buffer* in, const mdattn_buffer* out, const char* name, const char* aliases) {
  CHECK_BUF(e, in, name);
  CHECK_BUF(e, out, name);
  if (in->data != out->data)
    return e.fail(MDATTN_E_BADARG, "%s must be donated: the result has to alias the input (input_output_aliases=%s)", name, aliases);
  return MDATTN_OK;
}
int check_vec(const Err& e, const mdattn_buffer* b, const char* name, int want_dt, int64_t n) {
  CHECK_BUF(e, b, name);
  CHECK_DT(e, b, name, want_dt);
  if (count(b) != n) return e.fail(MDATTN_E_BADARG, "%s must hold %lld elements, got %lld", name, (long long)n, (long long)count(b));
  return MDATTN_OK;
}
#define TRY(expr)                  \
  do {                             \
    const int rc_ = (expr);        \
    if (rc_ != MDATTN_OK) return rc_; \
  } while (0)

}  // namespace

extern "C" int mdattn_xla_fwd_bf16(void* stream, const mdattn_buffer* q, const mdattn_buffer* k, const mdattn_buffer* v,
                                   const mdattn_buffer* out, const mdattn_buffer* lse, float scale, int64_t layout,
                                   char* err, int err_len) {
  const Err e{err, err_len, "mdattn_fwd_bf16"};
  View4 vq, vk, vv, vo;
  TRY(check_qkv(e, q, k, v, layout, false, &vq, &vk, &vv));
  TRY(check_out_bshd(e, out, "out", MDATTN_DT_BF16, vq, &vo));
  TRY(check_lse(e, lse, "lse", vq));
  return e.from(mdattn_fwd_bf16(stream, q->data, k->data, v->data, out->data, static_cast<float*>(lse->data), (int)vq.B, (int)vq.H,
                                (int)vq.S, (int)vk.S, (int)vq.D, &vq.st, &vk.st, &vv.st, &vo.st, scale));
}

extern "C" int mdattn_xla_fwd_bf16_bias(void* stream, const mdattn_buffer* q, const mdattn_buffer* k, const mdattn_buffer* v,
                                        const mdattn_buffer* key_bias, const mdattn_buffer* out, const mdattn_buffer* lse,
                                        float scale, int64_t layout, char* err, int err_len) {
  const Err e{err, err_len, "mdattn_fwd_bf16_bias"};
  View4 vq, vk, vv, vo;
  TRY(check_qkv(e, q, k, v, layout, false, &vq, &vk, &vv));
  TRY(check_out_bshd(e, out, "out", MDATTN_DT_BF16, vq, &vo));
  TRY(check_lse(e, lse, "lse", vq));
  CHECK_BUF(e, key_bias, "key_bias");
  CHECK_DT(e, key_bias, "key_bias", MDATTN_DT_F32);
  const int64_t padded = (vk.S + 31) / 32 * 32;
  if (key_bias->rank != 2 || key_bias->dims[0] != vq.B || key_bias->dims[1] != padded)
    return e.fail(MDATTN_E_BADARG, "key_bias must be [B, Skv rounded up to 32] = [%lld,%lld] (padding filled with the masked value)",
                  (long long)vq.B, (long long)padded);
  return e.from(mdattn_fwd_bf16_bias(stream, q->data, k->data, v->data, out->data, static_cast<float*>(lse->data), (int)vq.B, (int)vq.H,
                                     (int)vq.S, (int)vk.S, (int)vq.D, &vq.st, &vk.st, &vv.st, &vo.st, scale,
                                     static_cast<const float*>(key_bias->data), padded));
}

extern "C" int mdattn_xla_key_mask_bias(void* stream, const mdattn_buffer* keep, const mdattn_buffer* bias, float masked_value,
                                        char* err, int err_len) {
  const Err e{err, err_len, "mdattn_key_mask_bias"};
  CHECK_BUF(e, keep, "keep");
  CHECK_BUF(e, bias, "bias");
  CHECK_DT(e, keep, "keep", MDATTN_DT_U8);
  CHECK_DT(e, bias, "bias", MDATTN_DT_F32);
  if (keep->rank != 2) return e.fail(MDATTN_E_BADARG, "attention_mask must have shape [batch, kv_length], got rank %d", keep->rank);
  const int64_t B = keep->dims[0], Skv = keep->dims[1], padded = (Skv + 31) / 32 * 32;
  if (!fits_int(B) || !fits_int(Skv)) return e.fail(MDATTN_E_UNSUPPORTED, "mask dimensions beyond 2^31");
  if (bias->rank != 2 || bias->dims[0] != B || bias->dims[1] != padded)
    return e.fail(MDATTN_E_BADARG, "bias must be [B, Skv rounded up to 32] = [%lld,%lld]", (long long)B, (long long)padded);
  return e.from(mdattn_key_mask_bias(stream, keep->data, static_cast<float*>(bias->data), (int)B, (int)Skv, padded, masked_value));
}

extern "C" int mdattn_xla_fwd_bf16_merge(void* stream, const mdattn_buffer* q, const mdattn_buffer* k, const mdattn_buffer* v,
                                         const mdattn_buffer* o_run_in, const mdattn_buffer* lse_run_in,
                                         const mdattn_buffer* o_run, const mdattn_buffer* lse_run, float scale, int64_t layout,
                                         char* err, int err_len) {
  const Err e{err, err_len, "mdattn_fwd_bf16_merge"};
  View4 vq, vk, vv, vo;
  TRY(check_qkv(e, q, k, v, layout, false, &vq, &vk, &vv));
  TRY(check_alias(e, o_run_in, o_run, "o_run", "{3: 0, 4: 1}"));
  TRY(check_alias(e, lse_run_in, lse_run, "lse_run", "{3: 0, 4: 1}"));
  TRY(check_out_bshd(e, o_run, "o_run", MDATTN_DT_F32, vq, &vo));
  TRY(check_lse(e, lse_run, "lse_run", vq));
  return e.from(mdattn_fwd_bf16_merge(stream, q->data, k->data, v->data, static_cast<float*>(o_run->data),
                                      static_cast<float*>(lse_run->data), (int)vq.B, (int)vq.H, (int)vq.S, (int)vk.S, (int)vq.D,
                                      &vq.st, &vk.st, &vv.st, &vo.st, scale));
}

extern "C" int mdattn_xla_merge(void* stream, const mdattn_buffer* o_run_in, const mdattn_buffer* lse_run_in,
                                const mdattn_buffer* o_cur, const mdattn_buffer* lse_cur, const mdattn_buffer* o_run,
                                const mdattn_buffer* lse_run, char* err, int err_len) {
  const Err e{err, err_len, "mdattn_merge"};
  TRY(check_alias(e, o_run_in, o_run, "o_run", "{0: 0, 1: 1}"));
  TRY(check_alias(e, lse_run_in, lse_run, "lse_run", "{0: 0, 1: 1}"));
  CHECK_BUF(e, o_cur, "o_cur");
  if (o_cur->dtype != MDATTN_DT_BF16 && o_cur->dtype != MDATTN_DT_F32) return e.fail(MDATTN_E_BADARG, "o_cur must be bf16 or f32, got %s", dt_name(o_cur->dtype));
  View4 vc, vr;
  if (!describe(o_cur, 0, &vc)) return e.fail(MDATTN_E_BADARG, "o_cur must be a rank-4 [B,S,H,D] buffer");
  TRY(check_out_bshd(e, o_run, "o_run", MDATTN_DT_F32, vc, &vr));
  TRY(check_lse(e, lse_run, "lse_run", vc));
  TRY(check_lse(e, lse_cur, "lse_cur", vc));
  return e.from(mdattn_merge(stream, static_cast<float*>(o_run->data), static_cast<float*>(lse_run->data), o_cur->data,
                             static_cast<const float*>(lse_cur->data), o_cur->dtype == MDATTN_DT_F32, (int)vc.B, (int)vc.H, (int)vc.S,
                             (int)vc.D, &vr.st, &vc.st));
}

extern "C" int mdattn_xla_finalize(void* stream, const mdattn_buffer* o_run, const mdattn_buffer* out, char* err, int err_len) {
  const Err e{err, err_len, "mdattn_finalize"};
  CHECK_BUF(e, o_run, "o_run");
  CHECK_BUF(e, out, "out");
  CHECK_DT(e, o_run, "o_run", MDATTN_DT_F32);
  CHECK_DT(e, out, "out", MDATTN_DT_BF16);
  if (count(o_run) != count(out)) return e.fail(MDATTN_E_BADARG, "o_run and out must have the same number of elements");
  return e.from(mdattn_finalize(stream, static_cast<const float*>(o_run->data), out->data, count(o_run)));
}

extern "C" int mdattn_xla_norm_rope_fullrow(void* stream, const mdattn_buffer* q, const mdattn_buffer* k, const mdattn_buffer* wq,
                                            const mdattn_buffer* wk, const mdattn_buffer* cos, const mdattn_buffer* sin,
                                            const mdattn_buffer* q_out, const mdattn_buffer* k_out, float eps, float q_mul,
                                            int64_t heads, int64_t rope, int64_t has_k, char* err, int err_len) {
  const Err e{err, err_len, "mdattn_norm_rope_fullrow"};
  CHECK_BUF(e, q, "q");
  CHECK_DT(e, q, "q", MDATTN_DT_BF16);
  if (q->rank != 3 || heads <= 0 || q->dims[2] % heads) return e.fail(MDATTN_E_BADARG, "q must be [B,S,H*D] with H = heads = %lld", (long long)heads);
  const int64_t B = q->dims[0], S = q->dims[1], N = q->dims[2], D = N / heads;
  if (!fits_int(B) || !fits_int(S) || !fits_int(N)) return e.fail(MDATTN_E_UNSUPPORTED, "dimensions beyond 2^31");
  const int64_t shape4[4] = {B, S, heads, D};
  auto is_bshd = [&](const mdattn_buffer* b) {
    return b->rank == 4 && b->dims[0] == shape4[0] && b->dims[1] == shape4[1] && b->dims[2] == shape4[2] && b->dims[3] == shape4[3];
  };
  TRY(check_vec(e, wq, "wq", MDATTN_DT_BF16, N));
  CHECK_BUF(e, q_out, "q_out");
  CHECK_DT(e, q_out, "q_out", MDATTN_DT_BF16);
  if (!is_bshd(q_out)) return e.fail(MDATTN_E_BADARG, "q_out must be [B,S,H,D] = [%lld,%lld,%lld,%lld]", (long long)B, (long long)S, (long long)heads, (long long)D);
  if (has_k) {
    CHECK_BUF(e, k, "k");
    CHECK_DT(e, k, "k", MDATTN_DT_BF16);
    if (k->rank != 3 || k->dims[0] != B || k->dims[1] != S || k->dims[2] != N) return e.fail(MDATTN_E_BADARG, "k must have q's shape");
    TRY(check_vec(e, wk, "wk", MDATTN_DT_BF16, N));
    CHECK_BUF(e, k_out, "k_out");
    CHECK_DT(e, k_out, "k_out", MDATTN_DT_BF16);
    if (!is_bshd(k_out)) return e.fail(MDATTN_E_BADARG, "k_out must have q_out's shape");
  }
  if (rope) {
    TRY(check_vec(e, cos, "cos", MDATTN_DT_F32, S * (D / 2)));
    TRY(check_vec(e, sin, "sin", MDATTN_DT_F32, S * (D / 2)));
  }
  const mdattn_strides so{S * N, N, D};
  return e.from(mdattn_norm_rope_fullrow(stream, q->data, has_k ? k->data : nullptr, q_out->data, has_k ? k_out->data : nullptr,
                                         wq->data, has_k ? wk->data : nullptr, rope ? static_cast<const float*>(cos->data) : nullptr,
                                         rope ? static_cast<const float*>(sin->data) : nullptr, (int)B, (int)S, (int)heads, (int)D, eps,
                                         q_mul, S * N, N, &so));
}

extern "C" int mdattn_xla_norm_rope_qkv(void* stream, const mdattn_buffer* qkv, const mdattn_buffer* bias, const mdattn_buffer* wq,
                                        const mdattn_buffer* wk, const mdattn_buffer* cos, const mdattn_buffer* sin,
                                        const mdattn_buffer* q_out, const mdattn_buffer* k_out, const mdattn_buffer* v_out, float eps,
                                        float q_mul, int64_t heads, int64_t rope, int64_t has_bias, int64_t has_v, char* err,
                                        int err_len) {
  const Err e{err, err_len, "mdattn_norm_rope_qkv"};
  CHECK_BUF(e, qkv, "qkv");
  CHECK_DT(e, qkv, "qkv", MDATTN_DT_BF16);
  if (qkv->rank != 3 || heads <= 0 || qkv->dims[2] % (3 * heads))
    return e.fail(MDATTN_E_BADARG, "qkv must be [B,S,3*H*D] with H = heads = %lld", (long long)heads);
  const int64_t B = qkv->dims[0], S = qkv->dims[1], N = qkv->dims[2] / 3, D = N / heads;
  if (!fits_int(B) || !fits_int(S) || !fits_int(3 * N)) return e.fail(MDATTN_E_UNSUPPORTED, "dimensions beyond 2^31");
  if (has_bias && !has_v) return e.fail(MDATTN_E_BADARG, "with a bias the value block needs its bias too: has_v must be set");
  auto is_bshd = [&](const mdattn_buffer* b) {
    return b->rank == 4 && b->dims[0] == B && b->dims[1] == S && b->dims[2] == heads && b->dims[3] == D;
  };
  const mdattn_buffer* outs[3] = {q_out, k_out, v_out};
  const char* names[3] = {"q_out", "k_out", "v_out"};
  for (int i = 0; i < (has_v ? 3 : 2); ++i) {
    CHECK_BUF(e, outs[i], names[i]);
    CHECK_DT(e, outs[i], names[i], MDATTN_DT_BF16);
    if (!is_bshd(outs[i]))
      return e.fail(MDATTN_E_BADARG, "%s must be [B,S,H,D] = [%lld,%lld,%lld,%lld]", names[i], (long long)B, (long long)S, (long long)heads, (long long)D);
  }
  TRY(check_vec(e, wq, "wq", MDATTN_DT_BF16, N));
  TRY(check_vec(e, wk, "wk", MDATTN_DT_BF16, N));
  if (has_bias) TRY(check_vec(e, bias, "bias", MDATTN_DT_BF16, 3 * N));
  if (rope) {
    TRY(check_vec(e, cos, "cos", MDATTN_DT_F32, S * (D / 2)));
    TRY(check_vec(e, sin, "sin", MDATTN_DT_F32, S * (D / 2)));
  }
  const mdattn_strides so{S * N, N, D};
  return e.from(mdattn_norm_rope_qkv(stream, qkv->data, has_bias ? bias->data : nullptr, q_out->data, k_out->data,
                                     has_v ? v_out->data : nullptr, wq->data, wk->data,
                                     rope ? static_cast<const float*>(cos->data) : nullptr,
                                     rope ? static_cast<const float*>(sin->data) : nullptr, (int)B, (int)S, (int)heads, (int)D, eps,
                                     q_mul, S * 3 * N, 3 * N, &so));
}

extern "C" int mdattn_xla_norm_rope_perhead(void* stream, const mdattn_buffer* q, const mdattn_buffer* k, const mdattn_buffer* wq,
                                            const mdattn_buffer* wk, const mdattn_buffer* wq_txt, const mdattn_buffer* wk_txt,
                                            const mdattn_buffer* cos, const mdattn_buffer* sin, const mdattn_buffer* q_out,
                                            const mdattn_buffer* k_out, float eps, float q_mul, int64_t n_txt, int64_t rope,
                                            int64_t has_k, char* err, int err_len) {
  const Err e{err, err_len, "mdattn_norm_rope_perhead"};
  CHECK_BUF(e, q, "q");
  CHECK_DT(e, q, "q", MDATTN_DT_BF16);
  View4 vq, vo;
  if (!describe(q, 0, &vq)) return e.fail(MDATTN_E_BADARG, "q must be a rank-4 [B,S,H,D] buffer");
  if (n_txt < 0 || n_txt > vq.S) return e.fail(MDATTN_E_BADARG, "n_txt = %lld is outside [0, S = %lld]", (long long)n_txt, (long long)vq.S);
  TRY(check_vec(e, wq, "wq", MDATTN_DT_BF16, vq.D));
  TRY(check_out_bshd(e, q_out, "q_out", MDATTN_DT_BF16, vq, &vo));
  if (n_txt > 0) TRY(check_vec(e, wq_txt, "wq_txt", MDATTN_DT_BF16, vq.D));
  if (has_k) {
    CHECK_BUF(e, k, "k");
    CHECK_DT(e, k, "k", MDATTN_DT_BF16);
    View4 vk, vko;
    if (!describe(k, 0, &vk) || vk.B != vq.B || vk.S != vq.S || vk.H != vq.H || vk.D != vq.D) return e.fail(MDATTN_E_BADARG, "k must have q's shape");
    TRY(check_vec(e, wk, "wk", MDATTN_DT_BF16, vq.D));
    TRY(check_out_bshd(e, k_out, "k_out", MDATTN_DT_BF16, vq, &vko));
    if (n_txt > 0) TRY(check_vec(e, wk_txt, "wk_txt", MDATTN_DT_BF16, vq.D));
  }
  if (rope) {
    TRY(check_vec(e, cos, "cos", MDATTN_DT_F32, vq.S * (vq.D / 2)));
    TRY(check_vec(e, sin, "sin", MDATTN_DT_F32, vq.S * (vq.D / 2)));
  }
  return e.from(mdattn_norm_rope_perhead(stream, q->data, has_k ? k->data : nullptr, q_out->data, has_k ? k_out->data : nullptr, wq->data,
                                         has_k ? wk->data : nullptr, n_txt > 0 ? wq_txt->data : nullptr,
                                         (n_txt > 0 && has_k) ? wk_txt->data : nullptr, (int)n_txt,
                                         rope ? static_cast<const float*>(cos->data) : nullptr,
                                         rope ? static_cast<const float*>(sin->data) : nullptr, (int)vq.B, (int)vq.S, (int)vq.H, (int)vq.D,
                                         eps, q_mul, &vq.st, &vo.st));
}

extern "C" int mdattn_xla_norm_rope_rows(void* stream, const mdattn_buffer* x, const mdattn_buffer* w, const mdattn_buffer* cos,
                                         const mdattn_buffer* sin, const mdattn_buffer* x_out, float eps, int64_t heads,
                                         int64_t mode, char* err, int err_len) {
  const Err e{err, err_len, "mdattn_norm_rope_rows"};
  CHECK_BUF(e, x, "x");
  if (x->dtype != MDATTN_DT_BF16 && x->dtype != MDATTN_DT_F32) return e.fail(MDATTN_E_BADARG, "x must be bf16 or f32, got %s", dt_name(x->dtype));
  if (x->rank != 3 || heads <= 0 || x->dims[2] % heads) return e.fail(MDATTN_E_BADARG, "x must be [B,S,H*D] with H = heads = %lld", (long long)heads);
  if (mode < 0 || mode > 2) return e.fail(MDATTN_E_BADARG, "mode must be 0 (norm only), 1 (interleaved) or 2 (split), got %lld", (long long)mode);
  const int64_t B = x->dims[0], S = x->dims[1], N = x->dims[2], D = N / heads;
  if (!fits_int(B) || !fits_int(S) || !fits_int(N)) return e.fail(MDATTN_E_UNSUPPORTED, "dimensions beyond 2^31");
  TRY(check_vec(e, w, "w", MDATTN_DT_F32, N));
  CHECK_BUF(e, x_out, "x_out");
  CHECK_DT(e, x_out, "x_out", MDATTN_DT_BF16);
  if (x_out->rank != 4 || x_out->dims[0] != B || x_out->dims[1] != S || x_out->dims[2] != heads || x_out->dims[3] != D)
    return e.fail(MDATTN_E_BADARG, "x_out must be [B,S,H,D] = [%lld,%lld,%lld,%lld]", (long long)B, (long long)S, (long long)heads, (long long)D);
  if (mode) {
    const int64_t n = mode == 1 ? B * S * N : B * heads * S * (D / 2);
    TRY(check_vec(e, cos, "cos", MDATTN_DT_F32, n));
    TRY(check_vec(e, sin, "sin", MDATTN_DT_F32, n));
    const int want_rank = mode == 1 ? 3 : 4;
    if (cos->rank != want_rank || sin->rank != want_rank)
      return e.fail(MDATTN_E_BADARG, "cos and sin must be %s for mode %lld", mode == 1 ? "[B,S,H*D]" : "[B,H,S,D/2]", (long long)mode);
  }
  const mdattn_strides so{S * N, N, D};
  return e.from(mdattn_norm_rope_rows(stream, x->data, x->dtype == MDATTN_DT_F32, x_out->data, static_cast<const float*>(w->data),
                                      mode ? static_cast<const float*>(cos->data) : nullptr,
                                      mode ? static_cast<const float*>(sin->data) : nullptr, (int)mode, (int)B, (int)S, (int)heads, (int)D,
                                      eps, S * N, N, &so));
}

namespace {
bool same_dims(const mdattn_buffer* a, const mdattn_buffer* b) {
  if (a->rank != b->rank) return false;
  for (int i = 0; i < a->rank; ++i)
    if (a->dims[i] != b->dims[i]) return false;
  return true;
}
int check_workspace(const Err& e, const mdattn_buffer* ws, int64_t columns) {
  CHECK_BUF(e, ws, "workspace");
  CHECK_DT(e, ws, "workspace", MDATTN_DT_F32);
  if (count(ws) < columns)
    return e.fail(MDATTN_E_BADARG, "workspace must hold at least %lld floats (one partial row), got %lld", (long long)columns, (long long)count(ws));
  return MDATTN_OK;
}
}  // namespace

extern "C" int mdattn_xla_norm_rope_fullrow_bwd(void* stream, const mdattn_buffer* q, const mdattn_buffer* k, const mdattn_buffer* gq,
                                                const mdattn_buffer* gk, const mdattn_buffer* wq, const mdattn_buffer* wk,
                                                const mdattn_buffer* cos, const mdattn_buffer* sin, const mdattn_buffer* bias,
                                                const mdattn_buffer* dq, const mdattn_buffer* dk, const mdattn_buffer* dwq,
                                                const mdattn_buffer* dwk, const mdattn_buffer* dbias, const mdattn_buffer* workspace,
                                                float eps, float q_mul, int64_t heads, int64_t rope, int64_t has_k, int64_t has_bias,
                                                char* err, int err_len) {
  const Err e{err, err_len, "mdattn_norm_rope_fullrow_bwd"};
  CHECK_BUF(e, q, "q");
  CHECK_DT(e, q, "q", MDATTN_DT_BF16);
  if (q->rank != 3 || heads <= 0 || q->dims[2] % heads) return e.fail(MDATTN_E_BADARG, "q must be [B,S,H*D] with H = heads = %lld", (long long)heads);
  const int64_t B = q->dims[0], S = q->dims[1], N = q->dims[2], D = N / heads;
  if (!fits_int(B) || !fits_int(S) || !fits_int(N)) return e.fail(MDATTN_E_UNSUPPORTED, "dimensions beyond 2^31");
  if (has_bias && !has_k) return e.fail(MDATTN_E_BADARG, "has_bias needs has_k (the fused q|k|v form carries both tensors)");
  auto is_bshd = [&](const mdattn_buffer* b) {
    return b->rank == 4 && b->dims[0] == B && b->dims[1] == S && b->dims[2] == heads && b->dims[3] == D;
  };
  auto check_side = [&](const mdattn_buffer* x, const mdattn_buffer* g, const mdattn_buffer* w, const mdattn_buffer* dx,
                        const mdattn_buffer* dw, const char* nx, const char* ng, const char* nw, const char* ndx, const char* ndw) -> int {
    CHECK_BUF(e, x, nx); CHECK_DT(e, x, nx, MDATTN_DT_BF16);
    if (!same_dims(x, q)) return e.fail(MDATTN_E_BADARG, "%s must have q's shape", nx);
    CHECK_BUF(e, g, ng); CHECK_DT(e, g, ng, MDATTN_DT_BF16);
    if (!is_bshd(g)) return e.fail(MDATTN_E_BADARG, "%s must be [B,S,H,D] = [%lld,%lld,%lld,%lld]", ng, (long long)B, (long long)S, (long long)heads, (long long)D);
    TRY(check_vec(e, w, nw, MDATTN_DT_BF16, N));
    CHECK_BUF(e, dx, ndx); CHECK_DT(e, dx, ndx, MDATTN_DT_BF16);
    if (!same_dims(dx, q)) return e.fail(MDATTN_E_BADARG, "%s must have q's shape", ndx);
    TRY(check_vec(e, dw, ndw, MDATTN_DT_F32, N));
    return MDATTN_OK;
  };
  TRY(check_side(q, gq, wq, dq, dwq, "q", "gq", "wq", "dq", "dwq"));
  if (has_k) TRY(check_side(k, gk, wk, dk, dwk, "k", "gk", "wk", "dk", "dwk"));
  if (rope) {
    TRY(check_vec(e, cos, "cos", MDATTN_DT_F32, S * (D / 2)));
    TRY(check_vec(e, sin, "sin", MDATTN_DT_F32, S * (D / 2)));
  }
  if (has_bias) {
    TRY(check_vec(e, bias, "bias", MDATTN_DT_BF16, 2 * N));
    TRY(check_vec(e, dbias, "dbias", MDATTN_DT_F32, 2 * N));
  }
  TRY(check_workspace(e, workspace, N * (has_k ? 2 : 1) * (has_bias ? 2 : 1)));
  const mdattn_strides sg{S * N, N, D};
  return e.from(mdattn_norm_rope_fullrow_bwd(
      stream, q->data, has_k ? k->data : nullptr, has_bias ? bias->data : nullptr, gq->data, has_k ? gk->data : nullptr, dq->data,
      has_k ? dk->data : nullptr, wq->data, has_k ? wk->data : nullptr, static_cast<float*>(dwq->data),
      has_k ? static_cast<float*>(dwk->data) : nullptr, has_bias ? static_cast<float*>(dbias->data) : nullptr,
      rope ? static_cast<const float*>(cos->data) : nullptr, rope ? static_cast<const float*>(sin->data) : nullptr, (int)B, (int)S,
      (int)heads, (int)D, eps, q_mul, S * N, N, S * N, N, &sg, static_cast<float*>(workspace->data), count(workspace)));
}

extern "C" int mdattn_xla_norm_rope_perhead_bwd(void* stream, const mdattn_buffer* q, const mdattn_buffer* k, const mdattn_buffer* gq,
                                                const mdattn_buffer* gk, const mdattn_buffer* wq, const mdattn_buffer* wk,
                                                const mdattn_buffer* wq_txt, const mdattn_buffer* wk_txt, const mdattn_buffer* cos,
                                                const mdattn_buffer* sin, const mdattn_buffer* dq, const mdattn_buffer* dk,
                                                const mdattn_buffer* dwq, const mdattn_buffer* dwk, const mdattn_buffer* dwq_txt,
                                                const mdattn_buffer* dwk_txt, const mdattn_buffer* workspace, float eps, float q_mul,
                                                int64_t n_txt, int64_t rope, int64_t has_k, char* err, int err_len) {
  const Err e{err, err_len, "mdattn_norm_rope_perhead_bwd"};
  CHECK_BUF(e, q, "q");
  CHECK_DT(e, q, "q", MDATTN_DT_BF16);
  View4 vq;
  if (!describe(q, 0, &vq)) return e.fail(MDATTN_E_BADARG, "q must be a rank-4 [B,S,H,D] buffer");
  if (n_txt < 0 || n_txt > vq.S) return e.fail(MDATTN_E_BADARG, "n_txt = %lld is outside [0, S = %lld]", (long long)n_txt, (long long)vq.S);
  auto check_side = [&](const mdattn_buffer* x, const mdattn_buffer* g, const mdattn_buffer* w, const mdattn_buffer* wt,
                        const mdattn_buffer* dx, const mdattn_buffer* dw, const mdattn_buffer* dwt, const char* nx, const char* ng,
                        const char* nw, const char* nwt, const char* ndx, const char* ndw, const char* ndwt) -> int {
    View4 t;
    CHECK_BUF(e, x, nx); CHECK_DT(e, x, nx, MDATTN_DT_BF16);
    if (!same_dims(x, q)) return e.fail(MDATTN_E_BADARG, "%s must have q's shape", nx);
    TRY(check_out_bshd(e, g, ng, MDATTN_DT_BF16, vq, &t));
    TRY(check_out_bshd(e, dx, ndx, MDATTN_DT_BF16, vq, &t));
    TRY(check_vec(e, w, nw, MDATTN_DT_BF16, vq.D));
    TRY(check_vec(e, dw, ndw, MDATTN_DT_F32, vq.D));
    if (n_txt > 0) {
      TRY(check_vec(e, wt, nwt, MDATTN_DT_BF16, vq.D));
      TRY(check_vec(e, dwt, ndwt, MDATTN_DT_F32, vq.D));
    }
    return MDATTN_OK;
  };
  TRY(check_side(q, gq, wq, wq_txt, dq, dwq, dwq_txt, "q", "gq", "wq", "wq_txt", "dq", "dwq", "dwq_txt"));
  if (has_k) TRY(check_side(k, gk, wk, wk_txt, dk, dwk, dwk_txt, "k", "gk", "wk", "wk_txt", "dk", "dwk", "dwk_txt"));
  if (rope) {
    TRY(check_vec(e, cos, "cos", MDATTN_DT_F32, vq.S * (vq.D / 2)));
    TRY(check_vec(e, sin, "sin", MDATTN_DT_F32, vq.S * (vq.D / 2)));
  }
  TRY(check_workspace(e, workspace, 4 * vq.D));
  const bool txt = n_txt > 0;
  return e.from(mdattn_norm_rope_perhead_bwd(
      stream, q->data, has_k ? k->data : nullptr, gq->data, has_k ? gk->data : nullptr, dq->data, has_k ? dk->data : nullptr, wq->data,
      has_k ? wk->data : nullptr, txt ? wq_txt->data : nullptr, (txt && has_k) ? wk_txt->data : nullptr, (int)n_txt,
      static_cast<float*>(dwq->data), has_k ? static_cast<float*>(dwk->data) : nullptr, txt ? static_cast<float*>(dwq_txt->data) : nullptr,
      (txt && has_k) ? static_cast<float*>(dwk_txt->data) : nullptr, rope ? static_cast<const float*>(cos->data) : nullptr,
      rope ? static_cast<const float*>(sin->data) : nullptr, (int)vq.B, (int)vq.S, (int)vq.H, (int)vq.D, eps, q_mul, &vq.st, &vq.st, &vq.st,
      static_cast<float*>(workspace->data), count(workspace)));
}

extern "C" int mdattn_xla_norm_rope_rows_bwd(void* stream, const mdattn_buffer* x, const mdattn_buffer* g, const mdattn_buffer* w,
                                             const mdattn_buffer* cos, const mdattn_buffer* sin, const mdattn_buffer* dx,
                                             const mdattn_buffer* dw, const mdattn_buffer* workspace, float eps, int64_t heads,
                                             int64_t mode, char* err, int err_len) {
  const Err e{err, err_len, "mdattn_norm_rope_rows_bwd"};
  CHECK_BUF(e, x, "x");
  if (x->dtype != MDATTN_DT_BF16 && x->dtype != MDATTN_DT_F32) return e.fail(MDATTN_E_BADARG, "x must be bf16 or f32, got %s", dt_name(x->dtype));
  if (x->rank != 3 || heads <= 0 || x->dims[2] % heads) return e.fail(MDATTN_E_BADARG, "x must be [B,S,H*D] with H = heads = %lld", (long long)heads);
  if (mode < 0 || mode > 2) return e.fail(MDATTN_E_BADARG, "mode must be 0 (norm only), 1 (interleaved) or 2 (split), got %lld", (long long)mode);
  const int64_t B = x->dims[0], S = x->dims[1], N = x->dims[2], D = N / heads;
  if (!fits_int(B) || !fits_int(S) || !fits_int(N)) return e.fail(MDATTN_E_UNSUPPORTED, "dimensions beyond 2^31");
  CHECK_BUF(e, g, "g");
  CHECK_DT(e, g, "g", MDATTN_DT_BF16);
  if (g->rank != 4 || g->dims[0] != B || g->dims[1] != S || g->dims[2] != heads || g->dims[3] != D)
    return e.fail(MDATTN_E_BADARG, "g must be [B,S,H,D] = [%lld,%lld,%lld,%lld]", (long long)B, (long long)S, (long long)heads, (long long)D);
  TRY(check_vec(e, w, "w", MDATTN_DT_F32, N));
  CHECK_BUF(e, dx, "dx");
  if (dx->dtype != x->dtype || !same_dims(dx, x)) return e.fail(MDATTN_E_BADARG, "dx must have x's dtype and shape");
  TRY(check_vec(e, dw, "dw", MDATTN_DT_F32, N));
  if (mode) {
    TRY(check_vec(e, cos, "cos", MDATTN_DT_F32, mode == 1 ? B * S * N : B * heads * S * (D / 2)));
    TRY(check_vec(e, sin, "sin", MDATTN_DT_F32, mode == 1 ? B * S * N : B * heads * S * (D / 2)));
  }
  TRY(check_workspace(e, workspace, N));
  const mdattn_strides sg{S * N, N, D};
  return e.from(mdattn_norm_rope_rows_bwd(stream, x->data, x->dtype == MDATTN_DT_F32, g->data, dx->data, static_cast<const float*>(w->data),
                                          static_cast<float*>(dw->data), mode ? static_cast<const float*>(cos->data) : nullptr,
                                          mode ? static_cast<const float*>(sin->data) : nullptr, (int)mode, (int)B, (int)S, (int)heads, (int)D,
                                          eps, S * N, N, S * N, N, &sg, static_cast<float*>(workspace->data), count(workspace)));
}

extern "C" int mdattn_xla_quant_e4m3(void* stream, const mdattn_buffer* x, const mdattn_buffer* x8, const mdattn_buffer* scale_out,
                                     float premul, int64_t pow2_scale, char* err, int err_len) {
  const Err e{err, err_len, "mdattn_quant_e4m3"};
  CHECK_BUF(e, x, "x");
  CHECK_BUF(e, x8, "x8");
  CHECK_DT(e, x, "x", MDATTN_DT_BF16);
  if (!is_fp8(x8)) return e.fail(MDATTN_E_BADARG, "x8 must be a u8 or f8e4m3fn buffer, got %s", dt_name(x8->dtype));
  if (count(x) != count(x8)) return e.fail(MDATTN_E_BADARG, "x and x8 must have the same number of elements");
  TRY(check_vec(e, scale_out, "scale_out", MDATTN_DT_F32, 2));
  return e.from(mdattn_quant_e4m3(stream, x->data, x8->data, static_cast<float*>(scale_out->data), count(x), premul, pow2_scale != 0));
}

extern "C" int mdattn_xla_fwd_fp8(void* stream, const mdattn_buffer* q8, const mdattn_buffer* k8, const mdattn_buffer* v8,
                                  const mdattn_buffer* q_scale, const mdattn_buffer* k_scale, const mdattn_buffer* v_scale,
                                  const mdattn_buffer* out, const mdattn_buffer* lse, float scale, int64_t layout,
                                  int64_t softmax_mode, char* err, int err_len) {
  const Err e{err, err_len, "mdattn_fwd_fp8"};
  View4 vq, vk, vv, vo;
  TRY(check_qkv(e, q8, k8, v8, layout, true, &vq, &vk, &vv));
  TRY(check_out_bshd(e, out, "out", MDATTN_DT_BF16, vq, &vo));
  TRY(check_lse(e, lse, "lse", vq));
  const mdattn_buffer* sc[3] = {q_scale, k_scale, v_scale};
  const char* names[3] = {"q_scale", "k_scale", "v_scale"};
  for (int i = 0; i < 3; ++i) {
    CHECK_BUF(e, sc[i], names[i]);
    CHECK_DT(e, sc[i], names[i], MDATTN_DT_F32);
  }
  if (softmax_mode != MDATTN_FP8_SOFTMAX_EXP2 && softmax_mode != MDATTN_FP8_SOFTMAX_BYTE_GRID)
    return e.fail(MDATTN_E_BADARG, "softmax_mode must be 0 (exp2) or 1 (byte grid), got %lld", (long long)softmax_mode);
  return e.from(mdattn_fwd_fp8(stream, q8->data, k8->data, v8->data, out->data, static_cast<float*>(lse->data), (int)vq.B, (int)vq.H,
                               (int)vq.S, (int)vk.S, (int)vq.D, &vq.st, &vk.st, &vv.st, &vo.st, scale,
                               static_cast<const float*>(q_scale->data), static_cast<const float*>(k_scale->data),
                               static_cast<const float*>(v_scale->data), (int)softmax_mode));
}

extern "C" int mdattn_xla_fwd_fp8_bias(void* stream, const mdattn_buffer* q8, const mdattn_buffer* k8, const mdattn_buffer* v8,
                                       const mdattn_buffer* q_scale, const mdattn_buffer* k_scale, const mdattn_buffer* v_scale,
                                       const mdattn_buffer* key_bias, const mdattn_buffer* out, const mdattn_buffer* lse, float scale,
                                       int64_t layout, char* err, int err_len) {
  const Err e{err, err_len, "mdattn_fwd_fp8_bias"};
  View4 vq, vk, vv, vo;
  TRY(check_qkv(e, q8, k8, v8, layout, true, &vq, &vk, &vv));
  TRY(check_out_bshd(e, out, "out", MDATTN_DT_BF16, vq, &vo));
  TRY(check_lse(e, lse, "lse", vq));
  const mdattn_buffer* sc[3] = {q_scale, k_scale, v_scale};
  const char* names[3] = {"q_scale", "k_scale", "v_scale"};
  for (int i = 0; i < 3; ++i) {
    CHECK_BUF(e, sc[i], names[i]);
    CHECK_DT(e, sc[i], names[i], MDATTN_DT_F32);
  }
  CHECK_BUF(e, key_bias, "key_bias");
  CHECK_DT(e, key_bias, "key_bias", MDATTN_DT_F32);
  const int64_t padded = (vk.S + 31) / 32 * 32;
  if (key_bias->rank != 2 || key_bias->dims[0] != vq.B || key_bias->dims[1] != padded)
    return e.fail(MDATTN_E_BADARG, "key_bias must be [B, Skv rounded up to 32] = [%lld,%lld]", (long long)vq.B, (long long)padded);
  return e.from(mdattn_fwd_fp8_bias(stream, q8->data, k8->data, v8->data, out->data, static_cast<float*>(lse->data), (int)vq.B,
                                    (int)vq.H, (int)vq.S, (int)vk.S, (int)vq.D, &vq.st, &vk.st, &vv.st, &vo.st, scale,
                                    static_cast<const float*>(q_scale->data), static_cast<const float*>(k_scale->data),
                                    static_cast<const float*>(v_scale->data), static_cast<const float*>(key_bias->data), padded));
}

namespace {
// the checks the backward handlers share; q, out, dout, dq are [B,Sq,H,D], k, v, dk, dv [B,Skv,H,D]
int check_bwd(const Err& e, const mdattn_buffer* q, const mdattn_buffer* k, const mdattn_buffer* v, const mdattn_buffer* out,
              const mdattn_buffer* dout, const mdattn_buffer* lse, const mdattn_buffer* dq, const mdattn_buffer* dk,
              const mdattn_buffer* dv, View4* vq, View4* vk) {
  View4 vv, t;
  TRY(check_qkv(e, q, k, v, 0, false, vq, vk, &vv));
  TRY(check_out_bshd(e, out, "out", MDATTN_DT_BF16, *vq, &t));
  TRY(check_out_bshd(e, dout, "dout", MDATTN_DT_BF16, *vq, &t));
  TRY(check_out_bshd(e, dq, "dq", MDATTN_DT_BF16, *vq, &t));
  TRY(check_out_bshd(e, dk, "dk", MDATTN_DT_BF16, *vk, &t));
  TRY(check_out_bshd(e, dv, "dv", MDATTN_DT_BF16, *vk, &t));
  return check_lse(e, lse, "lse", *vq);
}
}  // namespace

extern "C" int mdattn_xla_bwd_bf16(void* stream, const mdattn_buffer* q, const mdattn_buffer* k, const mdattn_buffer* v,
                                   const mdattn_buffer* out, const mdattn_buffer* dout, const mdattn_buffer* lse,
                                   const mdattn_buffer* dq, const mdattn_buffer* dk, const mdattn_buffer* dv,
                                   const mdattn_buffer* workspace, float scale, char* err, int err_len) {
  const Err e{err, err_len, "mdattn_bwd_bf16"};
  View4 vq, vk;
  TRY(check_bwd(e, q, k, v, out, dout, lse, dq, dk, dv, &vq, &vk));
  CHECK_BUF(e, workspace, "workspace");
  CHECK_DT(e, workspace, "workspace", MDATTN_DT_F32);
  const int64_t need = mdattn_bwd_workspace_floats((int)vq.B, (int)vq.H, (int)vq.S);
  if (count(workspace) < need) return e.fail(MDATTN_E_BADARG, "workspace must hold at least %lld floats, got %lld", (long long)need, (long long)count(workspace));
  return e.from(mdattn_bwd_bf16(stream, q->data, k->data, v->data, out->data, dout->data, static_cast<const float*>(lse->data), dq->data,
                                dk->data, dv->data, static_cast<float*>(workspace->data), count(workspace), (int)vq.B, (int)vq.H,
                                (int)vq.S, (int)vk.S, (int)vq.D, &vq.st, &vk.st, &vk.st, &vq.st, scale));
}

extern "C" int mdattn_xla_bwd_bf16_bias(void* stream, const mdattn_buffer* q, const mdattn_buffer* k, const mdattn_buffer* v,
                                        const mdattn_buffer* out, const mdattn_buffer* dout, const mdattn_buffer* lse,
                                        const mdattn_buffer* key_bias, const mdattn_buffer* dq, const mdattn_buffer* dk,
                                        const mdattn_buffer* dv, const mdattn_buffer* workspace, float scale, char* err,
                                        int err_len) {
  const Err e{err, err_len, "mdattn_bwd_bf16_bias"};
  View4 vq, vk;
  TRY(check_bwd(e, q, k, v, out, dout, lse, dq, dk, dv, &vq, &vk));
  CHECK_BUF(e, workspace, "workspace");
  CHECK_DT(e, workspace, "workspace", MDATTN_DT_F32);
  const int64_t need = mdattn_bwd_workspace_floats((int)vq.B, (int)vq.H, (int)vq.S);
  if (count(workspace) < need) return e.fail(MDATTN_E_BADARG, "workspace must hold at least %lld floats, got %lld", (long long)need, (long long)count(workspace));
  CHECK_BUF(e, key_bias, "key_bias");
  CHECK_DT(e, key_bias, "key_bias", MDATTN_DT_F32);
  const int64_t padded = (vk.S + 31) / 32 * 32;
  if (key_bias->rank != 2 || key_bias->dims[0] != vq.B || key_bias->dims[1] != padded)
    return e.fail(MDATTN_E_BADARG, "key_bias must be [B, Skv rounded up to 32] = [%lld,%lld]", (long long)vq.B, (long long)padded);
  return e.from(mdattn_bwd_bf16_bias(stream, q->data, k->data, v->data, out->data, dout->data, static_cast<const float*>(lse->data),
                                     dq->data, dk->data, dv->data, static_cast<float*>(workspace->data), count(workspace), (int)vq.B,
                                     (int)vq.H, (int)vq.S, (int)vk.S, (int)vq.D, &vq.st, &vk.st, &vk.st, &vq.st, scale,
                                     static_cast<const float*>(key_bias->data), padded));
}

extern "C" int mdattn_xla_bwd_bf16_static(void* stream, const mdattn_buffer* q, const mdattn_buffer* k, const mdattn_buffer* v,
                                          const mdattn_buffer* out, const mdattn_buffer* dout, const mdattn_buffer* lse,
                                          const mdattn_buffer* dq, const mdattn_buffer* dk, const mdattn_buffer* dv, float scale,
                                          char* err, int err_len) {
  const Err e{err, err_len, "mdattn_bwd_bf16_static"};
  View4 vq, vk;
  TRY(check_bwd(e, q, k, v, out, dout, lse, dq, dk, dv, &vq, &vk));
  return e.from(mdattn_bwd_bf16_static(stream, q->data, k->data, v->data, out->data, dout->data, static_cast<const float*>(lse->data),
                                       dq->data, dk->data, dv->data, (int)vq.B, (int)vq.H, (int)vq.S, (int)vk.S, (int)vq.D, &vq.st,
                                       &vk.st, &vk.st, &vq.st, scale));
}
