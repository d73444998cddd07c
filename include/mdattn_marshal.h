/*
 * mdattn_marshal.h -- the bodies of the XLA custom-call handlers, without any XLA type.
 *
 * maxdiffusion reaches a kernel through `register_kernel` / KERNEL_REGISTRY (models/attention_flax.py:1589-1597,
 * lookup :1965-1966); under JAX the registered Python function issues an XLA custom call (jax.ffi.ffi_call), and XLA
 * calls a handler with its buffers.  A handler has to turn those buffers (pointer, element type, dimensions) into the
 * pointers, sizes and strides of mdattn.h, and to refuse what does not fit BEFORE anything is launched.  That work is
 * here, on plain structs, compiled into libmdattn.so and testable without jaxlib; csrc/ffi/mdattn_ffi.cc, the only
 * file that includes xla/ffi/api/ffi.h, holds nothing but the conversion of ffi::AnyBuffer to mdattn_buffer and the
 * XLA_FFI_DEFINE_HANDLER_SYMBOL bind lines.
 *
 * Every function: returns MDATTN_OK or a negative MDATTN_E_* code; on failure writes a message that names the
 * offending argument into `err` (nullable, `err_len` bytes, always terminated); enqueues on `stream`, never
 * synchronises, never allocates.  Inputs come first, then results, then attributes, in the order of the bind lines.
 * `layout` 0: q, k, v are [B,S,H,D] (= the reference's rank-3 [B,S,H*D] reshaped, free); 1: [B,H,S,D] (what
 * FlaxWanAttention hands over after _unflatten_heads, attention_flax.py:2673-2675).  Attention results are always
 * [B,Sq,H,D], which reshapes for free to the [B,Sq,H*D] the registry contract returns (:146-152).
 */
#ifndef MDATTN_MARSHAL_H_
#define MDATTN_MARSHAL_H_

#include <stdint.h>

#include "mdattn.h"

#ifdef __cplusplus
extern "C" {
#endif

enum {
  MDATTN_DT_OTHER = 0,
  MDATTN_DT_BF16 = 1,
  MDATTN_DT_F32 = 2,
  MDATTN_DT_U8 = 3,      /* uint8, int8 and PRED (bool) buffers: one byte per element */
  MDATTN_DT_F8E4M3FN = 4 /* OCP float8 e4m3fn */
};

/* One XLA buffer: device pointer, element type (MDATTN_DT_*), rank and dimensions (dense, row-major). */
typedef struct mdattn_buffer {
  void* data;
  int32_t dtype;
  int32_t rank;
  const int64_t* dims;
} mdattn_buffer;

/* custom call "mdattn_fwd_bf16": (q, k, v) -> (out bf16 [B,Sq,H,D], lse f32 [B,H,Sq]) */
int mdattn_xla_fwd_bf16(void* stream, const mdattn_buffer* q, const mdattn_buffer* k, const mdattn_buffer* v,
                        const mdattn_buffer* out, const mdattn_buffer* lse, float scale, int64_t layout,
                        char* err, int err_len);

/* "mdattn_fwd_bf16_bias": (q, k, v, key_bias f32 [B, Skv rounded up to 32]) -> (out, lse) */
int mdattn_xla_fwd_bf16_bias(void* stream, const mdattn_buffer* q, const mdattn_buffer* k, const mdattn_buffer* v,
                             const mdattn_buffer* key_bias, const mdattn_buffer* out, const mdattn_buffer* lse,
                             float scale, int64_t layout, char* err, int err_len);

/* "mdattn_key_mask_bias": (keep bool/u8 [B,Skv]) -> (bias f32 [B, Skv rounded up to 32]) */
int mdattn_xla_key_mask_bias(void* stream, const mdattn_buffer* keep, const mdattn_buffer* bias, float masked_value,
                             char* err, int err_len);

/* "mdattn_fwd_bf16_merge": (q, k, v, o_run f32 [B,Sq,H,D], lse_run f32 [B,H,Sq]) -> (o_run, lse_run), the results
 * aliased to the inputs (input_output_aliases={3: 0, 4: 1}): the carry is updated in place. */
int mdattn_xla_fwd_bf16_merge(void* stream, const mdattn_buffer* q, const mdattn_buffer* k, const mdattn_buffer* v,
                              const mdattn_buffer* o_run_in, const mdattn_buffer* lse_run_in,
                              const mdattn_buffer* o_run, const mdattn_buffer* lse_run, float scale, int64_t layout,
                              char* err, int err_len);

/* "mdattn_merge": (o_run f32, lse_run f32, o_cur bf16|f32 [B,S,H,D], lse_cur f32 [B,H,S]) -> (o_run, lse_run),
 * aliased (input_output_aliases={0: 0, 1: 1}) */
int mdattn_xla_merge(void* stream, const mdattn_buffer* o_run_in, const mdattn_buffer* lse_run_in,
                     const mdattn_buffer* o_cur, const mdattn_buffer* lse_cur, const mdattn_buffer* o_run,
                     const mdattn_buffer* lse_run, char* err, int err_len);

/* "mdattn_finalize": (o_run f32, any shape) -> (out bf16, same shape): the cast of a merged carry
 * (ring_attention_kernel.py:1130) */
int mdattn_xla_finalize(void* stream, const mdattn_buffer* o_run, const mdattn_buffer* out, char* err, int err_len);

/* "mdattn_norm_rope_fullrow": (q, k bf16 [B,S,H*D], wq, wk bf16 [H*D], cos, sin f32 [S,D/2]) -> (q_out, k_out bf16
 * [B,S,H,D]).  rope == 0: cos / sin are ignored (any shape); has_k == 0: k, wk and k_out are ignored (the cached
 * text K/V case, attention_flax.py:2659-2660; XLA cannot pass an absent buffer, the caller passes any small one). */
int mdattn_xla_norm_rope_fullrow(void* stream, const mdattn_buffer* q, const mdattn_buffer* k, const mdattn_buffer* wq,
                                 const mdattn_buffer* wk, const mdattn_buffer* cos, const mdattn_buffer* sin,
                                 const mdattn_buffer* q_out, const mdattn_buffer* k_out, float eps, float q_mul,
                                 int64_t heads, int64_t rope, int64_t has_k, char* err, int err_len);

/* "mdattn_norm_rope_qkv": (qkv bf16 [B,S,3*H*D], bias bf16 [3*H*D], wq, wk bf16 [H*D], cos, sin f32 [S,D/2]) -> (q_out,
 * k_out, v_out bf16 [B,S,H,D]).  has_bias == 0: bias is ignored; has_v == 0 (only without bias): v_out is ignored and v
 * stays in the fused buffer (the caller slices it).  XLA cannot alias a result to a slice of an operand, so the
 * custom call always writes dense results; the in-place form is for callers of the C ABI. */
int mdattn_xla_norm_rope_qkv(void* stream, const mdattn_buffer* qkv, const mdattn_buffer* bias, const mdattn_buffer* wq,
                             const mdattn_buffer* wk, const mdattn_buffer* cos, const mdattn_buffer* sin,
                             const mdattn_buffer* q_out, const mdattn_buffer* k_out, const mdattn_buffer* v_out, float eps,
                             float q_mul, int64_t heads, int64_t rope, int64_t has_bias, int64_t has_v, char* err, int err_len);

/* "mdattn_norm_rope_perhead": (q, k bf16 [B,S,H,D], wq, wk, wq_txt, wk_txt bf16 [D], cos, sin f32 [S,D/2]) ->
 * (q_out, k_out bf16 [B,S,H,D]).  Tokens [0, n_txt) take the text weights (FlaxFluxAttention's encoder_*_norm,
 * attention_flax.py:3002-3003); n_txt == 0: wq_txt / wk_txt are ignored. */
int mdattn_xla_norm_rope_perhead(void* stream, const mdattn_buffer* q, const mdattn_buffer* k, const mdattn_buffer* wq,
                                 const mdattn_buffer* wk, const mdattn_buffer* wq_txt, const mdattn_buffer* wk_txt,
                                 const mdattn_buffer* cos, const mdattn_buffer* sin, const mdattn_buffer* q_out,
                                 const mdattn_buffer* k_out, float eps, float q_mul, int64_t n_txt, int64_t rope,
                                 int64_t has_k, char* err, int err_len);

/* "mdattn_norm_rope_rows": (x bf16|f32 [B,S,H*D], w f32 [H*D], cos, sin f32) -> (x_out bf16 [B,S,H,D]); mode 0:
 * norm only, 1: interleaved (cos/sin [B,S,H*D]), 2: split (cos/sin [B,H,S,D/2]) */
int mdattn_xla_norm_rope_rows(void* stream, const mdattn_buffer* x, const mdattn_buffer* w, const mdattn_buffer* cos,
                              const mdattn_buffer* sin, const mdattn_buffer* x_out, float eps, int64_t heads,
                              int64_t mode, char* err, int err_len);

/* "mdattn_norm_rope_fullrow_bwd": (q, k bf16 [B,S,H*D], gq, gk bf16 [B,S,H,D], wq, wk bf16 [H*D], cos, sin f32 [S,D/2],
 * bias bf16 [2*H*D]) -> (dq, dk bf16 [B,S,H*D], dwq, dwk f32 [H*D], dbias f32 [2*H*D], workspace f32 [>= columns]).
 * rope == 0: cos / sin ignored; has_k == 0: k, gk, wk, dk, dwk ignored; has_bias == 0: bias and dbias ignored.  XLA
 * allocates the scratch of the two-stage weight-gradient reduction as the last result
 * (mdattn_norm_rope_bwd_workspace_floats(B*S, columns) floats; columns = H*D x (2 with k) x (2 with bias)). */
int mdattn_xla_norm_rope_fullrow_bwd(void* stream, const mdattn_buffer* q, const mdattn_buffer* k, const mdattn_buffer* gq,
                                     const mdattn_buffer* gk, const mdattn_buffer* wq, const mdattn_buffer* wk,
                                     const mdattn_buffer* cos, const mdattn_buffer* sin, const mdattn_buffer* bias,
                                     const mdattn_buffer* dq, const mdattn_buffer* dk, const mdattn_buffer* dwq,
                                     const mdattn_buffer* dwk, const mdattn_buffer* dbias, const mdattn_buffer* workspace,
                                     float eps, float q_mul, int64_t heads, int64_t rope, int64_t has_k, int64_t has_bias,
                                     char* err, int err_len);

/* "mdattn_norm_rope_perhead_bwd": (q, k, gq, gk bf16 [B,S,H,D], wq, wk, wq_txt, wk_txt bf16 [D], cos, sin f32 [S,D/2]) ->
 * (dq, dk bf16 [B,S,H,D], dwq, dwk, dwq_txt, dwk_txt f32 [D], workspace f32 [>= 4*D]).  n_txt == 0: the text weights and
 * their gradients are ignored; has_k == 0: everything of k is ignored. */
int mdattn_xla_norm_rope_perhead_bwd(void* stream, const mdattn_buffer* q, const mdattn_buffer* k, const mdattn_buffer* gq,
                                     const mdattn_buffer* gk, const mdattn_buffer* wq, const mdattn_buffer* wk,
                                     const mdattn_buffer* wq_txt, const mdattn_buffer* wk_txt, const mdattn_buffer* cos,
                                     const mdattn_buffer* sin, const mdattn_buffer* dq, const mdattn_buffer* dk,
                                     const mdattn_buffer* dwq, const mdattn_buffer* dwk, const mdattn_buffer* dwq_txt,
                                     const mdattn_buffer* dwk_txt, const mdattn_buffer* workspace, float eps, float q_mul,
                                     int64_t n_txt, int64_t rope, int64_t has_k, char* err, int err_len);

/* "mdattn_norm_rope_rows_bwd": (x bf16|f32 [B,S,H*D], g bf16 [B,S,H,D], w f32 [H*D], cos, sin f32) -> (dx in x's dtype
 * [B,S,H*D], dw f32 [H*D], workspace f32 [>= H*D]); mode as for mdattn_norm_rope_rows */
int mdattn_xla_norm_rope_rows_bwd(void* stream, const mdattn_buffer* x, const mdattn_buffer* g, const mdattn_buffer* w,
                                  const mdattn_buffer* cos, const mdattn_buffer* sin, const mdattn_buffer* dx,
                                  const mdattn_buffer* dw, const mdattn_buffer* workspace, float eps, int64_t heads,
                                  int64_t mode, char* err, int err_len);

/* "mdattn_quant_e4m3": (x bf16, any shape) -> (x8 u8|f8e4m3fn same shape, scale f32 [2]) */
int mdattn_xla_quant_e4m3(void* stream, const mdattn_buffer* x, const mdattn_buffer* x8, const mdattn_buffer* scale_out,
                          float premul, int64_t pow2_scale, char* err, int err_len);

/* "mdattn_fwd_fp8": (q8, k8, v8 u8|f8e4m3fn, q_scale, k_scale, v_scale f32 [>=1]) -> (out bf16 [B,Sq,H,D], lse) */
int mdattn_xla_fwd_fp8(void* stream, const mdattn_buffer* q8, const mdattn_buffer* k8, const mdattn_buffer* v8,
                       const mdattn_buffer* q_scale, const mdattn_buffer* k_scale, const mdattn_buffer* v_scale,
                       const mdattn_buffer* out, const mdattn_buffer* lse, float scale, int64_t layout,
                       int64_t softmax_mode, char* err, int err_len);

/* "mdattn_fwd_fp8_bias": (q8, k8, v8, q_scale, k_scale, v_scale, key_bias f32 [B, Skv rounded up to 32]) -> (out, lse) */
int mdattn_xla_fwd_fp8_bias(void* stream, const mdattn_buffer* q8, const mdattn_buffer* k8, const mdattn_buffer* v8,
                            const mdattn_buffer* q_scale, const mdattn_buffer* k_scale, const mdattn_buffer* v_scale,
                            const mdattn_buffer* key_bias, const mdattn_buffer* out, const mdattn_buffer* lse, float scale,
                            int64_t layout, char* err, int err_len);

/* "mdattn_bwd_bf16": (q, k, v, out, dout bf16 [B,S,H,D], lse f32 [B,H,Sq]) -> (dq, dk, dv bf16, workspace f32
 * [mdattn_bwd_workspace_floats(B,H,Sq)]): XLA allocates the workspace as a fourth result */
int mdattn_xla_bwd_bf16(void* stream, const mdattn_buffer* q, const mdattn_buffer* k, const mdattn_buffer* v,
                        const mdattn_buffer* out, const mdattn_buffer* dout, const mdattn_buffer* lse,
                        const mdattn_buffer* dq, const mdattn_buffer* dk, const mdattn_buffer* dv,
                        const mdattn_buffer* workspace, float scale, char* err, int err_len);

/* "mdattn_bwd_bf16_bias": (q, k, v, out, dout, lse, key_bias f32 [B, Skv rounded up to 32]) -> (dq, dk, dv, workspace) */
int mdattn_xla_bwd_bf16_bias(void* stream, const mdattn_buffer* q, const mdattn_buffer* k, const mdattn_buffer* v,
                             const mdattn_buffer* out, const mdattn_buffer* dout, const mdattn_buffer* lse,
                             const mdattn_buffer* key_bias, const mdattn_buffer* dq, const mdattn_buffer* dk,
                             const mdattn_buffer* dv, const mdattn_buffer* workspace, float scale, char* err, int err_len);

/* "mdattn_bwd_bf16_static": the same without the workspace result (mdattn_bwd_bf16_static's static scratch) */
int mdattn_xla_bwd_bf16_static(void* stream, const mdattn_buffer* q, const mdattn_buffer* k, const mdattn_buffer* v,
                               const mdattn_buffer* out, const mdattn_buffer* dout, const mdattn_buffer* lse,
                               const mdattn_buffer* dq, const mdattn_buffer* dk, const mdattn_buffer* dv, float scale,
                               char* err, int err_len);

#ifdef __cplusplus
}
#endif
#endif /* MDATTN_MARSHAL_H_ */
