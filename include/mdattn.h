/*
 * mdattn.h -- C ABI of the MI355X (gfx950) DiT attention hot path.
 *
 * One shared library (libmdattn.so).  Every entry point
 *   - takes a HIP stream (hipStream_t passed as void*; NULL = the default stream),
 *   - only enqueues work on that stream: never synchronises, never allocates,
 *   - validates its arguments on the host BEFORE any launch and returns a negative
 *     MDATTN_E_* code instead of launching a kernel that could fault,
 *   - is re-entrant: no mutable global state, with two documented exceptions -- the test hook
 *     mdattn_set_fwd_schedule (a process-wide switch read once per forward call) and the static scratch of
 *     mdattn_bwd_bf16_static (shared by all calls on one GPU).  Once-initialised read-only caches (a kernel's LDS
 *     opt-in, the resident-workgroup count of a persistent kernel, the scratch address) are filled under atomics.
 *   - reads and clears a HIP error left pending on the calling thread before each launch, so that MDATTN_E_LAUNCH
 *     always means one of its own launches was rejected.
 * All pointers are device pointers owned by the caller.  "bf16" tensors hold
 * bfloat16 bit patterns (uint16_t); the innermost (head_dim) axis is contiguous and
 * every other axis is described by an element stride, so [B,S,H,D] (= the
 * reference's rank-3 [B,S,H*D]) and [B,H,S,D] are both accepted without a copy.
 *
 * The reference these replace is Python (paths relative to src/maxdiffusion/ of
 * AI-Hypercomputer/maxdiffusion); each declaration cites the code it stands in for.
 */
#ifndef MDATTN_H_
#define MDATTN_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MDATTN_VERSION 100 /* major*10000 + minor*100 + patch */

enum {
  MDATTN_OK = 0,
  MDATTN_E_BADARG = -1,      /* null pointer, non-positive size, inconsistent shape   */
  MDATTN_E_UNSUPPORTED = -2, /* well-formed request this build has no kernel for      */
  MDATTN_E_ALIGN = -3,       /* pointer or stride not aligned as the kernels require  */
  MDATTN_E_LAUNCH = -4,      /* the HIP runtime rejected the launch                   */
  MDATTN_E_TOOBIG = -5       /* larger than the static scratch of a no-allocation entry point */
};

/* Element strides of one rank-4 tensor [batch, seq, head, dim] with dim contiguous. */
typedef struct mdattn_strides {
  int64_t batch;
  int64_t seq;
  int64_t head;
} mdattn_strides;

int mdattn_version(void);
const char* mdattn_strerror(int code);
/* Hash of the sources and compiler flags the library was built from (the build script passes it in): lets the
 * host side refuse a library that was not built from the sources next to it. */
const char* mdattn_build_id(void);

/*
 * Test and tuning hook, no counterpart in the reference: forces the schedule that mdattn_fwd_bf16 and
 * mdattn_fwd_bf16_merge use at head dim 128, for the whole process, until set again.  0 restores the choice by shape.
 * Returns the previous value (>= 0) or MDATTN_E_BADARG.  The parity tests use it to run every schedule on every shape;
 * nothing else should: it is the one piece of mutable state in the library, read once per call.
 */
#define MDATTN_FWD_SCHEDULE_AUTO 0
#define MDATTN_FWD_SCHEDULE_PIPELINED8 1 /* 8 waves x 32 rows, software-pipelined, 64-key tiles */
#define MDATTN_FWD_SCHEDULE_PIPELINED4 2 /* 4 waves x 32 rows, same loop                        */
#define MDATTN_FWD_SCHEDULE_FLAT 3       /* 4 waves x 32 rows, 32-key tiles, 3 workgroups per CU */
#define MDATTN_FWD_SCHEDULE_LAST 3
int mdattn_set_fwd_schedule(int schedule);

/*
 * Fused RMSNorm over the FULL inner dimension H*D + 3-axis RoPE, for q and k in one pass.
 * Replaces: FlaxWanAttention.__call__'s norm_q / norm_k (models/attention_flax.py:2657,
 * :2669; module definition :2529-2553), _unflatten_heads (:2673-2675) and _apply_rope
 * (:2596-2620, called :2677).
 *   q_in, k_in   bf16 [B,S,H*D]; k_in may be NULL (only q is processed: the cached-text-KV
 *                case, attention_flax.py:2659-2660)
 *   q_out,k_out  bf16, strides out_strides (any of [B,S,H,D] / [B,H,S,D]); may alias the inputs
 *                when the layouts are identical
 *   wq, wk       bf16 [H*D] RMSNorm scales
 *   cos, sin     f32 [S, D/2]: real/imaginary part of the rotary table the unchanged host
 *                code builds (WanRotaryPosEmbed, models/wan/transformers/transformer_wan.py:63-95);
 *                both NULL = norm only (cross-attention, rotary_emb is None, attention_flax.py:2671)
 *   q_mul        constant multiplied into q_out before its rounding (1.0f = none).  With
 *                q_mul = scale * log2(e) and scale = ln 2 handed to the attention entry points the
 *                softmax scale costs no rounding and no instruction: the reference multiplies k by
 *                scale and q by log2(e) in bf16 before its kernels (attention_flax.py:1783, :610, :890).
 * Arithmetic: statistics, scale and rotation in f32, ONE rounding to bf16.
 * Requires D % 8 == 0, H*D <= 8192, 16-byte aligned pointers, strides % 8 == 0.
 */
int mdattn_norm_rope_fullrow(void* stream, const void* q_in, const void* k_in, void* q_out, void* k_out,
                             const void* wq, const void* wk, const float* cos, const float* sin,
                             int B, int S, int H, int D, float eps, float q_mul,
                             int64_t in_stride_batch, int64_t in_stride_seq,
                             const mdattn_strides* out_strides);

/*
 * The same prologue over the output of ONE fused q|k|v projection, with the projections' bias adds folded in: one
 * launch reads the GEMM output once and leaves q, k (and v) ready for the attention entry points.
 * Replaces: the bias adds of FlaxWanAttention's query / key / value Linear layers (models/attention_flax.py:2471-2510,
 * called :2653-2663), norm_q / norm_k (:2657, :2669), _unflatten_heads of q, k and v (:2673-2675) and _apply_rope
 * (:2677).  (The reference runs three GEMMs; fusing them into one [hidden, 3*H*D] GEMM is the maintainer's choice:
 * this entry point only asks that the three outputs sit side by side in one row.)
 *   qkv          bf16 [B,S,3*H*D]: column blocks q | k | v of each token row; row stride qkv_stride_seq >= 3*H*D
 *   bias         bf16 [3*H*D] (q | k | v) or NULL.  Given: the GEMM ran without its bias epilogue, and the biases
 *                are added here in f32 before the statistics (one rounding fewer than the reference's bf16 Linear
 *                output).  NULL: qkv already holds the biased projections.
 *   q_out,k_out  bf16 by out_strides ([B,S,H,D] or [B,H,S,D]); v_out likewise, or NULL
 *   v_out        NULL (only without bias): v is not touched; the attention entry points read it in place from the
 *                fused buffer (pointer qkv + 2*H*D, strides {qkv_stride_batch, qkv_stride_seq, D}).
 *   In place: with out_strides = {qkv_stride_batch, qkv_stride_seq, D}, q_out = qkv, k_out = qkv + H*D (and
 *   v_out = qkv + 2*H*D) the fused buffer itself becomes the attention operands; outputs may alias the input only
 *   like this, element for element.
 *   wq, wk, cos, sin, eps, q_mul and the arithmetic as for mdattn_norm_rope_fullrow.
 */
int mdattn_norm_rope_qkv(void* stream, const void* qkv, const void* bias, void* q_out, void* k_out, void* v_out,
                         const void* wq, const void* wk, const float* cos, const float* sin,
                         int B, int S, int H, int D, float eps, float q_mul,
                         int64_t qkv_stride_batch, int64_t qkv_stride_seq, const mdattn_strides* out_strides);

/*
 * Fused per-head RMSNorm (over D) + 3-axis RoPE, for q and k in one pass.
 * Replaces: FlaxFluxAttention's query_norm / key_norm / encoder_*_norm
 * (models/attention_flax.py:2947-2967, applied :2989-2990 and :3002-3003; single blocks
 * models/flux/transformers/transformer_flux_flax.py:192-193) and apply_rope
 * (models/attention_flax.py:2079-2115, called :3018).
 *   q_in, k_in   bf16 [B,S,H,D] described by in_strides (k_in may be NULL)
 *   wq, wk       bf16 [D]; wq_txt / wk_txt (nullable) are used for tokens [0, n_txt)
 *   cos, sin     f32 [S, D/2] from FluxPosEmbed (models/embeddings_flax.py:437-469); NULL = norm only
 *   q_mul        as for mdattn_norm_rope_fullrow
 * Requires D in {64,128,256}.
 */
int mdattn_norm_rope_perhead(void* stream, const void* q_in, const void* k_in, void* q_out, void* k_out,
                             const void* wq, const void* wk, const void* wq_txt, const void* wk_txt, int n_txt,
                             const float* cos, const float* sin, int B, int S, int H, int D, float eps, float q_mul,
                             const mdattn_strides* in_strides, const mdattn_strides* out_strides);

/*
 * Full-row RMSNorm + rotary embedding of ONE tensor with position tables that differ per batch element and per
 * head.  Replaces, for q and for k separately: `norm_q` / `norm_k` (f32 statistics and f32 weight) followed by
 * `apply_rotary_emb` or `apply_split_rotary_emb` in LTX2Attention.__call__ (models/ltx2/attention_ltx2.py:556-585,
 * :33-60, :62-102); tables as LTX2RotaryPosEmbed returns them (:292-324).
 *   x_in         [B,S,H*D] bf16 (x_is_f32 = 0) or f32 (1), strides in elements
 *   x_out        bf16 [B,S,H,D] by out_strides
 *   w            f32 [H*D]
 *   rope_mode    0: norm only (cross-attention keys);  1: interleaved, cos/sin f32 [B,S,H*D];
 *                2: split, cos/sin f32 [B,H,S,D/2]
 * Requires D % 16 == 0 and H*D <= 8192.
 */
int mdattn_norm_rope_rows(void* stream, const void* x_in, int x_is_f32, void* x_out, const float* w,
                          const float* cos, const float* sin, int rope_mode, int B, int S, int H, int D, float eps,
                          int64_t in_stride_batch, int64_t in_stride_seq, const mdattn_strides* out_strides);

/*
 * Backward of the fused prologues: input gradients and weight gradients from the saved inputs and the upstream
 * gradients of the prologue's outputs (what the attention backward returns as dq, dk).  Replaces: JAX autodiff through
 * norm_q / norm_k and _apply_rope (models/attention_flax.py:2655-2677, :2596-2620; Flux :2989-3020; LTX-2
 * models/ltx2/attention_ltx2.py:556-585) -- the reference has no hand-written backward here, the trainer
 * differentiates straight through these lines (trainers/wan_trainer.py:169).
 *   forward  u = x (+ bias);  r = rsqrt(mean(u^2) + eps);  y = u r w;  out = q_mul * R(y)
 *   backward dy = q_mul * R^T g;  du = r (w dy) - u r^3 mean(u w dy);  dw = sum over tokens of dy u r
 * The row statistics are recomputed from the saved input; statistics, rotation and VJP in f32, ONE rounding of du to
 * the input's dtype; dw in f32.  dw is reduced over tokens without atomics in two stages through `workspace` (every
 * workgroup writes one partial row, a second kernel adds the rows in a fixed order: bit-reproducible).
 *   workspace    f32 device scratch, 16-byte aligned; mdattn_norm_rope_bwd_workspace_floats(rows, columns) floats
 *                give the kernels their full grid (1024 partial rows); a smaller one (>= columns floats) is accepted
 *                and lowers the number of workgroups.  rows / columns: B*S and 2*H*D (one tensor: H*D; with bias
 *                twice that) for the full-row form; B*S*H and 4*D for the per-head form; B*S and H*D for the rows form.
 */
int64_t mdattn_norm_rope_bwd_workspace_floats(int64_t rows, int64_t columns);

/*
 * Backward of mdattn_norm_rope_fullrow and, with `bias`, of mdattn_norm_rope_qkv's q and k blocks (its v block is a
 * copy: dv is the attention backward's dv, summed over tokens for the v bias by the caller).
 *   q_in, k_in   the saved inputs, bf16 rows of H*D by (in_stride_batch, in_stride_seq); k_in may be NULL, and then
 *                gk, dk_in, wk, dwk are NULL too
 *   bias         bf16 [2*H*D] (q | k blocks of the projection biases the forward added) or NULL; needs k_in
 *   gq, gk       bf16 [B,S,H,D] by g_strides: gradients of q_out, k_out
 *   dq_in, dk_in bf16 rows of H*D by (dx_stride_batch, dx_stride_seq): gradients of the inputs (with dx strides of
 *                3*H*D and dk_in = dq_in + H*D they are the q | k blocks of a fused gradient buffer)
 *   dwq, dwk     f32 [H*D];  dbias f32 [2*H*D] (with bias; = column sums of dq_in | dk_in) or NULL
 *   wq, wk, cos, sin, eps, q_mul as given to the forward.  Requires D % 8 == 0, H*D <= 8192.
 */
int mdattn_norm_rope_fullrow_bwd(void* stream, const void* q_in, const void* k_in, const void* bias,
                                 const void* gq, const void* gk, void* dq_in, void* dk_in,
                                 const void* wq, const void* wk, float* dwq, float* dwk, float* dbias,
                                 const float* cos, const float* sin, int B, int S, int H, int D, float eps, float q_mul,
                                 int64_t in_stride_batch, int64_t in_stride_seq,
                                 int64_t dx_stride_batch, int64_t dx_stride_seq, const mdattn_strides* g_strides,
                                 float* workspace, int64_t workspace_floats);

/*
 * Backward of mdattn_norm_rope_perhead.  q_in, k_in bf16 [B,S,H,D] by in_strides (k_in may be NULL with gk, dk_in,
 * wk, dwk); gq, gk by g_strides; dq_in, dk_in by dx_strides; dwq, dwk f32 [D]: weight gradients over the tokens that
 * used wq / wk; dwq_txt, dwk_txt f32 [D] (given exactly when wq_txt / wk_txt are): over the tokens [0, n_txt).
 */
int mdattn_norm_rope_perhead_bwd(void* stream, const void* q_in, const void* k_in, const void* gq, const void* gk,
                                 void* dq_in, void* dk_in, const void* wq, const void* wk, const void* wq_txt,
                                 const void* wk_txt, int n_txt, float* dwq, float* dwk, float* dwq_txt, float* dwk_txt,
                                 const float* cos, const float* sin, int B, int S, int H, int D, float eps, float q_mul,
                                 const mdattn_strides* in_strides, const mdattn_strides* dx_strides,
                                 const mdattn_strides* g_strides, float* workspace, int64_t workspace_floats);

/*
 * Backward of mdattn_norm_rope_rows (LTX-2): x_in [B,S,H*D] bf16 or f32 as given to the forward, g bf16 [B,S,H,D] by
 * g_strides, dx in x_in's dtype by (dx_stride_batch, dx_stride_seq), dw f32 [H*D]; tables and rope_mode as for the
 * forward (the two members of a pair may carry different table values: the transposed rotation is applied as written,
 * not as the rotation by the opposite angle).
 */
int mdattn_norm_rope_rows_bwd(void* stream, const void* x_in, int x_is_f32, const void* g, void* dx, const float* w,
                              float* dw, const float* cos, const float* sin, int rope_mode, int B, int S, int H, int D,
                              float eps, int64_t in_stride_batch, int64_t in_stride_seq,
                              int64_t dx_stride_batch, int64_t dx_stride_seq, const mdattn_strides* g_strides,
                              float* workspace, int64_t workspace_floats);

/*
 * Non-causal softmax attention forward, bf16 MFMA, online softmax in f32, optional LSE.
 * Replaces: the kernel a KERNEL_REGISTRY entry dispatches to (models/attention_flax.py:1589-1597,
 * :1965-1966), i.e. what _tpu_flash_attention (:563-809) / kernels/custom_splash_attention.py:69-320
 * compute, with results matching `_apply_attention_dot` (:1487-1567).
 *   q            bf16 [B,Sq,H,D] by q_strides;  k, v  bf16 [B,Skv,H,D] by k_/v_strides
 *   out          bf16 [B,Sq,H,D] by o_strides
 *   lse          f32 [B,H,Sq] contiguous or NULL: natural-log logsumexp of scale*q.k
 *                (kernels/splash_attention/base.py:103-105)
 *   scale        applied to q.k inside the kernel (the reference pre-multiplies k, :1783).  scale = ln 2, i.e.
 *                scale * log2(e) == 1, says that q already carries the softmax scale times log2(e)
 *                (mdattn_norm_rope_*'s q_mul): the kernels then form exp2 of the raw products and save the
 *                multiply per logit; the result is that of the softmax scale on the plain q.
 * Requires D == 128, or D == 64 (LTX-2's audio stream, models/ltx2/transformer_ltx2.py:788-789).  Any Sq, Skv >= 1
 * (ragged tails handled in-kernel).
 */
int mdattn_fwd_bf16(void* stream, const void* q, const void* k, const void* v, void* out, float* lse,
                    int B, int H, int Sq, int Skv, int D,
                    const mdattn_strides* q_strides, const mdattn_strides* k_strides,
                    const mdattn_strides* v_strides, const mdattn_strides* o_strides, float scale);

/*
 * The same forward with an additive per-key bias: logits = scale*q.k + key_bias[b, key] (natural-log units;
 * -inf excludes a key).  Replaces: the key padding mask of `_apply_attention` (models/attention_flax.py:1926-1939:
 * a [B,Skv] keep-mask becomes an additive bias; rows whose keys are all masked return 0, :1552-1554) and the
 * segment-id masking of the flash wrappers (:390-438).
 *   key_bias     f32 [B, bias_stride]; bias_stride a multiple of 32 and >= Skv rounded up to 32 (entries at and
 *                past Skv are ignored); 16-byte aligned
 * Rows without any kept key give out = 0 and lse = -inf.
 */
int mdattn_fwd_bf16_bias(void* stream, const void* q, const void* k, const void* v, void* out, float* lse,
                         int B, int H, int Sq, int Skv, int D,
                         const mdattn_strides* q_strides, const mdattn_strides* k_strides,
                         const mdattn_strides* v_strides, const mdattn_strides* o_strides, float scale,
                         const float* key_bias, int64_t bias_stride);

/*
 * Keep-mask -> additive bias for mdattn_fwd_bf16_bias: bias[b, j] = keep[b, j] ? 0 : masked_value for j < Skv,
 * masked_value for the padding up to bias_stride.  Replaces: the mask canonicalisation of
 * models/attention_flax.py:1931-1939 (which uses -10000; the flash kernels exclude masked keys, i.e. -inf).
 *   keep         u8 [B, Skv] contiguous (non-zero = keep);  bias  f32 [B, bias_stride]
 */
int mdattn_key_mask_bias(void* stream, const void* keep, float* bias, int B, int Skv, int64_t bias_stride,
                         float masked_value);

/*
 * Per-tensor absmax quantisation bf16 -> OCP float8 e4m3fn (the benchmark's fp8 configuration; no reference
 * counterpart: the reference's fp8 is qwix quantisation of dense layers, pipelines/wan/wan_pipeline.py:581-626).
 *   x_bf16 [n] contiguous, x_fp8 [n] bytes,
 *   premul       constant multiplied into x before the (single) rounding to e4m3; 1.0f = none.  For q,
 *                scale * log2(e) here and scale = ln 2 in mdattn_fwd_fp8 carry the softmax scale at no cost.
 *   pow2_scale   non-zero: the scale is rounded up to a power of two (e4m3 is a floating-point format: no
 *                precision is lost, at most one binade of range).  With power-of-two q and k scales and the
 *                softmax scale carried by premul, mdattn_fwd_fp8 applies the whole logit scale through the
 *                MFMA's block-scale operand, saves its multiply per logit and can form P without exponentials
 *                (see mdattn_fwd_fp8's softmax_mode).
 *   scale_out f32[2] device: [0] = s with x * premul ~= x_fp8 * s (absmax(x * premul) / 448, or the next
 *                power of two), [1] = absmax(x) (scratch of the reduction)
 * n % 16 == 0.
 */
int mdattn_quant_e4m3(void* stream, const void* x_bf16, void* x_fp8, float* scale_out, int64_t n,
                      float premul, int pow2_scale);

/*
 * fp8-e4m3 attention forward: q8/k8/v8 are e4m3 bytes [B,S,H,D] by strides, *_scale device f32[1]
 * de-quantisation factors; P is re-quantised to e4m3 per tile before the PV MFMA; f32 accumulation;
 * bf16 out; lse as above.  Requires D == 128, or D == 64 (LTX-2's audio stream).
 * When scale * log2(e) * q_scale * k_scale is a power of two (see mdattn_quant_e4m3: premul, pow2_scale, and
 * scale = ln 2 here) the logit scale is applied inside the MFMAs and the softmax needs no multiply; the scales are
 * read on the device, so nothing has to be declared: the one kernel that is launched holds both code paths and every
 * wave takes the branch that the scales call for.
 *   softmax_mode  MDATTN_FP8_SOFTMAX_EXP2: P = e4m3(exp2(.)), the row sum over the unrounded P; lse is the exact
 *                 logsumexp of the quantised logits (usable as a partial for mdattn_merge).
 *                 MDATTN_FP8_SOFTMAX_BYTE_GRID: in the power-of-two case only (otherwise as EXP2), P is formed without
 *                 exponentials: the e4m3 byte of a probability is the integer round(8 * (log2-logit - reference) + 56),
 *                 i.e. P is a piecewise-linear exponential, exact at the powers of two and up to 6 % above them in
 *                 between (comparable to e4m3's own rounding); the row sum is taken over those P, so out is a properly
 *                 normalised average, and lse is corrected by the mean of the difference (log2 1.0404): within 0.08 of
 *                 the EXP2 lse for a row that a single key dominates, much closer otherwise.  12 % faster; meant for
 *                 callers that use `out` only.
 */
#define MDATTN_FP8_SOFTMAX_EXP2 0
#define MDATTN_FP8_SOFTMAX_BYTE_GRID 1
int mdattn_fwd_fp8(void* stream, const void* q8, const void* k8, const void* v8, void* out, float* lse,
                   int B, int H, int Sq, int Skv, int D,
                   const mdattn_strides* q_strides, const mdattn_strides* k_strides,
                   const mdattn_strides* v_strides, const mdattn_strides* o_strides, float scale,
                   const float* q_scale, const float* k_scale, const float* v_scale, int softmax_mode);

/*
 * mdattn_fwd_fp8 with the additive per-key bias of mdattn_fwd_bf16_bias (a key padding mask,
 * models/attention_flax.py:1926-1939): logits = scale * q.k (de-quantised) + key_bias[b, key]; rows without any kept
 * key give out = 0 and lse = -inf.  Always the exact-exponential softmax (MDATTN_FP8_SOFTMAX_EXP2 semantics), on the
 * path without a multiply per logit when the scales allow it, as for mdattn_fwd_fp8.  The tile's bias values travel
 * with the K/V tile, and key tiles whose bias is all zero (all but the last few, for a padding mask) skip the bias
 * arithmetic: a masked call costs a few per cent over an unmasked one.  key_bias as for mdattn_fwd_bf16_bias.
 */
int mdattn_fwd_fp8_bias(void* stream, const void* q8, const void* k8, const void* v8, void* out, float* lse,
                        int B, int H, int Sq, int Skv, int D,
                        const mdattn_strides* q_strides, const mdattn_strides* k_strides,
                        const mdattn_strides* v_strides, const mdattn_strides* o_strides, float scale,
                        const float* q_scale, const float* k_scale, const float* v_scale,
                        const float* key_bias, int64_t bias_stride);

/*
 * Backward of mdattn_fwd_bf16: dq, dk, dv from (q, k, v, out, dout, lse), non-causal, no mask.  Replaces: the
 * backward of the reference's attention kernels, contract in kernels/splash_attention/base.py:108-160
 * (`_attention_reference_custom_bwd`, "flash" form of di = rowsum(o * do)) and
 * kernels/splash_attention/splash_attention_kernel.py:1277-1600, with `scale` applied inside (logits = scale*q.k).
 *   dout, out    bf16 [B,Sq,H,D] by o_strides;  dq by q_strides;  dk by k_strides;  dv by v_strides
 *   lse          f32 [B,H,Sq] as written by the forward
 *   workspace    f32 device buffer of at least mdattn_bwd_workspace_floats(B,H,Sq) elements, 16-byte aligned;
 *                scratch of the call (per padded q row: -lse in log2 units and -rowsum(dout*out)), nothing to keep
 * Two passes, no atomics: dq; then dk and dv together.  When scale * log2(e) == 1 (the caller's q carries the softmax
 * scale, as for the forward) the logits need no multiply; dq is then the gradient for the q that was passed.
 * Requires D == 128 or D == 64 (LTX-2's audio stream); sequence strides below 2^23 elements and
 * B * H * ceil32(Sq) below 2^29 (MDATTN_E_UNSUPPORTED beyond).
 */
int64_t mdattn_bwd_workspace_floats(int B, int H, int Sq);
int mdattn_bwd_bf16(void* stream, const void* q, const void* k, const void* v, const void* out, const void* dout,
                    const float* lse, void* dq, void* dk, void* dv, float* workspace, int64_t workspace_floats,
                    int B, int H, int Sq, int Skv, int D,
                    const mdattn_strides* q_strides, const mdattn_strides* k_strides,
                    const mdattn_strides* v_strides, const mdattn_strides* o_strides, float scale);

/*
 * Backward of mdattn_fwd_bf16_bias: the same gradients with the additive per-key bias of the forward (a key padding
 * mask, models/attention_flax.py:1926-1939) inside the recomputed probabilities.  Masked keys (-inf) get dk = dv = 0;
 * query rows without any kept key (forward: out = 0, lse = -inf) get dq = 0 and contribute nothing.
 *   key_bias     f32 [B, bias_stride] as for mdattn_fwd_bf16_bias (entries past Skv are ignored)
 */
int mdattn_bwd_bf16_bias(void* stream, const void* q, const void* k, const void* v, const void* out, const void* dout,
                         const float* lse, void* dq, void* dk, void* dv, float* workspace, int64_t workspace_floats,
                         int B, int H, int Sq, int Skv, int D,
                         const mdattn_strides* q_strides, const mdattn_strides* k_strides,
                         const mdattn_strides* v_strides, const mdattn_strides* o_strides, float scale,
                         const float* key_bias, int64_t bias_stride);

/*
 * mdattn_bwd_bf16 for callers that cannot allocate device memory and have no workspace to hand over: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.
 * Same arguments and results as mdattn_bwd_bf16 without `workspace`: the lse / delta scratch lives in a device array
 * that is part of the library image (MDATTN_BWD_STATIC_MAX_FLOATS floats = 32 MiB, held by every GPU the library runs
 * on until the process ends).  Requests with mdattn_bwd_workspace_floats(B,H,Sq) above that limit (more than
 * 4,194,304 padded query rows over all batches and heads) return MDATTN_E_TOOBIG and launch nothing.  The call
 * allocates nothing and frees nothing.  All calls on one GPU share the array: calls that may overlap on one GPU (two
 * streams, two threads) race on it and must be serialised by the caller; calls on different GPUs are independent.
 * The device that `stream` belongs to must be the current device.
 * Warm-up: the first use on a device looks up the array's device address (hipGetSymbolAddress), which can make the
 * runtime load the library's code object and place the 32 MiB array -- not something to happen under graph capture or
 * in a no-allocation region.  Call mdattn_bwd_static_max_floats() once per device beforehand, with that device
 * current (it performs the lookup), or make one un-captured call of the entry point; after that the entry point only
 * enqueues kernels.
 */
#define MDATTN_BWD_STATIC_MAX_FLOATS (8 * 1024 * 1024)
int64_t mdattn_bwd_static_max_floats(void);
int mdattn_bwd_bf16_static(void* stream, const void* q, const void* k, const void* v, const void* out, const void* dout,
                           const float* lse, void* dq, void* dk, void* dv,
                           int B, int H, int Sq, int Skv, int D,
                           const mdattn_strides* q_strides, const mdattn_strides* k_strides,
                           const mdattn_strides* v_strides, const mdattn_strides* o_strides, float scale);

/*
 * In-place LSE-space merge of a normalised partial (o_cur, lse_cur) into the running
 * (o_run f32, lse_run f32); start from o_run = 0, lse_run = -1e30.
 * Replaces: kernels/splash_attention/ring_attention_kernel.py:1062-1073 (same result as the
 * (m,l,o) forms :1120-1130 and models/attention_flax.py:753-772).
 *   o_run  f32 [B,S,H,D] by run_strides; o_cur bf16 (cur_is_f32 == 0) or f32 by cur_strides
 *   lse_run, lse_cur f32 [B,H,S] contiguous
 */
int mdattn_merge(void* stream, float* o_run, float* lse_run, const void* o_cur, const float* lse_cur,
                 int cur_is_f32, int B, int H, int S, int D,
                 const mdattn_strides* run_strides, const mdattn_strides* cur_strides);

/*
 * mdattn_fwd_bf16 and mdattn_merge in one launch: attention of q against one K/V chunk, merged in LSE space into
 * the running (o_run, lse_run) pair by the attention kernel's own epilogue, so the chunk's (out, lse) never goes
 * to memory and its merge traffic hides behind the other workgroups' matrix work.  One ring step of the reference:
 * kernels/splash_attention/ring_attention_kernel.py:1045-1073 (attention on the visiting K/V shard, then the merge),
 * models/attention_flax.py:736-772.  Same result as the two calls, except that the chunk's output is not rounded to
 * bf16 before the merge (the reference's ring step merges its f32 numerator too, :1058-1065).  Start from o_run = 0, lse_run = -1e30; mdattn_finalize turns o_run into bf16.
 *   o_run  f32 [B,Sq,H,D] by run_strides (in floats; multiples of 8, 16-byte aligned base), lse_run f32 [B,H,Sq]
 *   q, k, v, scale, D as for mdattn_fwd_bf16
 */
int mdattn_fwd_bf16_merge(void* stream, const void* q, const void* k, const void* v, float* o_run, float* lse_run,
                          int B, int H, int Sq, int Skv, int D,
                          const mdattn_strides* q_strides, const mdattn_strides* k_strides,
                          const mdattn_strides* v_strides, const mdattn_strides* run_strides, float scale);

/* f32 -> bf16 cast of the merged numerator (the `.astype(q.dtype)` of ring_attention_kernel.py:1130).
 * n % 8 == 0, both contiguous. */
int mdattn_finalize(void* stream, const float* o_run, void* out_bf16, int64_t n);

#ifdef __cplusplus
}
#endif
#endif /* MDATTN_H_ */
