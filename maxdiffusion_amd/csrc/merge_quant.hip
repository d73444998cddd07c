// HBM-bound helpers around the attention kernel: LSE-space chunk merge, f32->bf16 finalize,
// per-tensor absmax e4m3 quantisation.
#include "mdattn_common.h"

namespace mdattn {

struct MergeArgs {
  float* o_run;
  float* lse_run;
  const void* o_cur;
  const float* lse_cur;
  int H, S;
  int64_t rows;  // B*H*S
  int h_fast;    // rows are walked with the head index fastest (what [B,S,H,D] storage wants) instead of the token index
  int64_t r_sb, r_ss, r_sh, c_sb, c_ss, c_sh;
};

// LPR = D/8 lanes per (b,h,s) row, all in one wave: every lane reads the row's two lse values
// in the same instruction, before lane 0 of the row overwrites lse_run.
template <int LPR, bool CUR_F32>
__global__ __launch_bounds__(256) void merge_kernel(MergeArgs a) {
  const int tid = threadIdx.x, lane = tid % LPR;
  const int64_t row = (int64_t)blockIdx.x * (256 / LPR) + tid / LPR;
  if (row >= a.rows) return;
  int s, h;
  int64_t b;
  if (a.h_fast) {  // consecutive rows of a workgroup are consecutive in memory
    h = (int)(row % a.H);
    const int64_t bs = row / a.H;
    s = (int)(bs % a.S);
    b = bs / a.S;
  } else {
    s = (int)(row % a.S);
    const int64_t bh = row / a.S;
    h = (int)(bh % a.H);
    b = bh / a.H;
  }
  const int64_t lidx = (b * a.H + h) * a.S + s;
  const float l1 = a.lse_run[lidx], l2 = a.lse_cur[lidx];
  float4* pr = reinterpret_cast<float4*>(a.o_run + b * a.r_sb + s * a.r_ss + h * a.r_sh) + 2 * lane;
  float4 r0 = pr[0], r1 = pr[1];
  float cur[8];
  if (CUR_F32) {
    const float4* pc = reinterpret_cast<const float4*>((const float*)a.o_cur + b * a.c_sb + s * a.c_ss + h * a.c_sh) + 2 * lane;
    float4 c0 = ld_nt(pc), c1 = ld_nt(pc + 1);
    cur[0] = c0.x; cur[1] = c0.y; cur[2] = c0.z; cur[3] = c0.w; cur[4] = c1.x; cur[5] = c1.y; cur[6] = c1.z; cur[7] = c1.w;
  } else {
    const uint4* pc = reinterpret_cast<const uint4*>((const unsigned short*)a.o_cur + b * a.c_sb + s * a.c_ss + h * a.c_sh) + lane;
    unpack8(ld_nt(pc), cur);
  }
  const float L = fmaxf(l1, l2);
  float w1 = 0.f, w2 = 0.f;
  if (L > -INFINITY) { w1 = expf(l1 - L); w2 = expf(l2 - L); }
  const float den = w1 + w2;
  const float inv = den > 0.f ? 1.0f / den : 0.f;
  w1 *= inv; w2 *= inv;
  r0.x = w1 * r0.x + w2 * cur[0]; r0.y = w1 * r0.y + w2 * cur[1]; r0.z = w1 * r0.z + w2 * cur[2]; r0.w = w1 * r0.w + w2 * cur[3];
  r1.x = w1 * r1.x + w2 * cur[4]; r1.y = w1 * r1.y + w2 * cur[5]; r1.z = w1 * r1.z + w2 * cur[6]; r1.w = w1 * r1.w + w2 * cur[7];
  pr[0] = r0; pr[1] = r1;
  if (lane == 0) a.lse_run[lidx] = den > 0.f ? L + logf(den) : L;
}

__global__ __launch_bounds__(256) void finalize_kernel(const float4* __restrict__ in, uint4* __restrict__ out, int64_t n8) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n8; i += (int64_t)gridDim.x * 256) {
    const float4 a = ld_nt(in + 2 * i), b = ld_nt(in + 2 * i + 1);
    const float f[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    st_nt(out + i, pack8(f));
  }
}

__global__ void zero2_kernel(float* p) { if (threadIdx.x < 2) p[threadIdx.x] = 0.f; }

// |x| of a non-negative-masked bf16 orders like its bit pattern, so the absmax is an integer max.  Eight independent
// 16-byte loads in flight per lane and trip; one atomic per workgroup (thousands of same-address atomics from every
// wave would cost as much as the read itself).
__global__ __launch_bounds__(256) void absmax_kernel(const uint4* __restrict__ x, int64_t n8, unsigned* amax_bits) {
  __shared__ unsigned wmax[4];
  unsigned m = 0;
  auto fold = [&](const uint4& u) {
    const unsigned w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const unsigned lo = (w[j] << 16) & 0x7FFF0000u, hi = w[j] & 0x7FFF0000u;
      m = max(m, max(lo, hi));
    }
  };
  const int64_t stride = (int64_t)gridDim.x * 256;
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  for (; i + 7 * stride < n8; i += 8 * stride) {
    uint4 u[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) u[j] = ld_nt(x + i + j * stride);
#pragma unroll
    for (int j = 0; j < 8; ++j) fold(u[j]);
  }
  for (; i < n8; i += stride) fold(x[i]);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) m = max(m, (unsigned)__shfl_xor((int)m, o));
  if ((threadIdx.x & 63) == 0) wmax[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
    m = max(max(wmax[0], wmax[1]), max(wmax[2], wmax[3]));
    if (m) atomicMax(amax_bits, m);
  }
}

// x8 = e4m3(x * premul / s) with s = absmax(x * premul) / 448, or the next power of two above it (pow2): a
// power-of-two scale costs e4m3, a floating-point format, no precision, only up to one binade of its range.
__global__ __launch_bounds__(256) void quant_kernel(const uint4* __restrict__ x, uint4* __restrict__ y, int64_t n16, float* scale,
                                                    float premul, int pow2) {
  float amax = scale[1] * premul;
  amax = amax > 1e-12f ? amax : 1e-12f;
  float s = amax * (1.0f / 448.0f);
  if (pow2) {
    const unsigned b = __float_as_uint(s);
    s = __uint_as_float(((b & 0x007FFFFFu) ? b + 0x00800000u : b) & 0x7F800000u);
  }
  const float r = premul / s;
  if (blockIdx.x == 0 && threadIdx.x == 0) scale[0] = s;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (int64_t)gridDim.x * 256) {
    float f[16];
    unpack8(x[2 * i], f);
    unpack8(x[2 * i + 1], f + 8);
    unsigned o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float v[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) v[t] = fminf(fmaxf(f[4 * j + t] * r, -448.f), 448.f);
      int pk = 0;
      pk = __builtin_amdgcn_cvt_pk_fp8_f32(v[0], v[1], pk, false);
      pk = __builtin_amdgcn_cvt_pk_fp8_f32(v[2], v[3], pk, true);
      o[j] = (unsigned)pk;
    }
    y[i] = make_uint4(o[0], o[1], o[2], o[3]);
  }
}

}  // namespace mdattn

using namespace mdattn;

extern "C" int mdattn_merge(void* stream, float* o_run, float* lse_run, const void* o_cur, const float* lse_cur,
                            int cur_is_f32, int B, int H, int S, int D,
                            const mdattn_strides* run_strides, const mdattn_strides* cur_strides) {
  if (!o_run || !lse_run || !o_cur || !lse_cur || B <= 0 || H <= 0 || S <= 0 || D <= 0) return MDATTN_E_BADARG;
  if (!run_strides || !cur_strides) return MDATTN_E_BADARG;
  if (D != 64 && D != 128 && D != 256) return MDATTN_E_UNSUPPORTED;
  if (!aligned16(o_run) || !aligned16(o_cur) || (reinterpret_cast<uintptr_t>(lse_run) & 3u) || (reinterpret_cast<uintptr_t>(lse_cur) & 3u))
    return MDATTN_E_ALIGN;
  if (!strides_ok(run_strides, 8) || !strides_ok(cur_strides, 8)) return MDATTN_E_ALIGN;
  MergeArgs a;
  a.o_run = o_run; a.lse_run = lse_run; a.o_cur = o_cur; a.lse_cur = lse_cur;
  a.H = H; a.S = S; a.rows = (int64_t)B * H * S;
  a.h_fast = run_strides->head < run_strides->seq;
  a.r_sb = run_strides->batch; a.r_ss = run_strides->seq; a.r_sh = run_strides->head;
  a.c_sb = cur_strides->batch; a.c_ss = cur_strides->seq; a.c_sh = cur_strides->head;
  const int lpr = D / 8;
  const int64_t nblocks = (a.rows + (256 / lpr) - 1) / (256 / lpr);
  if (nblocks > 0x7FFFFFFF) return MDATTN_E_UNSUPPORTED;
  dim3 grid((unsigned)nblocks), block(256);
  hipStream_t st = (hipStream_t)stream;
#define MDATTN_MERGE_CASE(L)                                                          \
  if (lpr == L) {                                                                     \
    if (cur_is_f32) MDATTN_LAUNCH((merge_kernel<L, true>), grid, block, 0, st, a); \
    else MDATTN_LAUNCH((merge_kernel<L, false>), grid, block, 0, st, a);           \
  }
  MDATTN_MERGE_CASE(8) MDATTN_MERGE_CASE(16) MDATTN_MERGE_CASE(32)
#undef MDATTN_MERGE_CASE
  return launch_status();
}

extern "C" int mdattn_finalize(void* stream, const float* o_run, void* out_bf16, int64_t n) {
  if (!o_run || !out_bf16 || n <= 0) return MDATTN_E_BADARG;
  if (n % 8) return MDATTN_E_UNSUPPORTED;
  if (!aligned16(o_run) || !aligned16(out_bf16)) return MDATTN_E_ALIGN;
  const int64_t n8 = n / 8;
  const unsigned grid = (unsigned)((n8 + 255) / 256 < 65536 ? (n8 + 255) / 256 : 65536);
  MDATTN_LAUNCH(finalize_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream, (const float4*)o_run, (uint4*)out_bf16, n8);
  return launch_status();
}

extern "C" int mdattn_quant_e4m3(void* stream, const void* x_bf16, void* x_fp8, float* scale_out, int64_t n,
                                 float premul, int pow2_scale) {
  if (!x_bf16 || !x_fp8 || !scale_out || n <= 0) return MDATTN_E_BADARG;
  if (!(premul > 0.f) || !(premul < 1e30f)) return MDATTN_E_BADARG;
  if (n % 16) return MDATTN_E_UNSUPPORTED;
  if (!aligned16(x_bf16) || !aligned16(x_fp8) || (reinterpret_cast<uintptr_t>(scale_out) & 7u)) return MDATTN_E_ALIGN;
  hipStream_t st = (hipStream_t)stream;
  const int64_t n8 = n / 8, n16 = n / 16;
  const unsigned g1 = (unsigned)((n8 + 255) / 256 < 2048 ? (n8 + 255) / 256 : 2048);
  const unsigned g2 = (unsigned)((n16 + 255) / 256 < 16384 ? (n16 + 255) / 256 : 16384);
  MDATTN_LAUNCH(zero2_kernel, dim3(1), dim3(64), 0, st, scale_out);
  if (launch_status() != MDATTN_OK) return MDATTN_E_LAUNCH;
  MDATTN_LAUNCH(absmax_kernel, dim3(g1), dim3(256), 0, st, (const uint4*)x_bf16, n8, (unsigned*)(scale_out + 1));
  if (launch_status() != MDATTN_OK) return MDATTN_E_LAUNCH;
  MDATTN_LAUNCH(quant_kernel, dim3(g2), dim3(256), 0, st, (const uint4*)x_bf16, (uint4*)x_fp8, n16, scale_out,
                     premul, pow2_scale);
  return launch_status();
}

// ------------------------------------------------------------------------------------------- key mask -> bias
namespace mdattn {
__global__ __launch_bounds__(256) void key_mask_bias_kernel(const uint8_t* __restrict__ keep, float* __restrict__ bias,
                                                            int Skv, int64_t bias_stride, float masked_value) {
  const int b = blockIdx.y;
  for (int64_t j = (int64_t)blockIdx.x * 256 + threadIdx.x; j < bias_stride; j += (int64_t)gridDim.x * 256)
    bias[b * bias_stride + j] = (j < Skv && keep[(int64_t)b * Skv + j]) ? 0.f : masked_value;
}
}  // namespace mdattn

extern "C" int mdattn_key_mask_bias(void* stream, const void* keep, float* bias, int B, int Skv, int64_t bias_stride,
                                    float masked_value) {
  if (!keep || !bias || B <= 0 || Skv <= 0 || bias_stride < Skv) return MDATTN_E_BADARG;
  if (B > 65535) return MDATTN_E_UNSUPPORTED;
  const unsigned gx = (unsigned)((bias_stride + 255) / 256 < 1024 ? (bias_stride + 255) / 256 : 1024);
  MDATTN_LAUNCH(mdattn::key_mask_bias_kernel, dim3(gx, B), dim3(256), 0, (hipStream_t)stream,
                     (const uint8_t*)keep, bias, Skv, bias_stride, masked_value);
  return mdattn::launch_status();
}
