// Fused q/k RMSNorm + interleaved-pair RoPE for gfx950.  HBM-bound: every q and k element is
// read once (16-byte loads) and written once (16-byte stores); statistics, scale and rotation
// are f32 in registers with a single rounding to bf16.
#include "mdattn_common.h"

namespace mdattn {

struct NormRopeFullArgs {
  const uint4* x_in[2];   // q, k  (k may be null)
  uint4* x_out[2];
  const uint4* w[2];
  const float4* cos;
  const float4* sin;
  int S, H, D, N;         // N = H*D
  float eps, inv_n;
  float q_mul;            // constant folded into the q output before its rounding
  int64_t in_sb, in_ss;
  int64_t out_sb, out_ss, out_sh;
  // FUSED (mdattn_norm_rope_qkv): the projection biases still to be added (null: none), and the value block
  const uint4* bias[3];   // q, k, v
  const uint4* v_in;
  uint4* v_out;           // null: v is left where it is
};

// One workgroup (256 lanes) per token row; lane t owns 16-byte chunks t, t+256, ... (<= MAXC).
// FUSED: the row is the output of a fused q|k|v projection; the projection biases are added in f32 before the
// statistics, and the value block is passed through (bias added, laid out like q and k) in the same launch.
template <int MAXC, bool FUSED = false>
__global__ __launch_bounds__(256) void norm_rope_fullrow_kernel(NormRopeFullArgs a) {
  const int tid = threadIdx.x;
  const int s = blockIdx.x, b = blockIdx.y;
  const int nchunks = a.N >> 3;
  const int ntens = a.x_in[1] ? 2 : 1;
  __shared__ float red[2][16];

  uint4 raw[2][MAXC];
  float ss[2] = {0.f, 0.f};
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    if (t < ntens) {
      const uint4* row = a.x_in[t] + ((b * a.in_sb + s * a.in_ss) >> 3);
#pragma unroll
      for (int i = 0; i < MAXC; ++i) {
        const int c = tid + i * 256;
        if (c < nchunks) raw[t][i] = ld_nt(row + c);
      }
    }
  }
  [[maybe_unused]] uint4 vraw[MAXC];
  if constexpr (FUSED) {
    if (a.v_out) {
      const uint4* row = a.v_in + ((b * a.in_sb + s * a.in_ss) >> 3);
#pragma unroll
      for (int i = 0; i < MAXC; ++i) {
        const int c = tid + i * 256;
        if (c < nchunks) vraw[i] = ld_nt(row + c);
      }
    }
  }
  // value of chunk c of tensor t as the statistics and the output see it: the projection plus its bias
  auto chunk_f32 = [&](int t, int i, int c, float* f) __attribute__((always_inline)) {
    unpack8(raw[t][i], f);
    if constexpr (FUSED) {
      if (a.bias[t]) {
        float bb[8];
        unpack8(a.bias[t][c], bb);
#pragma unroll
        for (int j = 0; j < 8; ++j) f[j] += bb[j];
      }
    }
  };
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    if (t < ntens) {
#pragma unroll
      for (int i = 0; i < MAXC; ++i) {
        const int c = tid + i * 256;
        if (c < nchunks) {
          float f[8];
          chunk_f32(t, i, c, f);
#pragma unroll
          for (int j = 0; j < 8; ++j) ss[t] = __builtin_fmaf(f[j], f[j], ss[t]);
        }
      }
      ss[t] = row16_sum(ss[t]);
      if ((tid & 15) == 0) red[t][tid >> 4] = ss[t];
    }
  }
  __syncthreads();
  float inv[2] = {0.f, 0.f};
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    if (t < ntens) {
      float tot = 0.f;
#pragma unroll
      for (int j = 0; j < 16; ++j) tot += red[t][j];
      const float x = tot * a.inv_n + a.eps;
      const float y = __builtin_amdgcn_rsqf(x);
      // one Newton step brings v_rsq_f32 (1 ulp) to f32 round-off: y*(1.5 - 0.5*x*y*y)
      inv[t] = y * (1.5f - 0.5f * x * y * y);
      if (t == 0) inv[t] *= a.q_mul;
    }
  }

  const bool rope = a.cos != nullptr;
  const int halfd4 = a.D >> 3;  // float4 chunks per table row
#pragma unroll
  for (int i = 0; i < MAXC; ++i) {
    const int c = tid + i * 256;
    if (c < nchunks) {
      const int e = c << 3;
      const int h = e / a.D, d = e - h * a.D;
      float4 cs = {1.f, 1.f, 1.f, 1.f}, sn = {0.f, 0.f, 0.f, 0.f};
      if (rope) {
        cs = a.cos[(int64_t)s * halfd4 + (d >> 3)];
        sn = a.sin[(int64_t)s * halfd4 + (d >> 3)];
      }
      const float cc[4] = {cs.x, cs.y, cs.z, cs.w}, sv[4] = {sn.x, sn.y, sn.z, sn.w};
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        if (t < ntens) {
          float f[8], w[8], o[8];
          chunk_f32(t, i, c, f);
          unpack8(a.w[t][c], w);
#pragma unroll
          for (int j = 0; j < 8; ++j) f[j] = f[j] * inv[t] * w[j];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            o[2 * j] = f[2 * j] * cc[j] - f[2 * j + 1] * sv[j];
            o[2 * j + 1] = f[2 * j] * sv[j] + f[2 * j + 1] * cc[j];
          }
          uint4* dst = a.x_out[t] + ((b * a.out_sb + s * a.out_ss + h * a.out_sh + d) >> 3);
          st_nt(dst, pack8(o));
        }
      }
      if constexpr (FUSED) {
        if (a.v_out) {
          uint4 u = vraw[i];
          if (a.bias[2]) {
            float f[8], bb[8];
            unpack8(u, f);
            unpack8(a.bias[2][c], bb);
#pragma unroll
            for (int j = 0; j < 8; ++j) f[j] += bb[j];
            u = pack8(f);
          }
          st_nt(a.v_out + ((b * a.out_sb + s * a.out_ss + h * a.out_sh + d) >> 3), u);
        }
      }
    }
  }
}

struct NormRopeHeadArgs {
  const uint4* x_in[2];
  uint4* x_out[2];
  const uint4* w[2];
  const uint4* w_txt[2];
  const float4* cos;
  const float4* sin;
  int S, H, n_txt;
  int64_t rows;  // B*S*H
  float eps;
  float q_mul;   // constant folded into the q output before its rounding
  int64_t in_sb, in_ss, in_sh, out_sb, out_ss, out_sh;
};

// LPR = D/8 lanes per (token, head) row; each lane owns one 16-byte chunk; RPT rows per lane group
// in flight so that enough bytes are outstanding per CU.
template <int LPR, int RPT>
__global__ __launch_bounds__(256) void norm_rope_perhead_kernel(NormRopeHeadArgs a) {
  constexpr int D = LPR * 8;
  constexpr int GROUPS = 256 / LPR;
  const int tid = threadIdx.x;
  const int lane = tid % LPR;
  const int64_t row0 = ((int64_t)blockIdx.x * GROUPS + tid / LPR) * RPT;
  const int ntens = a.x_in[1] ? 2 : 1;
  const bool rope = a.cos != nullptr;

  uint4 raw[2][RPT];
  int64_t oofs[RPT];
  int tok[RPT];
#pragma unroll
  for (int r = 0; r < RPT; ++r) {
    int64_t row = row0 + r;
    if (row >= a.rows) row = a.rows - 1;  // clamp loads; stores are predicated below
    const int h = (int)(row % a.H);
    const int64_t bs = row / a.H;
    const int s = (int)(bs % a.S);
    const int64_t b = bs / a.S;
    tok[r] = s;
    oofs[r] = b * a.out_sb + s * a.out_ss + h * a.out_sh;
    const int64_t iofs = b * a.in_sb + s * a.in_ss + h * a.in_sh;
#pragma unroll
    for (int t = 0; t < 2; ++t)
      if (t < ntens) raw[t][r] = ld_nt(a.x_in[t] + (iofs >> 3) + lane);
  }
#pragma unroll
  for (int r = 0; r < RPT; ++r) {
    float4 cs = {1.f, 1.f, 1.f, 1.f}, sn = {0.f, 0.f, 0.f, 0.f};
    if (rope) {
      cs = a.cos[(int64_t)tok[r] * LPR + lane];
      sn = a.sin[(int64_t)tok[r] * LPR + lane];
    }
    const float cc[4] = {cs.x, cs.y, cs.z, cs.w}, sv[4] = {sn.x, sn.y, sn.z, sn.w};
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      if (t < ntens) {
        float f[8], w[8], o[8];
        unpack8(raw[t][r], f);
        float ss = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) ss = __builtin_fmaf(f[j], f[j], ss);
        if (LPR >= 16) {
          ss = row16_sum(ss);
          if (LPR == 32) ss += __shfl_xor(ss, 16);
        } else {  // LPR == 8
          ss += __shfl_xor(ss, 1); ss += __shfl_xor(ss, 2); ss += __shfl_xor(ss, 4);
        }
        const float x = ss * (1.0f / D) + a.eps;
        float inv = __builtin_amdgcn_rsqf(x);
        inv = inv * (1.5f - 0.5f * x * inv * inv);
        if (t == 0) inv *= a.q_mul;
        const uint4* wp = (a.w_txt[t] && tok[r] < a.n_txt) ? a.w_txt[t] : a.w[t];
        unpack8(wp[lane], w);
#pragma unroll
        for (int j = 0; j < 8; ++j) f[j] = f[j] * inv * w[j];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          o[2 * j] = f[2 * j] * cc[j] - f[2 * j + 1] * sv[j];
          o[2 * j + 1] = f[2 * j] * sv[j] + f[2 * j + 1] * cc[j];
        }
        if (row0 + r < a.rows) st_nt(a.x_out[t] + (oofs[r] >> 3) + lane, pack8(o));
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------
// One tensor at a time, with position tables that differ per batch element and per head (LTX-2):
// full-row RMSNorm with an f32 weight, then either the interleaved rotation with full-size tables
// [B,S,H*D] (out = x*cos + rot(x)*sin, rot pairs neighbours as (-x1, x0)) or the split rotation with
// tables [B,H,S,D/2] (element i of a head pairs with element i + D/2).  A lane works on "units" of two
// 8-element chunks of one head, c and c + D/16, which holds both partners of either pairing.
struct NormRopeRowsArgs {
  const void* x_in;
  uint4* x_out;
  const float* w;
  const float* cos;
  const float* sin;
  int S, H, D, N, mode;  // mode 0: no rotation, 1: interleaved, 2: split
  float eps, inv_n;
  int64_t in_sb, in_ss;
  int64_t out_sb, out_ss, out_sh;
};

template <int MAXU, bool F32IN>
__global__ __launch_bounds__(256) void norm_rope_rows_kernel(NormRopeRowsArgs a) {
  const int tid = threadIdx.x;
  const int s = blockIdx.x, b = blockIdx.y;
  const int cph = a.D >> 4;            // chunk pairs (units) per head
  const int nunits = a.H * cph;
  __shared__ float red[16];

  float x[MAXU][16];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < MAXU; ++i) {
    const int u = tid + i * 256;
    if (u < nunits) {
      const int h = u / cph, c = u - h * cph;
      const int64_t e0 = b * a.in_sb + s * a.in_ss + h * a.D + c * 8;  // first chunk; partner at + D/2
      if (F32IN) {
        const float4* p0 = reinterpret_cast<const float4*>(static_cast<const float*>(a.x_in) + e0);
        const float4* p1 = reinterpret_cast<const float4*>(static_cast<const float*>(a.x_in) + e0 + (a.D >> 1));
        const float4 v0 = ld_nt(p0), v1 = ld_nt(p0 + 1), v2 = ld_nt(p1), v3 = ld_nt(p1 + 1);
        const float t[16] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w, v2.x, v2.y, v2.z, v2.w, v3.x, v3.y, v3.z, v3.w};
#pragma unroll
        for (int j = 0; j < 16; ++j) x[i][j] = t[j];
      } else {
        const uint4* p = reinterpret_cast<const uint4*>(static_cast<const __bf16*>(a.x_in) + e0);
        unpack8(ld_nt(p), x[i]);
        unpack8(ld_nt(p + (a.D >> 4)), x[i] + 8);
      }
#pragma unroll
      for (int j = 0; j < 16; ++j) ss = __builtin_fmaf(x[i][j], x[i][j], ss);
    }
  }
  ss = row16_sum(ss);
  if ((tid & 15) == 0) red[tid >> 4] = ss;
  __syncthreads();
  float tot = 0.f;
#pragma unroll
  for (int j = 0; j < 16; ++j) tot += red[j];
  const float xx = tot * a.inv_n + a.eps;
  const float y0 = __builtin_amdgcn_rsqf(xx);
  const float inv = y0 * (1.5f - 0.5f * xx * y0 * y0);

#pragma unroll
  for (int i = 0; i < MAXU; ++i) {
    const int u = tid + i * 256;
    if (u < nunits) {
      const int h = u / cph, c = u - h * cph;
      const int half = a.D >> 1;
      const float4* wp0 = reinterpret_cast<const float4*>(a.w + h * a.D + c * 8);
      const float4* wp1 = reinterpret_cast<const float4*>(a.w + h * a.D + c * 8 + half);
      const float4 w0 = wp0[0], w1 = wp0[1], w2 = wp1[0], w3 = wp1[1];
      const float w[16] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w, w2.x, w2.y, w2.z, w2.w, w3.x, w3.y, w3.z, w3.w};
      float y[16], o[16];
#pragma unroll
      for (int j = 0; j < 16; ++j) y[j] = x[i][j] * inv * w[j];
      if (a.mode == 1) {
        // tables [B,S,H*D]: one cos and one sin per element
        const int64_t t0 = ((int64_t)b * a.S + s) * a.N + h * a.D + c * 8;
#pragma unroll
        for (int part = 0; part < 2; ++part) {
          const float4* cp = reinterpret_cast<const float4*>(a.cos + t0 + part * half);
          const float4* sp = reinterpret_cast<const float4*>(a.sin + t0 + part * half);
          const float4 c0 = cp[0], c1 = cp[1], s0 = sp[0], s1 = sp[1];
          const float cc[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
          const float sv[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float x0 = y[part * 8 + 2 * j], x1 = y[part * 8 + 2 * j + 1];
            o[part * 8 + 2 * j] = x0 * cc[2 * j] - x1 * sv[2 * j];
            o[part * 8 + 2 * j + 1] = x1 * cc[2 * j + 1] + x0 * sv[2 * j + 1];
          }
        }
      } else if (a.mode == 2) {
        // tables [B,H,S,D/2]: element c*8+e of the first half pairs with the same element of the second half
        const int64_t t0 = (((int64_t)b * a.H + h) * a.S + s) * half + c * 8;
        const float4* cp = reinterpret_cast<const float4*>(a.cos + t0);
        const float4* sp = reinterpret_cast<const float4*>(a.sin + t0);
        const float4 c0 = cp[0], c1 = cp[1], s0 = sp[0], s1 = sp[1];
        const float cc[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
        const float sv[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          o[j] = y[j] * cc[j] - y[8 + j] * sv[j];
          o[8 + j] = y[8 + j] * cc[j] + y[j] * sv[j];
        }
      } else {
#pragma unroll
        for (int j = 0; j < 16; ++j) o[j] = y[j];
      }
      uint4* dst = a.x_out + ((b * a.out_sb + s * a.out_ss + h * a.out_sh + c * 8) >> 3);
      st_nt(dst, pack8(o));
      st_nt(dst + (a.D >> 4), pack8(o + 8));
    }
  }
}

}  // namespace mdattn

using namespace mdattn;

extern "C" int mdattn_norm_rope_fullrow(void* stream, const void* q_in, const void* k_in, void* q_out, void* k_out,
                                        const void* wq, const void* wk, const float* cos, const float* sin,
                                        int B, int S, int H, int D, float eps, float q_mul,
                                        int64_t in_stride_batch, int64_t in_stride_seq,
                                        const mdattn_strides* out_strides) {
  if (!q_in || !q_out || !wq || B <= 0 || S <= 0 || H <= 0 || D <= 0 || !out_strides) return MDATTN_E_BADARG;
  if ((k_in == nullptr) != (k_out == nullptr) || (k_in && !wk)) return MDATTN_E_BADARG;
  if ((cos == nullptr) != (sin == nullptr)) return MDATTN_E_BADARG;
  if (!(eps >= 0.f) || !(q_mul > 0.f) || !(q_mul < 1e30f)) return MDATTN_E_BADARG;
  const int64_t N = (int64_t)H * D;
  if (D % 8 != 0 || N > 8192) return MDATTN_E_UNSUPPORTED;
  if (B > 65535) return MDATTN_E_UNSUPPORTED;
  if (in_stride_seq < N || in_stride_batch < 0) return MDATTN_E_BADARG;
  if (!aligned16(q_in) || !aligned16(q_out) || !aligned16(wq) || !aligned16(k_in) || !aligned16(k_out) ||
      !aligned16(wk) || !aligned16(cos) || !aligned16(sin))
    return MDATTN_E_ALIGN;
  if (in_stride_batch % 8 || in_stride_seq % 8 || !strides_ok(out_strides, 8)) return MDATTN_E_ALIGN;

  NormRopeFullArgs a;
  a.x_in[0] = (const uint4*)q_in; a.x_in[1] = (const uint4*)k_in;
  a.x_out[0] = (uint4*)q_out; a.x_out[1] = (uint4*)k_out;
  a.w[0] = (const uint4*)wq; a.w[1] = (const uint4*)wk;
  a.cos = (const float4*)cos; a.sin = (const float4*)sin;
  a.S = S; a.H = H; a.D = D; a.N = (int)N; a.eps = eps; a.inv_n = 1.0f / (float)N; a.q_mul = q_mul;
  a.in_sb = in_stride_batch; a.in_ss = in_stride_seq;
  a.out_sb = out_strides->batch; a.out_ss = out_strides->seq; a.out_sh = out_strides->head;
  a.bias[0] = a.bias[1] = a.bias[2] = nullptr; a.v_in = nullptr; a.v_out = nullptr;
  dim3 grid(S, B), block(256);
  hipStream_t st = (hipStream_t)stream;
  const int nchunks = (int)(N / 8);
  if (nchunks <= 256) MDATTN_LAUNCH(norm_rope_fullrow_kernel<1>, grid, block, 0, st, a);
  else if (nchunks <= 512) MDATTN_LAUNCH(norm_rope_fullrow_kernel<2>, grid, block, 0, st, a);
  else if (nchunks <= 768) MDATTN_LAUNCH(norm_rope_fullrow_kernel<3>, grid, block, 0, st, a);
  else MDATTN_LAUNCH(norm_rope_fullrow_kernel<4>, grid, block, 0, st, a);
  return launch_status();
}

extern "C" int mdattn_norm_rope_qkv(void* stream, const void* qkv, const void* bias, void* q_out, void* k_out, void* v_out,
                                    const void* wq, const void* wk, const float* cos, const float* sin,
                                    int B, int S, int H, int D, float eps, float q_mul,
                                    int64_t qkv_stride_batch, int64_t qkv_stride_seq, const mdattn_strides* out_strides) {
  if (!qkv || !q_out || !k_out || !wq || !wk || B <= 0 || S <= 0 || H <= 0 || D <= 0 || !out_strides) return MDATTN_E_BADARG;
  if ((cos == nullptr) != (sin == nullptr)) return MDATTN_E_BADARG;
  if (bias && !v_out) return MDATTN_E_BADARG;  // the value block needs its bias too: it cannot stay where it is
  if (!(eps >= 0.f) || !(q_mul > 0.f) || !(q_mul < 1e30f)) return MDATTN_E_BADARG;
  const int64_t N = (int64_t)H * D;
  if (D % 8 != 0 || N > 8192) return MDATTN_E_UNSUPPORTED;
  if (B > 65535) return MDATTN_E_UNSUPPORTED;
  if (qkv_stride_seq < 3 * N || qkv_stride_batch < 0) return MDATTN_E_BADARG;
  if (!aligned16(qkv) || !aligned16(bias) || !aligned16(q_out) || !aligned16(k_out) || !aligned16(v_out) || !aligned16(wq) ||
      !aligned16(wk) || !aligned16(cos) || !aligned16(sin))
    return MDATTN_E_ALIGN;
  if (qkv_stride_batch % 8 || qkv_stride_seq % 8 || !strides_ok(out_strides, 8)) return MDATTN_E_ALIGN;

  NormRopeFullArgs a;
  const uint4* base = (const uint4*)qkv;
  a.x_in[0] = base; a.x_in[1] = base + N / 8; a.v_in = base + 2 * N / 8;
  a.x_out[0] = (uint4*)q_out; a.x_out[1] = (uint4*)k_out; a.v_out = (uint4*)v_out;
  a.w[0] = (const uint4*)wq; a.w[1] = (const uint4*)wk;
  const uint4* bb = (const uint4*)bias;
  a.bias[0] = bb; a.bias[1] = bb ? bb + N / 8 : nullptr; a.bias[2] = bb ? bb + 2 * N / 8 : nullptr;
  a.cos = (const float4*)cos; a.sin = (const float4*)sin;
  a.S = S; a.H = H; a.D = D; a.N = (int)N; a.eps = eps; a.inv_n = 1.0f / (float)N; a.q_mul = q_mul;
  a.in_sb = qkv_stride_batch; a.in_ss = qkv_stride_seq;
  a.out_sb = out_strides->batch; a.out_ss = out_strides->seq; a.out_sh = out_strides->head;
  dim3 grid(S, B), block(256);
  hipStream_t st = (hipStream_t)stream;
  const int nchunks = (int)(N / 8);
  if (nchunks <= 256) MDATTN_LAUNCH((norm_rope_fullrow_kernel<1, true>), grid, block, 0, st, a);
  else if (nchunks <= 512) MDATTN_LAUNCH((norm_rope_fullrow_kernel<2, true>), grid, block, 0, st, a);
  else if (nchunks <= 768) MDATTN_LAUNCH((norm_rope_fullrow_kernel<3, true>), grid, block, 0, st, a);
  else MDATTN_LAUNCH((norm_rope_fullrow_kernel<4, true>), grid, block, 0, st, a);
  return launch_status();
}

extern "C" int mdattn_norm_rope_perhead(void* stream, const void* q_in, const void* k_in, void* q_out, void* k_out,
                                        const void* wq, const void* wk, const void* wq_txt, const void* wk_txt,
                                        int n_txt, const float* cos, const float* sin, int B, int S, int H, int D,
                                        float eps, float q_mul, const mdattn_strides* in_strides,
                                        const mdattn_strides* out_strides) {
  if (!q_in || !q_out || !wq || B <= 0 || S <= 0 || H <= 0 || D <= 0 || !in_strides || !out_strides) return MDATTN_E_BADARG;
  if ((k_in == nullptr) != (k_out == nullptr) || (k_in && !wk)) return MDATTN_E_BADARG;
  if ((cos == nullptr) != (sin == nullptr)) return MDATTN_E_BADARG;
  if (n_txt < 0 || n_txt > S || !(eps >= 0.f) || !(q_mul > 0.f) || !(q_mul < 1e30f)) return MDATTN_E_BADARG;
  if (D != 64 && D != 128 && D != 256) return MDATTN_E_UNSUPPORTED;
  if (!aligned16(q_in) || !aligned16(q_out) || !aligned16(wq) || !aligned16(k_in) || !aligned16(k_out) ||
      !aligned16(wk) || !aligned16(wq_txt) || !aligned16(wk_txt) || !aligned16(cos) || !aligned16(sin))
    return MDATTN_E_ALIGN;
  if (!strides_ok(in_strides, 8) || !strides_ok(out_strides, 8)) return MDATTN_E_ALIGN;

  NormRopeHeadArgs a;
  a.x_in[0] = (const uint4*)q_in; a.x_in[1] = (const uint4*)k_in;
  a.x_out[0] = (uint4*)q_out; a.x_out[1] = (uint4*)k_out;
  a.w[0] = (const uint4*)wq; a.w[1] = (const uint4*)wk;
  a.w_txt[0] = (const uint4*)wq_txt; a.w_txt[1] = k_in ? (const uint4*)wk_txt : nullptr;
  a.cos = (const float4*)cos; a.sin = (const float4*)sin;
  a.S = S; a.H = H; a.n_txt = n_txt; a.rows = (int64_t)B * S * H; a.eps = eps; a.q_mul = q_mul;
  a.in_sb = in_strides->batch; a.in_ss = in_strides->seq; a.in_sh = in_strides->head;
  a.out_sb = out_strides->batch; a.out_ss = out_strides->seq; a.out_sh = out_strides->head;
  constexpr int RPT = 4;
  const int lpr = D / 8;
  const int64_t rows_per_block = (256 / lpr) * RPT;
  const int64_t nblocks = (a.rows + rows_per_block - 1) / rows_per_block;
  if (nblocks > 0x7FFFFFFF) return MDATTN_E_UNSUPPORTED;
  dim3 grid((unsigned)nblocks), block(256);
  hipStream_t st = (hipStream_t)stream;
  if (lpr == 8) MDATTN_LAUNCH((norm_rope_perhead_kernel<8, RPT>), grid, block, 0, st, a);
  else if (lpr == 16) MDATTN_LAUNCH((norm_rope_perhead_kernel<16, RPT>), grid, block, 0, st, a);
  else MDATTN_LAUNCH((norm_rope_perhead_kernel<32, RPT>), grid, block, 0, st, a);
  return launch_status();
}

extern "C" int mdattn_norm_rope_rows(void* stream, const void* x_in, int x_is_f32, void* x_out, const float* w,
                                     const float* cos, const float* sin, int rope_mode, int B, int S, int H, int D,
                                     float eps, int64_t in_stride_batch, int64_t in_stride_seq,
                                     const mdattn_strides* out_strides) {
  if (!x_in || !x_out || !w || B <= 0 || S <= 0 || H <= 0 || D <= 0 || !out_strides) return MDATTN_E_BADARG;
  if (rope_mode < 0 || rope_mode > 2 || (rope_mode != 0 && (!cos || !sin)) || !(eps >= 0.f)) return MDATTN_E_BADARG;
  if (B > 65535) return MDATTN_E_UNSUPPORTED;
  if (D % 16 != 0) return MDATTN_E_UNSUPPORTED;
  const int64_t N = (int64_t)H * D;
  if (N / 16 > 2 * 256) return MDATTN_E_UNSUPPORTED;  // up to 8192 channels per row
  const int in_mult = x_is_f32 ? 4 : 8;
  if (!aligned16(x_in) || !aligned16(x_out) || !aligned16(w) || !aligned16(cos) || !aligned16(sin)) return MDATTN_E_ALIGN;
  if (in_stride_batch % in_mult || in_stride_seq % in_mult || in_stride_seq < N || !strides_ok(out_strides, 8)) return MDATTN_E_ALIGN;
  if (out_strides->head < D) return MDATTN_E_BADARG;
  NormRopeRowsArgs a;
  a.x_in = x_in; a.x_out = (uint4*)x_out; a.w = w; a.cos = cos; a.sin = sin;
  a.S = S; a.H = H; a.D = D; a.N = (int)N; a.mode = rope_mode; a.eps = eps; a.inv_n = 1.0f / (float)N;
  a.in_sb = in_stride_batch; a.in_ss = in_stride_seq;
  a.out_sb = out_strides->batch; a.out_ss = out_strides->seq; a.out_sh = out_strides->head;
  dim3 grid(S, B), block(256);
  hipStream_t st = (hipStream_t)stream;
  const bool two = N / 16 > 256;
  if (x_is_f32) {
    if (two) MDATTN_LAUNCH((norm_rope_rows_kernel<2, true>), grid, block, 0, st, a);
    else MDATTN_LAUNCH((norm_rope_rows_kernel<1, true>), grid, block, 0, st, a);
  } else {
    if (two) MDATTN_LAUNCH((norm_rope_rows_kernel<2, false>), grid, block, 0, st, a);
    else MDATTN_LAUNCH((norm_rope_rows_kernel<1, false>), grid, block, 0, st, a);
  }
  return launch_status();
}

