// Backward of the fused q/k RMSNorm + RoPE prologue for gfx950.  HBM-bound: per element the saved input and the
// upstream gradient are read once (16-byte loads) and the input gradient is written once.
//
//   forward   u = x (+ bias);  r = rsqrt(mean(u^2) + eps);  y = u r w;  out = q_mul * R(y)   (R: rotation of pairs)
//   backward  dy = q_mul * R^T g;  du = r (w dy) - u r^3 mean(u w dy);  dw = sum over tokens of dy u r
//
// The row statistics are recomputed from the saved input (nothing but the input is kept from the forward), in the
// same pass that rotates the gradient back: one workgroup walks a strided set of token rows, holds a row's input and
// gradient in registers, forms both row sums (u^2 and u w dy) with one barrier, then writes du.  The weight
// gradients are reduced without atomics in two stages: every workgroup accumulates its tokens' contributions to
// its lanes' columns in registers and writes one partial row to the workspace; a second kernel sums the partial rows
// in a fixed order, so results are bit-reproducible.
#include "mdattn_common.h"

namespace mdattn {

constexpr int kBwdMaxBlocks = 1024;  // partial rows of the weight-gradient reduction (4 workgroups per CU)

__device__ __forceinline__ float rsqrt_newton(float x) {
  const float y = __builtin_amdgcn_rsqf(x);
  return y * (1.5f - 0.5f * x * y * y);
}

// ------------------------------------------------------------------------------------------------ full row (Wan)
struct NormRopeBwdFullArgs {
  const uint4* x_in[2];   // saved inputs q, k (k may be null)
  const __bf16* g[2];     // upstream gradients, [B,S,H,D] by (g_sb, g_ss, g_sh)
  uint4* dx[2];           // input gradients, laid out like the inputs but with their own strides
  const uint4* w[2];
  const uint4* bias[2];   // BIAS: the projection biases the forward added (null: none)
  const float4* cos;
  const float4* sin;
  float* part;            // [nb][ncols] partial weight (and bias) gradients
  int S, H, D, N, ntok, nb, ncols;
  float eps, inv_n, q_mul;
  int64_t in_sb, in_ss, dx_sb, dx_ss, g_sb, g_ss, g_sh;
};

// One workgroup (256 lanes) per token row at a time, blockIdx.y = tensor (q, k); lane t owns the 16-byte chunks
// t, t+256, ... (<= MAXC) of every row it sees, so its weight-gradient accumulators are per-lane registers.
template <int MAXC, bool BIAS>
__global__ __launch_bounds__(256) void norm_rope_fullrow_bwd_kernel(NormRopeBwdFullArgs a) {
  const int tid = threadIdx.x, t = blockIdx.y;
  const int nchunks = a.N >> 3;
  __shared__ float red[2][2][16];
  const float mul = t == 0 ? a.q_mul : 1.0f;
  const bool rope = a.cos != nullptr;
  const int halfd4 = a.D >> 3;

  uint4 wraw[MAXC];
  int goff[MAXC], tofs[MAXC];
  float accw[MAXC][8];
  [[maybe_unused]] float accb[MAXC][8];
#pragma unroll
  for (int i = 0; i < MAXC; ++i) {
    const int c = tid + i * 256;
    const int cc = c < nchunks ? c : 0;
    const int e = cc << 3;
    const int h = e / a.D, d = e - h * a.D;
    wraw[i] = a.w[t][cc];
    goff[i] = (int)(h * a.g_sh) + d;
    tofs[i] = d >> 3;
#pragma unroll
    for (int j = 0; j < 8; ++j) { accw[i][j] = 0.f; if constexpr (BIAS) accb[i][j] = 0.f; }
  }

  int par = 0;
  for (int tok = blockIdx.x; tok < a.ntok; tok += a.nb, par ^= 1) {
    const int b = tok / a.S, s = tok - b * a.S;
    const uint4* xrow = a.x_in[t] + ((b * a.in_sb + s * a.in_ss) >> 3);
    const __bf16* grow = a.g[t] + b * a.g_sb + s * a.g_ss;
    uint4 xr[MAXC], gr[MAXC];
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
      const int c = tid + i * 256;
      if (c < nchunks) {
        xr[i] = ld_nt(xrow + c);
        gr[i] = ld_nt(reinterpret_cast<const uint4*>(grow + goff[i]));
      }
    }
    auto chunk_u = [&](int i, int c, float* u) __attribute__((always_inline)) {
      unpack8(xr[i], u);
      if constexpr (BIAS) {
        if (a.bias[t]) {
          float bb[8];
          unpack8(a.bias[t][c], bb);
#pragma unroll
          for (int j = 0; j < 8; ++j) u[j] += bb[j];
        }
      }
    };
    float dy[MAXC][8];
    float ss = 0.f, sd = 0.f;
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
      const int c = tid + i * 256;
      if (c < nchunks) {
        float u[8], gf[8], w[8];
        chunk_u(i, c, u);
        unpack8(gr[i], gf);
        unpack8(wraw[i], w);
        if (rope) {  // transposed rotation: dy0 = g0 c + g1 s, dy1 = g1 c - g0 s
          const float4 cs = a.cos[(int64_t)s * halfd4 + tofs[i]], sn = a.sin[(int64_t)s * halfd4 + tofs[i]];
          const float cc[4] = {cs.x, cs.y, cs.z, cs.w}, sv[4] = {sn.x, sn.y, sn.z, sn.w};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            dy[i][2 * j] = (gf[2 * j] * cc[j] + gf[2 * j + 1] * sv[j]) * mul;
            dy[i][2 * j + 1] = (gf[2 * j + 1] * cc[j] - gf[2 * j] * sv[j]) * mul;
          }
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j) dy[i][j] = gf[j] * mul;
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          ss = __builtin_fmaf(u[j], u[j], ss);
          sd = __builtin_fmaf(u[j], w[j] * dy[i][j], sd);
        }
      }
    }
    ss = row16_sum(ss);
    sd = row16_sum(sd);
    if ((tid & 15) == 0) { red[par][0][tid >> 4] = ss; red[par][1][tid >> 4] = sd; }
    // one barrier per row: the next row writes the other half of `red`, and the row after that comes after the next
    // barrier, which no lane passes before every lane has read this half
    __syncthreads();
    float tss = 0.f, tsd = 0.f;
#pragma unroll
    for (int j = 0; j < 16; ++j) { tss += red[par][0][j]; tsd += red[par][1][j]; }
    const float r = rsqrt_newton(tss * a.inv_n + a.eps);
    const float coef = r * r * r * tsd * a.inv_n;
    uint4* drow = a.dx[t] + ((b * a.dx_sb + s * a.dx_ss) >> 3);
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
      const int c = tid + i * 256;
      if (c < nchunks) {
        float u[8], w[8], du[8];
        chunk_u(i, c, u);
        unpack8(wraw[i], w);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          du[j] = r * w[j] * dy[i][j] - coef * u[j];
          accw[i][j] = __builtin_fmaf(dy[i][j] * r, u[j], accw[i][j]);
          if constexpr (BIAS) accb[i][j] += du[j];
        }
        st_nt(drow + c, pack8(du));
      }
    }
  }

  // partial row of this workgroup: [tensor][dw | db][N]
  float* prow = a.part + (int64_t)blockIdx.x * a.ncols + (int64_t)t * (BIAS ? 2 : 1) * a.N;
#pragma unroll
  for (int i = 0; i < MAXC; ++i) {
    const int c = tid + i * 256;
    if (c < nchunks) {
      float4* p = reinterpret_cast<float4*>(prow + c * 8);
      p[0] = make_float4(accw[i][0], accw[i][1], accw[i][2], accw[i][3]);
      p[1] = make_float4(accw[i][4], accw[i][5], accw[i][6], accw[i][7]);
      if constexpr (BIAS) {
        float4* pb = reinterpret_cast<float4*>(prow + a.N + c * 8);
        pb[0] = make_float4(accb[i][0], accb[i][1], accb[i][2], accb[i][3]);
        pb[1] = make_float4(accb[i][4], accb[i][5], accb[i][6], accb[i][7]);
      }
    }
  }
}

// Second stage: out[col] = sum over the nb partial rows, in a fixed order.  A workgroup covers 64 columns (16 lanes x
// float4) with 16 row slices; the slices are combined through LDS.  Column col goes to outs[col / seglen][col % seglen].
struct ColsumArgs {
  const float* part;
  float* outs[4];
  int nb, ncols, seglen;
};

__global__ __launch_bounds__(256) void colsum_kernel(ColsumArgs a) {
  const int tid = threadIdx.x, lane16 = tid & 15, slice = tid >> 4;
  const int col = blockIdx.x * 64 + lane16 * 4;
  __shared__ float4 sm[16][16];
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  if (col < a.ncols) {
    for (int r = slice; r < a.nb; r += 16) {
      const float4 v = *reinterpret_cast<const float4*>(a.part + (int64_t)r * a.ncols + col);
      acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
    }
  }
  sm[slice][lane16] = acc;
  __syncthreads();
  if (slice == 0 && col < a.ncols) {
    float4 tot = sm[0][lane16];
#pragma unroll
    for (int s = 1; s < 16; ++s) {
      const float4 v = sm[s][lane16];
      tot.x += v.x; tot.y += v.y; tot.z += v.z; tot.w += v.w;
    }
    const int seg = col / a.seglen, i = col - seg * a.seglen;  // seglen % 4 == 0: a float4 never straddles segments
    if (a.outs[seg]) *reinterpret_cast<float4*>(a.outs[seg] + i) = tot;
  }
}

// ------------------------------------------------------------------------------------------------ per head (Flux)
struct NormRopeBwdHeadArgs {
  const uint4* x_in[2];
  const uint4* g[2];
  uint4* dx[2];
  const uint4* w[2];
  const uint4* w_txt[2];
  const float4* cos;
  const float4* sin;
  float* part;  // [nb][4*D]: [tensor][image | text][D]
  int S, H, n_txt, nb;
  int64_t rows;  // B*S*H
  float eps, q_mul;
  int64_t in_sb, in_ss, in_sh, dx_sb, dx_ss, dx_sh, g_sb, g_ss, g_sh;
};

// LPR = D/8 lanes per (token, head) row, one 16-byte chunk per lane; a workgroup's 256/LPR lane groups walk the rows
// in strides.  Both row sums stay inside the lane group (no LDS, no barrier in the loop).
template <int LPR>
__global__ __launch_bounds__(256) void norm_rope_perhead_bwd_kernel(NormRopeBwdHeadArgs a) {
  constexpr int D = LPR * 8;
  constexpr int GROUPS = 256 / LPR;
  const int tid = threadIdx.x, lane = tid % LPR, grp = tid / LPR;
  const int ntens = a.x_in[1] ? 2 : 1;
  const bool rope = a.cos != nullptr;
  extern __shared__ __attribute__((aligned(16))) float sm_head[];  // [GROUPS][4*D]

  float acc[2][2][8];
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int k = 0; k < 2; ++k)
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[t][k][j] = 0.f;

  auto group_sum = [&](float v) __attribute__((always_inline)) {
    if (LPR >= 16) {
      v = row16_sum(v);
      if (LPR == 32) v += __shfl_xor(v, 16);
    } else {
      v += __shfl_xor(v, 1); v += __shfl_xor(v, 2); v += __shfl_xor(v, 4);
    }
    return v;
  };

  for (int64_t row = (int64_t)blockIdx.x * GROUPS + grp; row < a.rows; row += (int64_t)a.nb * GROUPS) {
    const int h = (int)(row % a.H);
    const int64_t bs = row / a.H;
    const int s = (int)(bs % a.S);
    const int64_t b = bs / a.S;
    const int64_t iofs = b * a.in_sb + s * a.in_ss + h * a.in_sh;
    const int64_t gofs = b * a.g_sb + s * a.g_ss + h * a.g_sh;
    const int64_t dofs = b * a.dx_sb + s * a.dx_ss + h * a.dx_sh;
    uint4 xr[2], gr[2];
#pragma unroll
    for (int t = 0; t < 2; ++t)
      if (t < ntens) {
        xr[t] = ld_nt(a.x_in[t] + (iofs >> 3) + lane);
        gr[t] = ld_nt(a.g[t] + (gofs >> 3) + lane);
      }
    float4 cs = {1.f, 1.f, 1.f, 1.f}, sn = {0.f, 0.f, 0.f, 0.f};
    if (rope) {
      cs = a.cos[(int64_t)s * LPR + lane];
      sn = a.sin[(int64_t)s * LPR + lane];
    }
    const float cc[4] = {cs.x, cs.y, cs.z, cs.w}, sv[4] = {sn.x, sn.y, sn.z, sn.w};
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      if (t < ntens) {
        const bool txt = a.w_txt[t] && s < a.n_txt;
        float u[8], gf[8], w[8], dy[8], du[8];
        unpack8(xr[t], u);
        unpack8(gr[t], gf);
        unpack8((txt ? a.w_txt[t] : a.w[t])[lane], w);
        const float mul = t == 0 ? a.q_mul : 1.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          dy[2 * j] = (gf[2 * j] * cc[j] + gf[2 * j + 1] * sv[j]) * mul;
          dy[2 * j + 1] = (gf[2 * j + 1] * cc[j] - gf[2 * j] * sv[j]) * mul;
        }
        float ss = 0.f, sd = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          ss = __builtin_fmaf(u[j], u[j], ss);
          sd = __builtin_fmaf(u[j], w[j] * dy[j], sd);
        }
        ss = group_sum(ss);
        sd = group_sum(sd);
        const float r = rsqrt_newton(ss * (1.0f / D) + a.eps);
        const float coef = r * r * r * sd * (1.0f / D);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          du[j] = r * w[j] * dy[j] - coef * u[j];
          const float dwj = dy[j] * r * u[j];
          acc[t][0][j] += txt ? 0.f : dwj;
          acc[t][1][j] += txt ? dwj : 0.f;
        }
        st_nt(a.dx[t] + (dofs >> 3) + lane, pack8(du));
      }
    }
  }

  // the workgroup's lane groups -> one partial row
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int k = 0; k < 2; ++k)
#pragma unroll
      for (int j = 0; j < 8; ++j) sm_head[grp * (4 * D) + (t * 2 + k) * D + lane * 8 + j] = acc[t][k][j];
  __syncthreads();
  for (int col = tid; col < 4 * D; col += 256) {
    float tot = 0.f;
#pragma unroll
    for (int gidx = 0; gidx < GROUPS; ++gidx) tot += sm_head[gidx * (4 * D) + col];
    a.part[(int64_t)blockIdx.x * (4 * D) + col] = tot;
  }
}

// ------------------------------------------------------------------------------------------------ rows (LTX-2)
struct NormRopeBwdRowsArgs {
  const void* x_in;
  const __bf16* g;   // [B,S,H,D] by (g_sb, g_ss, g_sh)
  void* dx;          // like x_in (bf16 or f32), strides dx_sb, dx_ss
  const float* w;
  const float* cos;
  const float* sin;
  float* part;       // [nb][N]
  int S, H, D, N, mode, ntok, nb;
  float eps, inv_n;
  int64_t in_sb, in_ss, dx_sb, dx_ss, g_sb, g_ss, g_sh;
};

// A lane works on "units" of two 8-element chunks of one head, c and c + D/16 (both partners of either pairing), as
// the forward kernel does.
template <int MAXU, bool F32IN>
__global__ __launch_bounds__(256) void norm_rope_rows_bwd_kernel(NormRopeBwdRowsArgs a) {
  const int tid = threadIdx.x;
  const int cph = a.D >> 4;
  const int nunits = a.H * cph;
  const int half = a.D >> 1;
  __shared__ float red[2][2][16];

  float accw[MAXU][16];
  int xoff[MAXU], goff[MAXU], hh[MAXU], cc8[MAXU];
#pragma unroll
  for (int i = 0; i < MAXU; ++i) {
    const int u = tid + i * 256;
    const int uu = u < nunits ? u : 0;
    const int h = uu / cph, c = uu - h * cph;
    hh[i] = h; cc8[i] = c * 8;
    xoff[i] = h * a.D + c * 8;
    goff[i] = (int)(h * a.g_sh) + c * 8;
#pragma unroll
    for (int j = 0; j < 16; ++j) accw[i][j] = 0.f;
  }

  int par = 0;
  for (int tok = blockIdx.x; tok < a.ntok; tok += a.nb, par ^= 1) {
    const int b = tok / a.S, s = tok - b * a.S;
    float x[MAXU][16], dy[MAXU][16];
    float ss = 0.f, sd = 0.f;
#pragma unroll
    for (int i = 0; i < MAXU; ++i) {
      const int u = tid + i * 256;
      if (u < nunits) {
        const int64_t e0 = b * a.in_sb + s * a.in_ss + xoff[i];
        if (F32IN) {
          const float4* p0 = reinterpret_cast<const float4*>(static_cast<const float*>(a.x_in) + e0);
          const float4* p1 = reinterpret_cast<const float4*>(static_cast<const float*>(a.x_in) + e0 + half);
          const float4 v0 = ld_nt(p0), v1 = ld_nt(p0 + 1), v2 = ld_nt(p1), v3 = ld_nt(p1 + 1);
          const float tt[16] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w, v2.x, v2.y, v2.z, v2.w, v3.x, v3.y, v3.z, v3.w};
#pragma unroll
          for (int j = 0; j < 16; ++j) x[i][j] = tt[j];
        } else {
          const uint4* p = reinterpret_cast<const uint4*>(static_cast<const __bf16*>(a.x_in) + e0);
          unpack8(ld_nt(p), x[i]);
          unpack8(ld_nt(p + (a.D >> 4)), x[i] + 8);
        }
        float gf[16];
        const uint4* gp = reinterpret_cast<const uint4*>(a.g + b * a.g_sb + s * a.g_ss + goff[i]);
        unpack8(ld_nt(gp), gf);
        unpack8(ld_nt(gp + (a.D >> 4)), gf + 8);
        if (a.mode == 1) {
          // out[2j] = y[2j] c[2j] - y[2j+1] s[2j];  out[2j+1] = y[2j+1] c[2j+1] + y[2j] s[2j+1]
          const int64_t t0 = ((int64_t)b * a.S + s) * a.N + xoff[i];
#pragma unroll
          for (int part = 0; part < 2; ++part) {
            const float4* cp = reinterpret_cast<const float4*>(a.cos + t0 + part * half);
            const float4* sp = reinterpret_cast<const float4*>(a.sin + t0 + part * half);
            const float4 c0 = cp[0], c1 = cp[1], s0 = sp[0], s1 = sp[1];
            const float cc[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
            const float sv[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const float g0 = gf[part * 8 + 2 * j], g1 = gf[part * 8 + 2 * j + 1];
              dy[i][part * 8 + 2 * j] = g0 * cc[2 * j] + g1 * sv[2 * j + 1];
              dy[i][part * 8 + 2 * j + 1] = g1 * cc[2 * j + 1] - g0 * sv[2 * j];
            }
          }
        } else if (a.mode == 2) {
          const int64_t t0 = (((int64_t)b * a.H + hh[i]) * a.S + s) * half + cc8[i];
          const float4* cp = reinterpret_cast<const float4*>(a.cos + t0);
          const float4* sp = reinterpret_cast<const float4*>(a.sin + t0);
          const float4 c0 = cp[0], c1 = cp[1], s0 = sp[0], s1 = sp[1];
          const float cc[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
          const float sv[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            dy[i][j] = gf[j] * cc[j] + gf[8 + j] * sv[j];
            dy[i][8 + j] = gf[8 + j] * cc[j] - gf[j] * sv[j];
          }
        } else {
#pragma unroll
          for (int j = 0; j < 16; ++j) dy[i][j] = gf[j];
        }
        const float4* wp0 = reinterpret_cast<const float4*>(a.w + xoff[i]);
        const float4* wp1 = reinterpret_cast<const float4*>(a.w + xoff[i] + half);
        const float4 w0 = wp0[0], w1 = wp0[1], w2 = wp1[0], w3 = wp1[1];
        const float w[16] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w, w2.x, w2.y, w2.z, w2.w, w3.x, w3.y, w3.z, w3.w};
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          ss = __builtin_fmaf(x[i][j], x[i][j], ss);
          sd = __builtin_fmaf(x[i][j], w[j] * dy[i][j], sd);
        }
      }
    }
    ss = row16_sum(ss);
    sd = row16_sum(sd);
    if ((tid & 15) == 0) { red[par][0][tid >> 4] = ss; red[par][1][tid >> 4] = sd; }
    __syncthreads();  // one barrier per row: `red` alternates between two halves (see the full-row kernel)
    float tss = 0.f, tsd = 0.f;
#pragma unroll
    for (int j = 0; j < 16; ++j) { tss += red[par][0][j]; tsd += red[par][1][j]; }
    const float r = rsqrt_newton(tss * a.inv_n + a.eps);
    const float coef = r * r * r * tsd * a.inv_n;
#pragma unroll
    for (int i = 0; i < MAXU; ++i) {
      const int u = tid + i * 256;
      if (u < nunits) {
        const float4* wp0 = reinterpret_cast<const float4*>(a.w + xoff[i]);
        const float4* wp1 = reinterpret_cast<const float4*>(a.w + xoff[i] + half);
        const float4 w0 = wp0[0], w1 = wp0[1], w2 = wp1[0], w3 = wp1[1];
        const float w[16] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w, w2.x, w2.y, w2.z, w2.w, w3.x, w3.y, w3.z, w3.w};
        float du[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          du[j] = r * w[j] * dy[i][j] - coef * x[i][j];
          accw[i][j] = __builtin_fmaf(dy[i][j] * r, x[i][j], accw[i][j]);
        }
        const int64_t e0 = b * a.dx_sb + s * a.dx_ss + xoff[i];
        if (F32IN) {
          float4* p0 = reinterpret_cast<float4*>(static_cast<float*>(a.dx) + e0);
          float4* p1 = reinterpret_cast<float4*>(static_cast<float*>(a.dx) + e0 + half);
          p0[0] = make_float4(du[0], du[1], du[2], du[3]);
          p0[1] = make_float4(du[4], du[5], du[6], du[7]);
          p1[0] = make_float4(du[8], du[9], du[10], du[11]);
          p1[1] = make_float4(du[12], du[13], du[14], du[15]);
        } else {
          uint4* p = reinterpret_cast<uint4*>(static_cast<__bf16*>(a.dx) + e0);
          st_nt(p, pack8(du));
          st_nt(p + (a.D >> 4), pack8(du + 8));
        }
      }
    }
  }

  float* prow = a.part + (int64_t)blockIdx.x * a.N;
#pragma unroll
  for (int i = 0; i < MAXU; ++i) {
    const int u = tid + i * 256;
    if (u < nunits) {
      float4* p0 = reinterpret_cast<float4*>(prow + xoff[i]);
      float4* p1 = reinterpret_cast<float4*>(prow + xoff[i] + half);
      p0[0] = make_float4(accw[i][0], accw[i][1], accw[i][2], accw[i][3]);
      p0[1] = make_float4(accw[i][4], accw[i][5], accw[i][6], accw[i][7]);
      p1[0] = make_float4(accw[i][8], accw[i][9], accw[i][10], accw[i][11]);
      p1[1] = make_float4(accw[i][12], accw[i][13], accw[i][14], accw[i][15]);
    }
  }
}

static int launch_colsum(hipStream_t st, const float* part, int nb, int ncols, int seglen, float* o0, float* o1, float* o2, float* o3) {
  ColsumArgs c;
  c.part = part; c.nb = nb; c.ncols = ncols; c.seglen = seglen;
  c.outs[0] = o0; c.outs[1] = o1; c.outs[2] = o2; c.outs[3] = o3;
  hipLaunchKernelGGL(colsum_kernel, dim3((ncols + 63) / 64), dim3(256), 0, st, c);
  return launch_status();
}

}  // namespace mdattn

using namespace mdattn;

extern "C" int64_t mdattn_norm_rope_bwd_workspace_floats(int64_t rows, int64_t columns) {
  if (rows <= 0 || columns <= 0) return 0;
  return (rows < kBwdMaxBlocks ? rows : kBwdMaxBlocks) * columns;
}

// number of partial rows a workspace of `floats` allows for `units` independent row units and `ncols` columns
static int partial_rows(int64_t units, int64_t ncols, int64_t floats) {
  int64_t nb = units < kBwdMaxBlocks ? units : kBwdMaxBlocks;
  if (floats / ncols < nb) nb = floats / ncols;
  return (int)nb;
}

extern "C" int mdattn_norm_rope_fullrow_bwd(void* stream, const void* q_in, const void* k_in, const void* bias,
                                            const void* gq, const void* gk, void* dq_in, void* dk_in,
                                            const void* wq, const void* wk, float* dwq, float* dwk, float* dbias,
                                            const float* cos, const float* sin, int B, int S, int H, int D, float eps, float q_mul,
                                            int64_t in_stride_batch, int64_t in_stride_seq,
                                            int64_t dx_stride_batch, int64_t dx_stride_seq, const mdattn_strides* g_strides,
                                            float* workspace, int64_t workspace_floats) {
  if (!q_in || !gq || !dq_in || !wq || !dwq || B <= 0 || S <= 0 || H <= 0 || D <= 0 || !g_strides || !workspace) return MDATTN_E_BADARG;
  const bool has_k = k_in != nullptr;
  if (has_k != (gk != nullptr) || has_k != (dk_in != nullptr) || has_k != (dwk != nullptr) || (has_k && !wk)) return MDATTN_E_BADARG;
  if ((cos == nullptr) != (sin == nullptr)) return MDATTN_E_BADARG;
  if ((bias == nullptr) != (dbias == nullptr) || (bias && !has_k)) return MDATTN_E_BADARG;  // the fused q|k|v form carries both
  if (!(eps >= 0.f) || !(q_mul > 0.f) || !(q_mul < 1e30f)) return MDATTN_E_BADARG;
  const int64_t N = (int64_t)H * D;
  if (D % 8 != 0 || N > 8192) return MDATTN_E_UNSUPPORTED;
  const int64_t ntok = (int64_t)B * S;
  if (ntok > 0x7FFFFFFF) return MDATTN_E_UNSUPPORTED;
  if (in_stride_seq < N || in_stride_batch < 0 || dx_stride_seq < N || dx_stride_batch < 0) return MDATTN_E_BADARG;
  if ((int64_t)(H - 1) * g_strides->head + D >= (int64_t)1 << 31) return MDATTN_E_UNSUPPORTED;  // per-lane offsets inside a gradient row are 32-bit
  if (!aligned16(q_in) || !aligned16(k_in) || !aligned16(bias) || !aligned16(gq) || !aligned16(gk) || !aligned16(dq_in) ||
      !aligned16(dk_in) || !aligned16(wq) || !aligned16(wk) || !aligned16(dwq) || !aligned16(dwk) || !aligned16(dbias) ||
      !aligned16(cos) || !aligned16(sin) || !aligned16(workspace))
    return MDATTN_E_ALIGN;
  if (in_stride_batch % 8 || in_stride_seq % 8 || dx_stride_batch % 8 || dx_stride_seq % 8 || !strides_ok(g_strides, 8)) return MDATTN_E_ALIGN;
  const int ntens = has_k ? 2 : 1;
  const int64_t ncols = (int64_t)ntens * (bias ? 2 : 1) * N;
  const int nb = partial_rows(ntok, ncols, workspace_floats);
  if (nb < 1) return MDATTN_E_BADARG;

  NormRopeBwdFullArgs a;
  a.x_in[0] = (const uint4*)q_in; a.x_in[1] = (const uint4*)k_in;
  a.g[0] = (const __bf16*)gq; a.g[1] = (const __bf16*)gk;
  a.dx[0] = (uint4*)dq_in; a.dx[1] = (uint4*)dk_in;
  a.w[0] = (const uint4*)wq; a.w[1] = (const uint4*)wk;
  const uint4* bb = (const uint4*)bias;
  a.bias[0] = bb; a.bias[1] = bb ? bb + N / 8 : nullptr;
  a.cos = (const float4*)cos; a.sin = (const float4*)sin;
  a.part = workspace;
  a.S = S; a.H = H; a.D = D; a.N = (int)N; a.ntok = (int)ntok; a.nb = nb; a.ncols = (int)ncols;
  a.eps = eps; a.inv_n = 1.0f / (float)N; a.q_mul = q_mul;
  a.in_sb = in_stride_batch; a.in_ss = in_stride_seq; a.dx_sb = dx_stride_batch; a.dx_ss = dx_stride_seq;
  a.g_sb = g_strides->batch; a.g_ss = g_strides->seq; a.g_sh = g_strides->head;
  dim3 grid(nb, ntens), block(256);
  hipStream_t st = (hipStream_t)stream;
  const int nchunks = (int)(N / 8);
#define MDATTN_LAUNCH_FULL_BWD(MAXC)                                                                             \
  do {                                                                                                           \
    if (bias) hipLaunchKernelGGL((norm_rope_fullrow_bwd_kernel<MAXC, true>), grid, block, 0, st, a);             \
    else hipLaunchKernelGGL((norm_rope_fullrow_bwd_kernel<MAXC, false>), grid, block, 0, st, a);                 \
  } while (0)
  if (nchunks <= 256) MDATTN_LAUNCH_FULL_BWD(1);
  else if (nchunks <= 512) MDATTN_LAUNCH_FULL_BWD(2);
  else if (nchunks <= 768) MDATTN_LAUNCH_FULL_BWD(3);
  else MDATTN_LAUNCH_FULL_BWD(4);
#undef MDATTN_LAUNCH_FULL_BWD
  int rc = launch_status();
  if (rc != MDATTN_OK) return rc;
  // columns: [q: dw (, db)] [k: dw (, db)], each N wide
  if (bias) return launch_colsum(st, workspace, nb, (int)ncols, (int)N, dwq, dbias, dwk, dbias + N);
  return launch_colsum(st, workspace, nb, (int)ncols, (int)N, dwq, dwk, nullptr, nullptr);
}

extern "C" int mdattn_norm_rope_perhead_bwd(void* stream, const void* q_in, const void* k_in, const void* gq, const void* gk,
                                            void* dq_in, void* dk_in, const void* wq, const void* wk, const void* wq_txt,
                                            const void* wk_txt, int n_txt, float* dwq, float* dwk, float* dwq_txt, float* dwk_txt,
                                            const float* cos, const float* sin, int B, int S, int H, int D, float eps, float q_mul,
                                            const mdattn_strides* in_strides, const mdattn_strides* dx_strides,
                                            const mdattn_strides* g_strides, float* workspace, int64_t workspace_floats) {
  if (!q_in || !gq || !dq_in || !wq || !dwq || B <= 0 || S <= 0 || H <= 0 || D <= 0 || !in_strides || !dx_strides || !g_strides || !workspace)
    return MDATTN_E_BADARG;
  const bool has_k = k_in != nullptr;
  if (has_k != (gk != nullptr) || has_k != (dk_in != nullptr) || has_k != (dwk != nullptr) || (has_k && !wk)) return MDATTN_E_BADARG;
  if ((cos == nullptr) != (sin == nullptr)) return MDATTN_E_BADARG;
  if ((wq_txt == nullptr) != (dwq_txt == nullptr) || (wk_txt == nullptr) != (dwk_txt == nullptr)) return MDATTN_E_BADARG;
  if (n_txt < 0 || n_txt > S || !(eps >= 0.f) || !(q_mul > 0.f) || !(q_mul < 1e30f)) return MDATTN_E_BADARG;
  if (D != 64 && D != 128 && D != 256) return MDATTN_E_UNSUPPORTED;
  if (!aligned16(q_in) || !aligned16(k_in) || !aligned16(gq) || !aligned16(gk) || !aligned16(dq_in) || !aligned16(dk_in) ||
      !aligned16(wq) || !aligned16(wk) || !aligned16(wq_txt) || !aligned16(wk_txt) || !aligned16(dwq) || !aligned16(dwk) ||
      !aligned16(dwq_txt) || !aligned16(dwk_txt) || !aligned16(cos) || !aligned16(sin) || !aligned16(workspace))
    return MDATTN_E_ALIGN;
  if (!strides_ok(in_strides, 8) || !strides_ok(dx_strides, 8) || !strides_ok(g_strides, 8)) return MDATTN_E_ALIGN;
  const int lpr = D / 8, groups = 256 / lpr;
  const int64_t rows = (int64_t)B * S * H;
  const int64_t ncols = 4 * (int64_t)D;
  const int nb = partial_rows((rows + groups - 1) / groups, ncols, workspace_floats);
  if (nb < 1) return MDATTN_E_BADARG;

  NormRopeBwdHeadArgs a;
  a.x_in[0] = (const uint4*)q_in; a.x_in[1] = (const uint4*)k_in;
  a.g[0] = (const uint4*)gq; a.g[1] = (const uint4*)gk;
  a.dx[0] = (uint4*)dq_in; a.dx[1] = (uint4*)dk_in;
  a.w[0] = (const uint4*)wq; a.w[1] = (const uint4*)wk;
  a.w_txt[0] = (const uint4*)wq_txt; a.w_txt[1] = has_k ? (const uint4*)wk_txt : nullptr;
  a.cos = (const float4*)cos; a.sin = (const float4*)sin;
  a.part = workspace;
  a.S = S; a.H = H; a.n_txt = n_txt; a.nb = nb; a.rows = rows; a.eps = eps; a.q_mul = q_mul;
  a.in_sb = in_strides->batch; a.in_ss = in_strides->seq; a.in_sh = in_strides->head;
  a.dx_sb = dx_strides->batch; a.dx_ss = dx_strides->seq; a.dx_sh = dx_strides->head;
  a.g_sb = g_strides->batch; a.g_ss = g_strides->seq; a.g_sh = g_strides->head;
  dim3 grid(nb), block(256);
  hipStream_t st = (hipStream_t)stream;
  const int lds = groups * 4 * D * (int)sizeof(float);  // 32 KB for every supported D
  if (lpr == 8) hipLaunchKernelGGL((norm_rope_perhead_bwd_kernel<8>), grid, block, lds, st, a);
  else if (lpr == 16) hipLaunchKernelGGL((norm_rope_perhead_bwd_kernel<16>), grid, block, lds, st, a);
  else hipLaunchKernelGGL((norm_rope_perhead_bwd_kernel<32>), grid, block, lds, st, a);
  int rc = launch_status();
  if (rc != MDATTN_OK) return rc;
  // columns: [q image][q text][k image][k text], each D wide; outputs that do not exist are skipped
  return launch_colsum(st, workspace, nb, (int)ncols, D, dwq, dwq_txt, dwk, has_k ? dwk_txt : nullptr);
}

extern "C" int mdattn_norm_rope_rows_bwd(void* stream, const void* x_in, int x_is_f32, const void* g, void* dx, const float* w,
                                         float* dw, const float* cos, const float* sin, int rope_mode, int B, int S, int H, int D,
                                         float eps, int64_t in_stride_batch, int64_t in_stride_seq,
                                         int64_t dx_stride_batch, int64_t dx_stride_seq, const mdattn_strides* g_strides,
                                         float* workspace, int64_t workspace_floats) {
  if (!x_in || !g || !dx || !w || !dw || B <= 0 || S <= 0 || H <= 0 || D <= 0 || !g_strides || !workspace) return MDATTN_E_BADARG;
  if (rope_mode < 0 || rope_mode > 2 || (rope_mode != 0 && (!cos || !sin)) || !(eps >= 0.f)) return MDATTN_E_BADARG;
  if (D % 16 != 0) return MDATTN_E_UNSUPPORTED;
  const int64_t N = (int64_t)H * D;
  if (N / 16 > 2 * 256) return MDATTN_E_UNSUPPORTED;
  const int64_t ntok = (int64_t)B * S;
  if (ntok > 0x7FFFFFFF || (int64_t)(H - 1) * g_strides->head + D >= (int64_t)1 << 31) return MDATTN_E_UNSUPPORTED;
  const int in_mult = x_is_f32 ? 4 : 8;
  if (!aligned16(x_in) || !aligned16(g) || !aligned16(dx) || !aligned16(w) || !aligned16(dw) || !aligned16(cos) || !aligned16(sin) ||
      !aligned16(workspace))
    return MDATTN_E_ALIGN;
  if (in_stride_batch % in_mult || in_stride_seq % in_mult || in_stride_seq < N || dx_stride_batch % in_mult ||
      dx_stride_seq % in_mult || dx_stride_seq < N || !strides_ok(g_strides, 8))
    return MDATTN_E_ALIGN;
  if (g_strides->head < D) return MDATTN_E_BADARG;
  const int nb = partial_rows(ntok, N, workspace_floats);
  if (nb < 1) return MDATTN_E_BADARG;
  NormRopeBwdRowsArgs a;
  a.x_in = x_in; a.g = (const __bf16*)g; a.dx = dx; a.w = w; a.cos = cos; a.sin = sin; a.part = workspace;
  a.S = S; a.H = H; a.D = D; a.N = (int)N; a.mode = rope_mode; a.ntok = (int)ntok; a.nb = nb;
  a.eps = eps; a.inv_n = 1.0f / (float)N;
  a.in_sb = in_stride_batch; a.in_ss = in_stride_seq; a.dx_sb = dx_stride_batch; a.dx_ss = dx_stride_seq;
  a.g_sb = g_strides->batch; a.g_ss = g_strides->seq; a.g_sh = g_strides->head;
  dim3 grid(nb), block(256);
  hipStream_t st = (hipStream_t)stream;
  const bool two = N / 16 > 256;
  if (x_is_f32) {
    if (two) hipLaunchKernelGGL((norm_rope_rows_bwd_kernel<2, true>), grid, block, 0, st, a);
    else hipLaunchKernelGGL((norm_rope_rows_bwd_kernel<1, true>), grid, block, 0, st, a);
  } else {
    if (two) hipLaunchKernelGGL((norm_rope_rows_bwd_kernel<2, false>), grid, block, 0, st, a);
    else hipLaunchKernelGGL((norm_rope_rows_bwd_kernel<1, false>), grid, block, 0, st, a);
  }
  int rc = launch_status();
  if (rc != MDATTN_OK) return rc;
  return launch_colsum(st, workspace, nb, (int)N, (int)N, dw, nullptr, nullptr, nullptr);
}
