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

// One workgroup per token row at a time, blockIdx.y = tensor (q, k).  The workgroup has NT = blockDim.x lanes, chosen
// by the host so that the row's 16-byte chunks divide evenly among them (5120 channels: 640 chunks = 320 lanes x 2);
// lane t owns the chunks t, t+NT, ... (<= MAXC) of every row it sees, so its weight-gradient accumulators are per-lane
// registers.
// Vector ALU: the kernel is as much an ALU load as a memory stream (two passes over a row, three tensors to unpack),
// so the rotated gradient is kept as f32 between the passes, the weights are unpacked once per workgroup, and q_mul
// rides on the per-row scalars instead of on every element.
// Memory: three register buffers rotate (the loop is unrolled three times by hand): while one row is worked on, the
// raw rows of the next two tokens are in flight.  Vector-memory loads return in order, so whatever a row needs must
// have been requested before the rows that are still to fly: a row's slice of the rotary table travels in its buffer,
// and all loads are unconditional (indices clamped) so that the count of loads in flight is the same on every path.
// Registers: what bounds the kernel is the number of row bytes in flight per CU, i.e. how many workgroups fit next to
// their row buffers.  The unpacked weights and the weight-gradient accumulators (8 floats per chunk each) therefore
// live in LDS, each lane reading and writing only its own chunks (no synchronisation; LDS traffic returns on its own
// counter and does not queue behind the global loads): three workgroups of five waves per CU at 5120 channels.
// TAB1: every chunk of a lane uses the same table slice (NT a multiple of D/8, true for power-of-two head dims).
template <int MAXC, bool BIAS, bool TAB1>
__global__ __launch_bounds__(512) void norm_rope_fullrow_bwd_kernel(NormRopeBwdFullArgs a) {
  const int tid = threadIdx.x, t = blockIdx.y, NT = blockDim.x;
  const int wave = tid >> 6, nwaves = NT >> 6;
  const int nchunks = a.N >> 3;
  __shared__ float red[2][2][8];
  const float mul = t == 0 ? a.q_mul : 1.0f;
  const bool rope = a.cos != nullptr;
  const int halfd4 = a.D >> 3;
  constexpr int TC = TAB1 ? 1 : MAXC;

  // LDS: [MAXC * NT] chunks of 8 floats each for the weights, then the same for the weight-gradient accumulators;
  // chunk (i, tid) belongs to lane tid alone
  extern __shared__ __attribute__((aligned(16))) float lds_full[];
  float4* wl = reinterpret_cast<float4*>(lds_full);
  float4* al = wl + 2 * MAXC * NT;
  int goff[MAXC], coff[MAXC], tofs[TC];
  [[maybe_unused]] float accb[MAXC][8];
  [[maybe_unused]] float bf[MAXC][8];
#pragma unroll
  for (int i = 0; i < MAXC; ++i) {
    const int c = tid + i * NT;
    const int cc = c < nchunks ? c : nchunks - 1;  // lanes past the row's end shadow its last chunk and never store
    const int e = cc << 3;
    const int h = e / a.D, d = e - h * a.D;
    float w8[8];
    unpack8(a.w[t][cc], w8);
    wl[2 * (i * NT + tid)] = make_float4(w8[0], w8[1], w8[2], w8[3]);
    wl[2 * (i * NT + tid) + 1] = make_float4(w8[4], w8[5], w8[6], w8[7]);
    al[2 * (i * NT + tid)] = make_float4(0.f, 0.f, 0.f, 0.f);
    al[2 * (i * NT + tid) + 1] = make_float4(0.f, 0.f, 0.f, 0.f);
    coff[i] = cc;
    goff[i] = (int)(h * a.g_sh) + d;
    if (i < TC) tofs[i] = d >> 3;
#pragma unroll
    for (int j = 0; j < 8; ++j) { if constexpr (BIAS) { accb[i][j] = 0.f; bf[i][j] = 0.f; } }
    if constexpr (BIAS) {
      if (a.bias[t]) unpack8(a.bias[t][cc], bf[i]);
    }
  }
  auto lds8 = [&](const float4* base, int i, float* f) __attribute__((always_inline)) {
    const float4 v0 = base[2 * (i * NT + tid)], v1 = base[2 * (i * NT + tid) + 1];
    f[0] = v0.x; f[1] = v0.y; f[2] = v0.z; f[3] = v0.w; f[4] = v1.x; f[5] = v1.y; f[6] = v1.z; f[7] = v1.w;
  };
  const float4* cosp = rope ? a.cos : reinterpret_cast<const float4*>(a.w[t]);  // norm only: any readable address, unused
  const float4* sinp = rope ? a.sin : reinterpret_cast<const float4*>(a.w[t]);
  const int64_t tstride = rope ? halfd4 : 0;

  struct RowBuf {
    uint4 x[MAXC], g[MAXC];
    float4 cs[TC], sn[TC];
  };
  const int last = a.ntok - 1;
  auto load_row = [&](int tok, RowBuf& r) __attribute__((always_inline)) {
    tok = min(tok, last);
    const int b = tok / a.S, s = tok - b * a.S;
    const uint4* xrow = a.x_in[t] + ((b * a.in_sb + s * a.in_ss) >> 3);
    const __bf16* grow = a.g[t] + b * a.g_sb + s * a.g_ss;
    // (the empty asm statements keep the compiler from moving loads of one row across those of another: the order
    // of issue is what the waits depend on)
    asm volatile("" ::: "memory");
#pragma unroll
    for (int i = 0; i < TC; ++i) {
      r.cs[i] = cosp[(int64_t)s * tstride + (rope ? tofs[i] : 0)];
      r.sn[i] = sinp[(int64_t)s * tstride + (rope ? tofs[i] : 0)];
    }
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
      r.x[i] = ld_nt(xrow + coff[i]);
      r.g[i] = ld_nt(reinterpret_cast<const uint4*>(grow + goff[i]));
    }
    asm volatile("" ::: "memory");
  };

  int par = 0;
  // one row: consumes `r` (the row of token tok), then refills it with the row three steps ahead
  auto step = [&](int tok_, RowBuf& r) __attribute__((always_inline)) {
    // past the end (the last trip of the three-step loop): the buffer holds the clamped last row; it goes through the
    // same code with its stores and accumulation switched off, so that the loop has no exit in its middle
    const bool valid = tok_ < a.ntok;
    const int tok = min(tok_, last);
    const int b = tok / a.S, s = tok - b * a.S;
    // dy0 = R^T g (transposed rotation: dy0 = g0 c + g1 s, dy1 = g1 c - g0 s), without q_mul
    float dy[MAXC][8];
    float ss = 0.f, sd = 0.f;
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
      float u[8], gf[8];
      unpack8(r.x[i], u);
      unpack8(r.g[i], gf);
      if constexpr (BIAS) {
#pragma unroll
        for (int j = 0; j < 8; ++j) u[j] += bf[i][j];
      }
      if (rope) {
        const float4 cs = r.cs[TAB1 ? 0 : i], sn = r.sn[TAB1 ? 0 : i];
        const float cc[4] = {cs.x, cs.y, cs.z, cs.w}, sv[4] = {sn.x, sn.y, sn.z, sn.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          dy[i][2 * j] = __builtin_fmaf(gf[2 * j], cc[j], gf[2 * j + 1] * sv[j]);
          dy[i][2 * j + 1] = __builtin_fmaf(gf[2 * j + 1], cc[j], -(gf[2 * j] * sv[j]));
        }
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) dy[i][j] = gf[j];
      }
      if (tid + i * NT < nchunks) {
        float w8[8];
        lds8(wl, i, w8);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          ss = __builtin_fmaf(u[j], u[j], ss);
          sd = __builtin_fmaf(u[j], w8[j] * dy[i][j], sd);
        }
      }
    }
    ss = row16_sum(ss);
    sd = row16_sum(sd);
    ss += __shfl_xor(ss, 16); sd += __shfl_xor(sd, 16);
    ss = xhalf_sum(ss); sd = xhalf_sum(sd);
    if ((tid & 63) == 0) { red[par][0][wave] = ss; red[par][1][wave] = sd; }
    // one barrier per row: the next row writes the other half of `red`, and the row after that comes after the next
    // barrier, which no lane passes before every lane has read this half
    __syncthreads();
    float tss = 0.f, tsd = 0.f;
    for (int j = 0; j < nwaves; ++j) { tss += red[par][0][j]; tsd += red[par][1][j]; }
    par ^= 1;
    const float r_ = rsqrt_newton(tss * a.inv_n + a.eps);
    const float rm = r_ * mul;                         // q_mul folded into the row scalars
    const float coef = r_ * r_ * rm * tsd * a.inv_n;
    uint4* drow = a.dx[t] + ((b * a.dx_sb + s * a.dx_ss) >> 3);
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
      float u[8], du[8];
      unpack8(r.x[i], u);  // unpacked again rather than kept: eight registers per chunk for one instruction per element
      if constexpr (BIAS) {
#pragma unroll
        for (int j = 0; j < 8; ++j) u[j] += bf[i][j];
      }
      if (valid && tid + i * NT < nchunks) {
        float w8[8], acc[8];
        lds8(wl, i, w8);
        lds8(al, i, acc);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float dyr = dy[i][j] * rm;
          du[j] = __builtin_fmaf(-coef, u[j], w8[j] * dyr);
          acc[j] = __builtin_fmaf(dyr, u[j], acc[j]);
          if constexpr (BIAS) accb[i][j] += du[j];
        }
        al[2 * (i * NT + tid)] = make_float4(acc[0], acc[1], acc[2], acc[3]);
        al[2 * (i * NT + tid) + 1] = make_float4(acc[4], acc[5], acc[6], acc[7]);
        st_nt(drow + coff[i], pack8(du));
      }
    }
    load_row(tok_ + 3 * a.nb, r);
  };

  // the three initial requests in the order the loop keeps them in (oldest first): the waits inside the loop are
  // derived from the order of issue on every path into it
  RowBuf r0, r1, r2;
  load_row(blockIdx.x, r0);
  __builtin_amdgcn_sched_barrier(0);
  load_row(blockIdx.x + a.nb, r1);
  __builtin_amdgcn_sched_barrier(0);
  load_row(blockIdx.x + 2 * a.nb, r2);
  __builtin_amdgcn_sched_barrier(0);
  for (int tok = blockIdx.x; tok < a.ntok; tok += 3 * a.nb) {
    step(tok, r0);
    step(tok + a.nb, r1);
    step(tok + 2 * a.nb, r2);
  }

  // partial row of this workgroup: [tensor][dw | db][N]
  float* prow = a.part + (int64_t)blockIdx.x * a.ncols + (int64_t)t * (BIAS ? 2 : 1) * a.N;
#pragma unroll
  for (int i = 0; i < MAXC; ++i) {
    const int c = tid + i * NT;
    if (c < nchunks) {
      float4* p = reinterpret_cast<float4*>(prow + c * 8);
      p[0] = al[2 * (i * NT + tid)];
      p[1] = al[2 * (i * NT + tid) + 1];
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

// Workgroups of `kernel` (block size nt, dynamic LDS lds) that the current device holds at once.  The backward kernels
// are persistent loops over token rows: a grid of exactly that many workgroups (or fewer) runs as one even wave, where
// a fixed grid of 1024 would run as one full round plus a partly filled one.  Asked of the runtime once per kernel,
// block size and device.
struct ResidentCache {
  std::atomic<int> value[8][16];  // [block size / 64 - 1][device]
};
static int resident_blocks(ResidentCache& cache, const void* kernel, int nt, int lds) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0) return 0;
  const int slot = nt / 64 - 1;
  const bool cached = slot >= 0 && slot < 8 && dev < 16;
  if (cached) {
    const int v = cache.value[slot][dev].load(std::memory_order_acquire);
    if (v > 0) return v;
  }
  // registers and wave slots from the runtime (asked without LDS: its LDS rule assumes 64 KB per CU), LDS by hand:
  // a gfx950 CU has 160 KB
  int per_cu = 0, cus = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, nt, 0) != hipSuccess || per_cu < 1) return 0;
  if (lds > 0 && (160 * 1024 - 1024) / lds < per_cu) per_cu = (160 * 1024 - 1024) / lds;
  if (per_cu < 1) per_cu = 1;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1) return 0;
  const int v = per_cu * cus;
  if (cached) cache.value[slot][dev].store(v, std::memory_order_release);
  return v;
}

static int launch_colsum(hipStream_t st, const float* part, int nb, int ncols, int seglen, float* o0, float* o1, float* o2, float* o3) {
  ColsumArgs c;
  c.part = part; c.nb = nb; c.ncols = ncols; c.seglen = seglen;
  c.outs[0] = o0; c.outs[1] = o1; c.outs[2] = o2; c.outs[3] = o3;
  MDATTN_LAUNCH(colsum_kernel, dim3((ncols + 63) / 64), dim3(256), 0, st, c);
  return launch_status();
}

}  // namespace mdattn

using namespace mdattn;

extern "C" int64_t mdattn_norm_rope_bwd_workspace_floats(int64_t rows, int64_t columns) {
  if (rows <= 0 || columns <= 0) return 0;
  return (rows < kBwdMaxBlocks ? rows : kBwdMaxBlocks) * columns;
}

// number of partial rows a workspace of `floats` allows for `units` independent row units and `ncols` columns
static int partial_rows(int64_t units, int64_t ncols, int64_t floats, int resident = 0) {
  int64_t nb = units < kBwdMaxBlocks ? units : kBwdMaxBlocks;
  if (resident > 0 && resident < nb) nb = resident;  // one even wave of workgroups
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
  // lanes per workgroup: the row's chunks split evenly over whole waves, at most two chunks per lane up to 8192 channels
  const int nchunks = (int)(N / 8);
  const int maxc = (nchunks + 511) / 512;
  const int nt = ((nchunks + maxc - 1) / maxc + 63) / 64 * 64;
  const int lds_bytes = 2 * maxc * nt * 8 * (int)sizeof(float);  // unpacked weights + accumulators, <= 64 KB
  const bool tab1 = nt % (D / 8) == 0;  // every chunk of a lane then sits at the same offset inside its head
  void (*kern)(NormRopeBwdFullArgs);
  if (tab1) kern = maxc == 1 ? (bias ? norm_rope_fullrow_bwd_kernel<1, true, true> : norm_rope_fullrow_bwd_kernel<1, false, true>)
                             : (bias ? norm_rope_fullrow_bwd_kernel<2, true, true> : norm_rope_fullrow_bwd_kernel<2, false, true>);
  else kern = maxc == 1 ? (bias ? norm_rope_fullrow_bwd_kernel<1, true, false> : norm_rope_fullrow_bwd_kernel<1, false, false>)
                        : (bias ? norm_rope_fullrow_bwd_kernel<2, true, false> : norm_rope_fullrow_bwd_kernel<2, false, false>);
  static ResidentCache resident[2][2][2];
  const int nb = partial_rows(ntok, ncols, workspace_floats,
                              resident_blocks(resident[maxc - 1][bias ? 1 : 0][tab1 ? 1 : 0], reinterpret_cast<const void*>(kern), nt, lds_bytes) / ntens);
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
  hipStream_t st = (hipStream_t)stream;
  MDATTN_LAUNCH(kern, dim3(nb, ntens), dim3(nt), lds_bytes, st, a);
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
  const int lds = groups * 4 * D * (int)sizeof(float);  // 32 KB for every supported D
  void (*kern)(NormRopeBwdHeadArgs) = lpr == 8 ? norm_rope_perhead_bwd_kernel<8> : lpr == 16 ? norm_rope_perhead_bwd_kernel<16> : norm_rope_perhead_bwd_kernel<32>;
  static ResidentCache resident[3];
  const int nb = partial_rows((rows + groups - 1) / groups, ncols, workspace_floats,
                              resident_blocks(resident[lpr == 8 ? 0 : lpr == 16 ? 1 : 2], reinterpret_cast<const void*>(kern), 256, lds));
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
  hipStream_t st = (hipStream_t)stream;
  MDATTN_LAUNCH(kern, dim3(nb), dim3(256), lds, st, a);
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
  const bool two = N / 16 > 256;
  void (*kern)(NormRopeBwdRowsArgs) = x_is_f32 ? (two ? norm_rope_rows_bwd_kernel<2, true> : norm_rope_rows_bwd_kernel<1, true>)
                                               : (two ? norm_rope_rows_bwd_kernel<2, false> : norm_rope_rows_bwd_kernel<1, false>);
  static ResidentCache resident[2][2];
  const int nb = partial_rows(ntok, N, workspace_floats, resident_blocks(resident[x_is_f32 ? 1 : 0][two ? 1 : 0], reinterpret_cast<const void*>(kern), 256, 0));
  if (nb < 1) return MDATTN_E_BADARG;
  NormRopeBwdRowsArgs a;
  a.x_in = x_in; a.g = (const __bf16*)g; a.dx = dx; a.w = w; a.cos = cos; a.sin = sin; a.part = workspace;
  a.S = S; a.H = H; a.D = D; a.N = (int)N; a.mode = rope_mode; a.ntok = (int)ntok; a.nb = nb;
  a.eps = eps; a.inv_n = 1.0f / (float)N;
  a.in_sb = in_stride_batch; a.in_ss = in_stride_seq; a.dx_sb = dx_stride_batch; a.dx_ss = dx_stride_seq;
  a.g_sb = g_strides->batch; a.g_ss = g_strides->seq; a.g_sh = g_strides->head;
  hipStream_t st = (hipStream_t)stream;
  MDATTN_LAUNCH(kern, dim3(nb), dim3(256), 0, st, a);
  int rc = launch_status();
  if (rc != MDATTN_OK) return rc;
  return launch_colsum(st, workspace, nb, (int)N, (int)N, dw, nullptr, nullptr, nullptr);
}
