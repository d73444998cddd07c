// Measurement hooks, not part of the C ABI (not declared in mdattn.h; bench.py binds them by name).
//
// mdattn_probe_dq_atomics: the f32 atomic-add traffic a single-pass backward would generate for dq.  Such a pass makes
// key rows the resident rows of a workgroup (8 waves x 32 keys) and streams the query tiles past them; every (query
// tile, key block) pair then yields a 32 x head_dim partial of dq that has to be added into global memory.  The probe
// issues exactly those atomics and nothing else: with `per_wave` every wave adds its own partial (no exchange inside
// the workgroup), without it the workgroup adds one partial per query tile, as if its eight waves had reduced theirs
// first (each wave adds an eighth).  The time of the launch is a lower bound of what the atomics would add to a
// backward pass that saved its two duplicate matrix products.
//
// mdattn_probe_mfma_rate: what the chip sustains on MFMA 32x32x16 bf16 issued back to back (two waves per SIMD, four
// independent accumulators per wave, nothing to wait for), alone and with the LDS reads and vector instructions an
// attention loop issues beside its MFMAs.  The shader clock is managed against a power limit, so the published peak
// (every SIMD starting an MFMA every 32 clocks at 2.4 GHz) is an upper bound that random operands do not reach; the
// probe gives the bound that applies to a given instruction mix and operand content.  `mode` bits: 1 = the A operand
// of every MFMA is read from LDS (1 KB per MFMA, as the K / V fragments are), 2 = of every second MFMA (two MFMAs
// share a fragment), 4 = two exp2, two adds and one bf16 pack per MFMA (the softmax of head dim 64), 16 = half of
// that (head dim 128), 8 = all operands zero instead of the caller's data.
#include "mdattn_common.h"

namespace mdattn {
__global__ __launch_bounds__(512) void probe_dq_atomics_kernel(float* dq, int Sq, int D, int nkt, int per_wave) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int h = blockIdx.x / nkt;
  float* base = dq + (int64_t)h * Sq * D;
  const int tile_floats = 32 * D;
  const int nqt = Sq / 32;
  const int per_lane = per_wave ? tile_floats / 64 : tile_floats / 512;
  const int first = per_wave ? 0 : wave * per_lane;
  // the workgroups of one head start at different query tiles, as drifting workgroups of a real pass would
  int t = (int)(((int64_t)(blockIdx.x % nkt) * nqt) / nkt);
  for (int i = 0; i < nqt; ++i) {
    float* tile = base + (int64_t)t * tile_floats;
    for (int j = 0; j < per_lane; ++j) unsafeAtomicAdd(tile + (first + j) * 64 + lane, 1.0f);
    t = t + 1 == nqt ? 0 : t + 1;
  }
}

template <int MODE>
__global__ __launch_bounds__(256, 2) void probe_mfma_rate_kernel(const unsigned* src, float* out, int iters) {
  __shared__ __attribute__((aligned(16))) unsigned smem[32768 / 4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int i = tid; i < 32768 / 4; i += 256) smem[i] = (MODE & 8) ? 0u : src[i];
  __syncthreads();
  bf16x8 bfr[4], afr[4];
  for (int j = 0; j < 4; ++j) {
    u32x4 t, u;
    for (int e = 0; e < 4; ++e) {
      t[e] = (MODE & 8) ? 0u : src[8192 + (j * 64 + lane) * 4 + e];
      u[e] = (MODE & 8) ? 0u : src[12288 + (j * 64 + lane) * 4 + e];
    }
    bfr[j] = __builtin_bit_cast(bf16x8, t);
    afr[j] = __builtin_bit_cast(bf16x8, u);
  }
  f32x16 acc[4];
  for (int j = 0; j < 4; ++j)
    for (int i = 0; i < 16; ++i) acc[j][i] = 0.f;
  float vs = 0.f, x = (MODE & 8) ? 0.f : 0.001f * lane;
  unsigned pk = 0;
  const u32x4* lds = reinterpret_cast<const u32x4*>(smem) + lane + wave * 512;  // 8 KB per wave, read 1 KB at a time
  bf16x8 win[2];
  win[0] = __builtin_bit_cast(bf16x8, lds[0]);
  win[1] = __builtin_bit_cast(bf16x8, lds[64]);
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if constexpr ((MODE & 1) != 0) {  // a window of two reads runs ahead of the MFMAs, as in the attention kernels
        acc[j & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(win[j & 1], bfr[j & 3], acc[j & 3], 0, 0, 0);
        win[j & 1] = __builtin_bit_cast(bf16x8, lds[((j + 2) & 7) * 64]);
      } else if constexpr ((MODE & 2) != 0) {
        acc[j & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(win[(j >> 1) & 1], bfr[j & 3], acc[j & 3], 0, 0, 0);
        if (j & 1) win[(j >> 1) & 1] = __builtin_bit_cast(bf16x8, lds[(((j >> 1) + 2) & 3) * 64]);
      } else {
        acc[j & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(afr[j & 3], bfr[j & 3], acc[j & 3], 0, 0, 0);
      }
      if ((MODE & 4) || ((MODE & 16) && (j & 1))) {
        const float e0 = __builtin_amdgcn_exp2f(x), e1 = __builtin_amdgcn_exp2f(-x);
        vs += e0;
        vs += e1;
        pk ^= pack2(e0, e1);
        asm volatile("" : "+v"(vs), "+v"(pk), "+v"(x));
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  float r = vs + __builtin_bit_cast(float, pk & 0x3fffffffu);
  for (int j = 0; j < 4; ++j)
    for (int i = 0; i < 16; ++i) r += acc[j][i];
  out[blockIdx.x * 256 + tid] = r;
}

// The same for the fp8 MFMA (32x32x64 f8f6f4 on e4m3 operands: four times the FLOP of the bf16 instruction in twice its
// clocks).  MODE bit 1: the A operand (2 KB) of every MFMA is read from
// LDS; bit 4: four exp2, four adds and two 4-byte packs per MFMA (an fp8 attention loop's softmax at head dim 128);
// bit 8: operands zero.
template <int MODE>
__global__ __launch_bounds__(256, 2) void probe_mfma_rate_fp8_kernel(const unsigned* src, float* out, int iters) {
  __shared__ __attribute__((aligned(16))) unsigned smem[65536 / 4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int i = tid; i < 65536 / 4; i += 256) smem[i] = (MODE & 8) ? 0u : src[i & 16383];
  __syncthreads();
  i32x8 bfr[4], afr[4];
  for (int j = 0; j < 4; ++j)
    for (int e = 0; e < 8; ++e) {
      bfr[j][e] = (MODE & 8) ? 0 : (int)src[(j * 64 + lane) * 8 + e];
      afr[j][e] = (MODE & 8) ? 0 : (int)src[4096 + (j * 64 + lane) * 8 + e];
    }
  f32x16 acc[4];
  for (int j = 0; j < 4; ++j)
    for (int i = 0; i < 16; ++i) acc[j][i] = 0.f;
  float vs = 0.f, x = (MODE & 8) ? 0.f : 0.001f * lane;
  unsigned pk = 0;
  const u32x4* lds = reinterpret_cast<const u32x4*>(smem) + lane + wave * 1024;  // 16 KB per wave, read 2 KB at a time
  auto rd = [&](int f) __attribute__((always_inline)) {
    const u32x4 lo = lds[f * 128], hi = lds[f * 128 + 64];
    return i32x8{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
  };
  i32x8 win[2];
  win[0] = rd(0);
  win[1] = rd(1);
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if constexpr ((MODE & 1) != 0) {
        acc[j & 3] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(win[j & 1], bfr[j & 3], acc[j & 3], 0, 0, 0, 0, 0, 0);
        win[j & 1] = rd((j + 2) & 7);
      } else {
        acc[j & 3] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(afr[j & 3], bfr[j & 3], acc[j & 3], 0, 0, 0, 0, 0, 0);
      }
      if constexpr ((MODE & 4) != 0) {
        const float e0 = __builtin_amdgcn_exp2f(x), e1 = __builtin_amdgcn_exp2f(-x);
        vs += e0;
        vs += e1;
        pk = (unsigned)__builtin_amdgcn_cvt_pk_fp8_f32(e0, e1, (int)pk, false);
        asm volatile("" : "+v"(vs), "+v"(pk), "+v"(x));
        const float e2 = __builtin_amdgcn_exp2f(x), e3 = __builtin_amdgcn_exp2f(-x);
        vs += e2;
        vs += e3;
        pk = (unsigned)__builtin_amdgcn_cvt_pk_fp8_f32(e2, e3, (int)pk, true);
        asm volatile("" : "+v"(vs), "+v"(pk), "+v"(x));
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  float r = vs + __builtin_bit_cast(float, pk & 0x3f3f3f3fu);
  for (int j = 0; j < 4; ++j)
    for (int i = 0; i < 16; ++i) r += acc[j][i];
  out[blockIdx.x * 256 + tid] = r;
}
}  // namespace mdattn

// src: 16384 words of operand data (bf16 pairs, or fp8 quadruples for modes >= 32); out: grid * 256 floats.  Every wave
// issues 8 * iters MFMAs.
extern "C" int mdattn_probe_mfma_rate(void* stream, int mode, int iters, int grid, const unsigned* src, float* out) {
  if (!src || !out || iters <= 0 || grid <= 0) return MDATTN_E_BADARG;
  hipStream_t st = (hipStream_t)stream;
#define MDATTN_PROBE_CASE(M) \
  case M: MDATTN_LAUNCH(mdattn::probe_mfma_rate_kernel<M>, dim3(grid), dim3(256), 0, st, src, out, iters); break;
  switch (mode) {
    MDATTN_PROBE_CASE(0) MDATTN_PROBE_CASE(1) MDATTN_PROBE_CASE(2) MDATTN_PROBE_CASE(4) MDATTN_PROBE_CASE(5) MDATTN_PROBE_CASE(6)
    MDATTN_PROBE_CASE(16) MDATTN_PROBE_CASE(17) MDATTN_PROBE_CASE(18) MDATTN_PROBE_CASE(8) MDATTN_PROBE_CASE(9)
#define MDATTN_PROBE_CASE8(M) \
  case 32 + M: MDATTN_LAUNCH(mdattn::probe_mfma_rate_fp8_kernel<M>, dim3(grid), dim3(256), 0, st, src, out, iters); break;
    MDATTN_PROBE_CASE8(0) MDATTN_PROBE_CASE8(1) MDATTN_PROBE_CASE8(4) MDATTN_PROBE_CASE8(5) MDATTN_PROBE_CASE8(8)
#undef MDATTN_PROBE_CASE8
    default: return MDATTN_E_BADARG;
  }
#undef MDATTN_PROBE_CASE
  return mdattn::launch_status();
}

extern "C" int mdattn_probe_dq_atomics(void* stream, float* dq, int H, int Sq, int Skv, int D, int per_wave) {
  if (!dq || H <= 0 || Sq < 32 || Skv < 256 || D <= 0 || D % 16) return MDATTN_E_BADARG;
  const int nkt = Skv / 256;
  MDATTN_LAUNCH(mdattn::probe_dq_atomics_kernel, dim3(H * nkt), dim3(512), 0, (hipStream_t)stream, dq, Sq / 32 * 32, D, nkt, per_wave);
  return mdattn::launch_status();
}
