// Non-causal flash-attention forward for gfx950 (MI355X), bf16 MFMA, head_dim 128.
//
// Work decomposition
//   workgroup  = NW waves, each wave owns QB blocks of 32 query rows  (BM = NW*QB*32 rows)
//   K/V tiles  = 64 keys x 128, staged through LDS in two stages (global loads of tile i+1 are in
//                flight while tile i is consumed; one barrier per tile)
//   S^T = K.Q^T with v_mfma_f32_32x32x16_bf16: A = K rows from LDS (ds_read_b128), B = Q fragment
//                held in registers for the whole kernel.  In the 32x32 accumulator layout every lane
//                then holds 16 keys of ONE query row, so the row max / row sum are in-lane
//                reductions plus a single swap between the two wave halves, and the running
//                max / sum / rescale factor are per-lane scalars.
//   O^T += V^T.P^T: the accumulator layout of S^T is already the B-operand layout of the next MFMA
//                (after the bf16 convert), and the A operand V^T comes from the row-major V tile
//                through the transposing LDS read (ds_read_b64_tr_b16).
//   softmax    = exp2 with scale*log2(e) folded into one FMA per logit; f32 state.
//   grid       = 1-D, remapped so that each XCD (workgroup id mod 8) walks a contiguous range of
//                (head, q-tile) pairs: the workgroups resident on one XCD stream the same K/V and
//                share it through that XCD's L2.
#include <stdlib.h>

#include <type_traits>

#include "mdattn_common.h"

namespace mdattn {


constexpr int kBN = 64;          // keys per tile
constexpr int kD = 128;          // head dim
constexpr int kKStr = kD + 8;    // K row stride in LDS (272 B: 16 rows x 16 B hit 64 distinct banks)
constexpr int kVStr = kD + 32;   // V row stride in LDS (320 B: 4 rows x 64 B hit 64 distinct banks)
constexpr int kStage = kBN * kKStr + kBN * kVStr;  // elements per stage
constexpr int kLdsBytes = 2 * kStage * 2;
constexpr float kLazy = 8.0f;      // log2 units a row max may lag behind before accumulators are rescaled

typedef s16x4 __attribute__((address_space(3))) * lds_s16x4_ptr;
typedef __attribute__((ext_vector_type(8))) short s16x8;

__device__ __forceinline__ bf16x8 read_vt(const __bf16* p0, const __bf16* p1) {
  s16x4 r0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)p0);
  s16x4 r1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)p1);
  s16x8 r = __builtin_shufflevector(r0, r1, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(bf16x8, r);
}

template <int QB, int NW>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(QB == 1 ? 2 : 1, QB == 1 ? 2 : 1)))
void attn_fwd_bf16_kernel(AttnArgs a) {
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  __bf16* smem = reinterpret_cast<__bf16*>(smem_raw);
  constexpr int NT = NW * 64;
  constexpr int LPT = (kBN * 16) / NT;  // 16-byte chunks per lane per tile and tensor
  constexpr int BM = NW * QB * 32;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, hh = lane >> 5;

  const int wg = blockIdx.x;
  const int w = (wg & 7) * a.chunk + (wg >> 3);
  if (w >= a.total) return;
  const int bh = w / a.nqt, qt = w - bh * a.nqt;
  const int b = bh / a.H, h = bh - b * a.H;

  const __bf16* qp = a.q + b * a.q_sb + h * a.q_sh;
  const __bf16* kp = a.k + b * a.k_sb + h * a.k_sh;
  const __bf16* vp = a.v + b * a.v_sb + h * a.v_sh;
  const int q0 = qt * BM + wave * (QB * 32);
  const int nt = (a.Skv + kBN - 1) / kBN;
  const float c = a.c;

  // ---- Q fragments (B operand of K.Q^T), kept in registers for the whole kernel
  bf16x8 qf[QB][8];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    int row = q0 + qb * 32 + l32;
    row = row < a.Sq ? row : a.Sq - 1;
    const __bf16* p = qp + (int64_t)row * a.q_ss + hh * 8;
#pragma unroll
    for (int s = 0; s < 8; ++s) qf[qb][s] = *reinterpret_cast<const bf16x8*>(p + s * 16);
  }

  // ---- stage tile 0
  u32x4 kr[LPT], vr[LPT];
#define MDATTN_GLOAD(IT)                                                                       \
  _Pragma("unroll") for (int i = 0; i < LPT; ++i) {                                            \
    const int id = tid + i * NT;                                                               \
    const int row = id >> 4, cc = id & 15;                                                     \
    int kv = (IT) * kBN + row;                                                                 \
    kv = kv < a.Skv ? kv : a.Skv - 1;                                                          \
    kr[i] = *reinterpret_cast<const u32x4*>(kp + (int64_t)kv * a.k_ss + cc * 8);               \
    vr[i] = *reinterpret_cast<const u32x4*>(vp + (int64_t)kv * a.v_ss + cc * 8);               \
  }
#define MDATTN_LSTORE(STAGE)                                                                   \
  {                                                                                            \
    __bf16* Ks_ = smem + (STAGE) * kStage;                                                     \
    __bf16* Vs_ = Ks_ + kBN * kKStr;                                                           \
    _Pragma("unroll") for (int i = 0; i < LPT; ++i) {                                          \
      const int id = tid + i * NT;                                                             \
      const int row = id >> 4, cc = id & 15;                                                   \
      *reinterpret_cast<u32x4*>(Ks_ + row * kKStr + cc * 8) = kr[i];                           \
      *reinterpret_cast<u32x4*>(Vs_ + row * kVStr + cc * 8) = vr[i];                           \
    }                                                                                          \
  }
  MDATTN_GLOAD(0)  // issued after the Q loads: waiting for tile 0 then also completes them

  f32x16 O[QB][4];
  float m[QB], l[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    m[qb] = -1e30f;
    l[qb] = 0.f;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) O[qb][db][i] = 0.f;
  }

  // every global load issued so far (Q fragments, tile 0) completes here: the loop starts with no
  // vector-memory operation pending, so its own prefetches are never waited on early
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
  MDATTN_LSTORE(0)
  __syncthreads();

  // lane-constant LDS offsets
  const int k_off = l32 * kKStr + hh * 8;
  const int v_off = (4 * hh + ((lane & 15) >> 2)) * kVStr + ((lane >> 4) & 1) * 16 + 4 * (lane & 3);

  // One KV tile.  MASK is set only for the last tile of a ragged key axis, so the main loop carries
  // no per-element compare/select.
  auto tile = [&](int it, auto mask_tag) {
    constexpr bool MASK = decltype(mask_tag)::value;
    const int stage = it & 1;
    const bool more = it + 1 < nt;
    if (more) { MDATTN_GLOAD(it + 1) }

    const __bf16* Ks = smem + stage * kStage;
    const __bf16* Vs = Ks + kBN * kKStr;

    // ---- S^T = K Q^T; accumulators alternate so that consecutive MFMAs are independent
    f32x16 S[QB][2];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb)
#pragma unroll
      for (int jb = 0; jb < 2; ++jb)
#pragma unroll
        for (int i = 0; i < 16; ++i) S[qb][jb][i] = 0.f;
    // all K fragments are requested before the first MFMA so that LDS latency is paid once per tile
    bf16x8 kf[2][8];
#pragma unroll
    for (int s = 0; s < 8; ++s)
#pragma unroll
      for (int jb = 0; jb < 2; ++jb) kf[jb][s] = *reinterpret_cast<const bf16x8*>(Ks + jb * 32 * kKStr + k_off + s * 16);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int s = 0; s < 8; ++s)
#pragma unroll
      for (int jb = 0; jb < 2; ++jb)
#pragma unroll
        for (int qb = 0; qb < QB; ++qb)
          S[qb][jb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[jb][s], qf[qb][s], S[qb][jb], 0, 0, 0);
    // V^T fragments for the PV product are requested now and land while the softmax runs
    bf16x8 vf[4][4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
      for (int db = 0; db < 4; ++db) {
        const __bf16* p0 = Vs + v_off + ks * 16 * kVStr + db * 32;
        vf[ks][db] = read_vt(p0, p0 + 8 * kVStr);
      }
    __builtin_amdgcn_sched_barrier(0);

    if (MASK) {
      const int kv_base = it * kBN + 4 * hh;
#pragma unroll
      for (int jb = 0; jb < 2; ++jb)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int kv = kv_base + jb * 32 + 8 * (i >> 2) + (i & 3);
          if (kv >= a.Skv) {
#pragma unroll
            for (int qb = 0; qb < QB; ++qb) S[qb][jb][i] = -INFINITY;
          }
        }
    }

    // ---- online softmax; P^T leaves in the B-operand layout of the PV MFMA
    bf16x8 P[QB][4];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      float mloc = S[qb][0][0];
#pragma unroll
      for (int jb = 0; jb < 2; ++jb)
#pragma unroll
        for (int i = 0; i < 16; ++i) mloc = fmaxf(mloc, S[qb][jb][i]);
      mloc = xhalf_max(mloc);
      // Lazy rescale: the running max only moves when some row of this wave would otherwise see
      // exp2 arguments above kLazy (P <= 2^kLazy stays exact enough in bf16/f32); with a stale max
      // the accumulators need no multiply.  The branch is wave-uniform.
      if (__builtin_amdgcn_ballot_w64((mloc - m[qb]) * c > kLazy) != 0) {
        const float mnew = fmaxf(m[qb], mloc);
        const float alpha = __builtin_amdgcn_exp2f((m[qb] - mnew) * c);
        m[qb] = mnew;
        l[qb] *= alpha;
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
          for (int i = 0; i < 16; ++i) O[qb][db][i] *= alpha;
      }
      const float mc = m[qb] * c;
      float lsum = 0.f;
#pragma unroll
      for (int jb = 0; jb < 2; ++jb) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          float p[8];
#pragma unroll
          for (int t = 0; t < 8; ++t) {
            p[t] = __builtin_amdgcn_exp2f(__builtin_fmaf(S[qb][jb][8 * j + t], c, -mc));
            lsum += p[t];
          }
          P[qb][2 * jb + j] = __builtin_bit_cast(bf16x8, pack8(p));
        }
      }
      l[qb] += lsum;
    }

    // ---- O^T += V^T P^T
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int qb = 0; qb < QB; ++qb)
          O[qb][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[ks][db], P[qb][ks], O[qb][db], 0, 0, 0);

    if (more) MDATTN_LSTORE(stage ^ 1)
    __syncthreads();
  };

  if (a.prio == 1 && NW == 8 && wave < 4) __builtin_amdgcn_s_setprio(2);
  if (a.prio == 2 && NW == 4 && ((blockIdx.x >> 3) & 1)) __builtin_amdgcn_s_setprio(2);
  const int nfull = a.Skv / kBN;  // tiles with 64 valid keys
  for (int it = 0; it < nfull; ++it) tile(it, std::false_type{});
  if (nfull < nt) tile(nfull, std::true_type{});

  // ---- epilogue: normalise, convert, store; lse = m*scale + ln(l)
  __bf16* op = a.out + b * a.o_sb + h * a.o_sh;
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const float lt = xhalf_sum(l[qb]);
    const float inv = 1.0f / lt;
    const int row = q0 + qb * 32 + l32;
    if (row < a.Sq) {
      __bf16* orow = op + (int64_t)row * a.o_ss + 4 * hh;
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          uint2 u;
          u.x = pack2(O[qb][db][4 * g] * inv, O[qb][db][4 * g + 1] * inv);
          u.y = pack2(O[qb][db][4 * g + 2] * inv, O[qb][db][4 * g + 3] * inv);
          *reinterpret_cast<uint2*>(orow + db * 32 + 8 * g) = u;
        }
      if (a.lse && hh == 0) a.lse[((int64_t)b * a.H + h) * a.Sq + row] = (m[qb] * c + __log2f(lt)) * kLn2;
    }
  }
}

template <int QB, int NW>
static int launch_fwd(hipStream_t st, AttnArgs a, int B) {
  constexpr int BM = NW * QB * 32;
  a.nqt = (a.Sq + BM - 1) / BM;
  const int64_t total = (int64_t)B * a.H * a.nqt;
  if (total > (int64_t)0x7FFFFFF0) return MDATTN_E_UNSUPPORTED;
  a.total = (int)total;
  a.chunk = (a.total + 7) / 8;
  auto kern = attn_fwd_bf16_kernel<QB, NW>;
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes) != hipSuccess)
    return MDATTN_E_LAUNCH;
  hipLaunchKernelGGL(kern, dim3(a.chunk * 8), dim3(NW * 64), kLdsBytes, st, a);
  return launch_status();
}

}  // namespace mdattn

using namespace mdattn;

extern "C" int mdattn_fwd_bf16(void* stream, const void* q, const void* k, const void* v, void* out, float* lse,
                               int B, int H, int Sq, int Skv, int D,
                               const mdattn_strides* q_strides, const mdattn_strides* k_strides,
                               const mdattn_strides* v_strides, const mdattn_strides* o_strides, float scale) {
  if (!q || !k || !v || !out || B <= 0 || H <= 0 || Sq <= 0 || Skv <= 0 || D <= 0) return MDATTN_E_BADARG;
  if (!q_strides || !k_strides || !v_strides || !o_strides) return MDATTN_E_BADARG;
  if (!(scale > 0.f) || !(scale < 1e30f)) return MDATTN_E_BADARG;
  if (D != kD) return MDATTN_E_UNSUPPORTED;
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(out) || (reinterpret_cast<uintptr_t>(lse) & 3u))
    return MDATTN_E_ALIGN;
  if (!strides_ok(q_strides, 8) || !strides_ok(k_strides, 8) || !strides_ok(v_strides, 8) || !strides_ok(o_strides, 8))
    return MDATTN_E_ALIGN;
  if (q_strides->seq < D || k_strides->seq < D || v_strides->seq < D || o_strides->seq < D) return MDATTN_E_BADARG;

  AttnArgs a;
  a.q = (const __bf16*)q; a.k = (const __bf16*)k; a.v = (const __bf16*)v; a.out = (__bf16*)out; a.lse = lse;
  a.H = H; a.Sq = Sq; a.Skv = Skv;
  a.q_sb = q_strides->batch; a.q_ss = q_strides->seq; a.q_sh = q_strides->head;
  a.k_sb = k_strides->batch; a.k_ss = k_strides->seq; a.k_sh = k_strides->head;
  a.v_sb = v_strides->batch; a.v_ss = v_strides->seq; a.v_sh = v_strides->head;
  a.o_sb = o_strides->batch; a.o_ss = o_strides->seq; a.o_sh = o_strides->head;
  a.c = scale * kLog2e;
  a.prio = getenv("MDATTN_PRIO") ? atoi(getenv("MDATTN_PRIO")) : 0;
  hipStream_t st = (hipStream_t)stream;

  // Tile choice.  8 waves x 32 query rows (two waves per SIMD: one wave's softmax overlaps the
  // other's MFMAs) measures fastest at every size tried; 4 waves x 32 rows gives more workgroups
  // when there are few (head, q-tile) pairs.  MDATTN_FWD_VARIANT overrides for experiments.
  int variant = 0;
  if (const char* e = getenv("MDATTN_FWD_VARIANT")) variant = atoi(e);
  if (variant == 0) {
    const int64_t wg256 = (int64_t)B * H * ((Sq + 255) / 256);
    variant = wg256 >= 256 ? 3 : 2;
  }
  switch (variant) {
    case 1: return launch_fwd<2, 4>(st, a, B);
    case 2: return launch_fwd<1, 4>(st, a, B);
    case 3: return launch_fwd<1, 8>(st, a, B);
    case 4: return launch_fwd_pipe(st, a, B, 64);
    case 5: return launch_fwd_pipe(st, a, B, 32);
    case 6: return launch_fwd_pipe(st, a, B, 0);
    default: return MDATTN_E_BADARG;
  }
}
