// Software-pipelined non-causal flash-attention forward for gfx950 (MI355X), bf16 MFMA, head_dim 128.
//
// Each wave owns QB*32 query rows and walks the keys in blocks of 32.  In iteration b the wave issues,
// interleaved in one instruction stream,
//     matrix pipe : O^T += V^T(b-1).P^T(b-1)   (8*QB MFMAs)   and   S^T(b+1) = K(b+1).Q^T   (8*QB MFMAs)
//     vector ALU  : P(b) = exp2(c*S(b) - c*m), row sums, bf16 convert
//     LDS         : the K / V^T fragments of MFMAs three issues ahead (rotating 4-register windows)
// so the softmax of one block hides under the MFMAs of its neighbours instead of alternating with
// them.  `sched_barrier` pins that interleaving; the compiler still places waits and hazards.
//
// Layouts (see attn_fwd_bf16.hip for the derivation): S^T = K.Q^T leaves every lane with 16 keys
// of ONE query row, so row max/sum are in-lane plus one half-wave swap; the accumulator layout of
// S^T is the B-operand layout of the PV MFMA; V^T fragments come from the row-major V tile through
// ds_read_b64_tr_b16.
//
// K/V tiles of 64 keys are staged through a 3-deep LDS ring.  Ring slot t%3 holds K(t) together with
// V(t-1): both are consumed during the same "period" (the two iterations 2t-1 and 2t).  One barrier
// per period; global loads for period t+3 are in flight in registers while t is consumed, and the
// fragment look-ahead may already read slot (t+1)%3.
#include <stdlib.h>

#include <type_traits>

#include "mdattn_common.h"

namespace mdattn {


namespace pipe {

constexpr int kBN = 64;                       // keys per LDS tile (two 32-key blocks)
constexpr int kD = 128;
constexpr int kKStr = kD + 8;                 // 272 B rows: 16 rows x 16 B cover all 64 banks
constexpr int kVStr = kD + 32;                // 320 B rows: 4 rows x 64 B cover all 64 banks
constexpr int kVOff = kBN * kKStr;            // V part of a ring slot, in elements
constexpr int kSlot = kBN * kKStr + kBN * kVStr;
constexpr int kRing = 3;
constexpr int kLdsBytes = kRing * kSlot * 2;  // 113 664 B
constexpr float kLazy = 8.0f;                 // log2 units a row max may lag before accumulators are rescaled

typedef s16x4 __attribute__((address_space(3))) * lds_s16x4_ptr;
typedef __attribute__((ext_vector_type(8))) short s16x8;

__device__ __forceinline__ bf16x8 read_vt(const __bf16* p0) {
  s16x4 r0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)p0);
  s16x4 r1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p0 + 8 * kVStr));
  s16x8 r = __builtin_shufflevector(r0, r1, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(bf16x8, r);
}

template <bool SM_, bool PV_, bool QK_, bool MASK_>
struct Flags {
  static constexpr bool SM = SM_, PV = PV_, QK = QK_, MASK = MASK_;
};

// softmax work of one iteration is cut into (query block, element pair) units, spread over the
// MFMA slots 3..15 (slot 0: the previous QK must drain; slots 1, 2: row maxima)
__device__ constexpr int pairs_in_slot(int n, int qb) {
  if (n < 3) return 0;
  if (qb == 1) return (n >= 3 && n <= 10) ? 1 : 0;
  return (n == 3 || n == 7 || n == 11) ? 2 : 1;  // 16 units over 13 slots
}
__device__ constexpr int first_pair_of_slot(int n, int qb) {
  int acc = 0;
  for (int i = 0; i < n; ++i) acc += pairs_in_slot(i, qb);
  return acc;
}

template <int QB, int NW>
__global__ __launch_bounds__(NW * 64) void attn_fwd_bf16_pipe_kernel(AttnArgs a) {
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  __bf16* smem = reinterpret_cast<__bf16*>(smem_raw);
  constexpr int NT = NW * 64;
  constexpr int LPT = (kBN * 16) / NT;  // 16-byte chunks per lane, tile and tensor
  constexpr int BM = NW * QB * 32;      // query rows per workgroup

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, hh = lane >> 5;

  const int wg = blockIdx.x;
  const int w = (wg & 7) * a.chunk + (wg >> 3);  // contiguous (head, q-tile) range per XCD
  if (w >= a.total) return;
  const int bh = w / a.nqt, qt = w - bh * a.nqt;
  const int b = bh / a.H, h = bh - b * a.H;

  const __bf16* qp = a.q + b * a.q_sb + h * a.q_sh;
  const __bf16* kp = a.k + b * a.k_sb + h * a.k_sh;
  const __bf16* vp = a.v + b * a.v_sb + h * a.v_sh;
  const int q0 = qt * BM + wave * (QB * 32);
  const int nt = (a.Skv + kBN - 1) / kBN;
  const bool tail = (a.Skv & (kBN - 1)) != 0;
  const float c = a.c;

  // ---- Q fragments (B operand of K.Q^T), resident for the whole kernel
  bf16x8 qf[QB][8];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    int row = q0 + qb * 32 + l32;
    row = row < a.Sq ? row : a.Sq - 1;
    const __bf16* p = qp + (int64_t)row * a.q_ss + hh * 8;
#pragma unroll
    for (int s = 0; s < 8; ++s) qf[qb][s] = *reinterpret_cast<const bf16x8*>(p + s * 16);
  }

  // ---- global -> register -> LDS staging of one ring slot: K(kt) and V(kt-1)
  u32x4 kr[LPT], vr[LPT];
  auto gload = [&](int kt) {
#pragma unroll
    for (int i = 0; i < LPT; ++i) {
      const int id = tid + i * NT;
      const int row = id >> 4, cc = id & 15;
      int kk = kt * kBN + row;
      kk = kk < a.Skv ? kk : a.Skv - 1;
      int kvv = (kt - 1) * kBN + row;
      kvv = kvv < a.Skv ? kvv : a.Skv - 1;
      kvv = kvv > 0 ? kvv : 0;
      kr[i] = *reinterpret_cast<const u32x4*>(kp + (int64_t)kk * a.k_ss + cc * 8);
      vr[i] = *reinterpret_cast<const u32x4*>(vp + (int64_t)kvv * a.v_ss + cc * 8);
    }
  };
  auto lstore = [&](int slot) {
    __bf16* Ks = smem + slot * kSlot;
#pragma unroll
    for (int i = 0; i < LPT; ++i) {
      const int id = tid + i * NT;
      const int row = id >> 4, cc = id & 15;
      *reinterpret_cast<u32x4*>(Ks + row * kKStr + cc * 8) = kr[i];
      *reinterpret_cast<u32x4*>(Ks + kVOff + row * kVStr + cc * 8) = vr[i];
    }
  };

  gload(0);
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): Q fragments and slot 0 have landed
  lstore(0);
  gload(1);
  __builtin_amdgcn_s_waitcnt(0x0F70);
  lstore(1);
  gload(2);  // stays in flight; stored at the top of period 0

  // lane-constant LDS offsets (elements)
  const int k_off = l32 * kKStr + hh * 8;
  const int v_off = kVOff + (4 * hh + ((lane & 15) >> 2)) * kVStr + ((lane >> 4) & 1) * 16 + 4 * (lane & 3);

  f32x16 O[QB][4];
  float m[QB], l[QB];
  f32x16 S0[QB], S1[QB];        // logits of even / odd blocks
  bf16x8 P0[QB][2], P1[QB][2];  // probabilities of even / odd blocks, PV B-operand layout
  bf16x8 kfr[4], vfr[4];        // rotating fragment windows
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    m[qb] = -1e30f;
    l[qb] = 0.f;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) O[qb][db][i] = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) { S0[qb][i] = 0.f; S1[qb][i] = 0.f; }
#pragma unroll
    for (int i = 0; i < 2; ++i) { P0[qb][i] = __builtin_bit_cast(bf16x8, make_uint4(0, 0, 0, 0)); P1[qb][i] = P0[qb][i]; }
  }

  // One iteration.  blk = block whose logits Scur holds.  Kc/Kn: K rows of block blk+1 / blk+2;
  // Vc/Vn: V rows of block blk-1 / blk (all already offset to the block's first row).
  auto iter = [&](auto flags, f32x16(&Scur)[QB], f32x16(&Snxt)[QB], bf16x8(&Pcur)[QB][2], bf16x8(&Pprev)[QB][2],
                  const __bf16* Kc, const __bf16* Kn, const __bf16* Vc, const __bf16* Vn, int blk) {
    using F = decltype(flags);
    float alpha[QB], mc[QB], lsum[QB];
    bool need = false;
    float p[QB][16];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) { alpha[qb] = 1.f; mc[qb] = 0.f; lsum[qb] = 0.f; }
#pragma unroll
    for (int n = 0; n < 16; ++n) {
      const int j = n >> 1;
      if ((n & 1) == 0) {
        if (F::PV) {
#pragma unroll
          for (int qb = 0; qb < QB; ++qb)
            O[qb][j & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vfr[j & 3], Pprev[qb][j >> 2], O[qb][j & 3], 0, 0, 0);
        }
        const int jn = j + 3;
        if (jn < 8) {
          if (F::PV) vfr[jn & 3] = read_vt(Vc + v_off + (jn >> 2) * 16 * kVStr + (jn & 3) * 32);
        } else {
          vfr[jn & 3] = read_vt(Vn + v_off + ((jn - 8) >> 2) * 16 * kVStr + ((jn - 8) & 3) * 32);
        }
      } else {
        if (F::QK) {
#pragma unroll
          for (int qb = 0; qb < QB; ++qb) {
            if (j == 0) {
              f32x16 z;
#pragma unroll
              for (int i = 0; i < 16; ++i) z[i] = 0.f;
              Snxt[qb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kfr[0], qf[qb][0], z, 0, 0, 0);
            } else {
              Snxt[qb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kfr[j & 3], qf[qb][j], Snxt[qb], 0, 0, 0);
            }
          }
        }
        const int jn = j + 3;
        if (jn < 8) {
          if (F::QK) kfr[jn & 3] = *reinterpret_cast<const bf16x8*>(Kc + k_off + jn * 16);
        } else {
          kfr[jn & 3] = *reinterpret_cast<const bf16x8*>(Kn + k_off + (jn - 8) * 16);
        }
      }
      if (F::SM) {
        if (n == 1 || (n == 2 && QB == 2)) {
          const int qb = n - 1;
          if (F::MASK) {
            const int kv_base = blk * 32 + 4 * hh;
#pragma unroll
            for (int i = 0; i < 16; ++i)
              if (kv_base + 8 * (i >> 2) + (i & 3) >= a.Skv) Scur[qb][i] = -INFINITY;
          }
          float mloc = Scur[qb][0];
#pragma unroll
          for (int i = 1; i < 16; ++i) mloc = fmaxf(mloc, Scur[qb][i]);
          mloc = xhalf_max(mloc);
          // Lazy rescale: a row's running max moves only when it would otherwise see an exp2 argument
          // above kLazy (a per-lane select, so the instruction stream stays one basic block); the
          // accumulator multiply is deferred to the iteration end, after every PV MFMA of the previous
          // block has been issued, and is skipped when no row of the wave moved.
          const bool moved = (mloc - m[qb]) * c > kLazy;
          const float mnew = moved ? mloc : m[qb];
          alpha[qb] = __builtin_amdgcn_exp2f((m[qb] - mnew) * c);  // exactly 1 for rows that keep their max
          m[qb] = mnew;
          need = need || (__builtin_amdgcn_ballot_w64(moved) != 0);
          mc[qb] = m[qb] * c;
          asm volatile("" : "+v"(alpha[qb]), "+v"(mc[qb]));
        }
        constexpr int kUnitsPerQb = 8;
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          if (u < pairs_in_slot(n, QB)) {
            const int unit = first_pair_of_slot(n, QB) + u;  // 0 .. 8*QB-1
            const int qb = unit / kUnitsPerQb, e = (unit % kUnitsPerQb) * 2;
            p[qb][e] = __builtin_amdgcn_exp2f(__builtin_fmaf(Scur[qb][e], c, -mc[qb]));
            p[qb][e + 1] = __builtin_amdgcn_exp2f(__builtin_fmaf(Scur[qb][e + 1], c, -mc[qb]));
            lsum[qb] += p[qb][e] + p[qb][e + 1];
            // keeps this pair's exp2 in its slot: without a use here the compiler sinks the whole softmax
            // below the MFMA stream, next to the first use of P in the following iteration
            asm volatile("" : "+v"(p[qb][e]), "+v"(p[qb][e + 1]), "+v"(lsum[qb]));
            if ((e & 7) == 6) {  // elements 0..7 / 8..15 of this query block complete
              const int g = e >> 3;
              Pcur[qb][g] = __builtin_bit_cast(bf16x8, pack8(&p[qb][8 * g]));
              asm volatile("" : "+v"(Pcur[qb][g]));
            }
          }
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if (F::SM) {
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) l[qb] = l[qb] * alpha[qb] + lsum[qb];
      if (need) {
#pragma unroll
        for (int qb = 0; qb < QB; ++qb)
#pragma unroll
          for (int db = 0; db < 4; ++db)
#pragma unroll
            for (int i = 0; i < 16; ++i) O[qb][db][i] *= alpha[qb];
      }
    }
  };

  // ring slot bookkeeping: slot of period t is t % 3
  int s_cur = 0, s_nxt = 1, s_fill = 2;
  auto period_top = [&](int t) {
    __syncthreads();                       // slot s_fill is no longer read; slots s_cur, s_nxt are complete
    __builtin_amdgcn_s_waitcnt(0x0F70);    // the loads issued one period ago have landed
    lstore(s_fill);                        // K(t+2), V(t+1)
    gload(t + 3);
  };
  auto kblk = [&](int slot, int half) { return smem + slot * kSlot + half * 32 * kKStr; };
  auto vblk = [&](int slot, int half) { return smem + slot * kSlot + half * 32 * kVStr; };
  auto rotate = [&]() { const int t = s_cur; s_cur = s_nxt; s_nxt = s_fill; s_fill = t; };

  // ---- period 0: iteration -1 (QK(0) only) and iteration 0 (softmax(0), QK(1))
  period_top(0);
#pragma unroll
  for (int s = 0; s < 3; ++s) kfr[s] = *reinterpret_cast<const bf16x8*>(kblk(s_cur, 0) + k_off + s * 16);
  iter(Flags<false, false, true, false>{}, S1, S0, P1, P0, kblk(s_cur, 0), kblk(s_cur, 1), vblk(s_cur, 0), vblk(s_cur, 0), -1);
  if (nt == 1 && tail)
    iter(Flags<true, false, true, true>{}, S0, S1, P0, P1, kblk(s_cur, 1), kblk(s_nxt, 0), vblk(s_cur, 0), vblk(s_nxt, 0), 0);
  else
    iter(Flags<true, false, true, false>{}, S0, S1, P0, P1, kblk(s_cur, 1), kblk(s_nxt, 0), vblk(s_cur, 0), vblk(s_nxt, 0), 0);
  rotate();

  // ---- periods 1 .. nt-1: iterations 2t-1 and 2t, fully pipelined
  for (int t = 1; t < nt; ++t) {
    period_top(t);
    const int b1 = 2 * t - 1;
    iter(Flags<true, true, true, false>{}, S1, S0, P1, P0, kblk(s_cur, 0), kblk(s_cur, 1), vblk(s_cur, 0), vblk(s_cur, 1), b1);
    if (t == nt - 1 && tail)
      iter(Flags<true, true, true, true>{}, S0, S1, P0, P1, kblk(s_cur, 1), kblk(s_nxt, 0), vblk(s_cur, 1), vblk(s_nxt, 0), b1 + 1);
    else
      iter(Flags<true, true, true, false>{}, S0, S1, P0, P1, kblk(s_cur, 1), kblk(s_nxt, 0), vblk(s_cur, 1), vblk(s_nxt, 0), b1 + 1);
    rotate();
  }

  // ---- period nt: iteration 2nt-1 (softmax of the last block, PV of the one before) and 2nt (last PV)
  period_top(nt);
  if (tail)
    iter(Flags<true, true, false, true>{}, S1, S0, P1, P0, kblk(s_cur, 0), kblk(s_cur, 1), vblk(s_cur, 0), vblk(s_cur, 1), 2 * nt - 1);
  else
    iter(Flags<true, true, false, false>{}, S1, S0, P1, P0, kblk(s_cur, 0), kblk(s_cur, 1), vblk(s_cur, 0), vblk(s_cur, 1), 2 * nt - 1);
  iter(Flags<false, true, false, false>{}, S0, S1, P0, P1, kblk(s_cur, 1), kblk(s_cur, 1), vblk(s_cur, 1), vblk(s_cur, 1), 2 * nt);

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

}  // namespace pipe

template <int QB, int NW>
static int launch_pipe(hipStream_t st, AttnArgs a, int B) {
  constexpr int BM = NW * QB * 32;
  a.nqt = (a.Sq + BM - 1) / BM;
  const int64_t total = (int64_t)B * a.H * a.nqt;
  if (total > (int64_t)0x7FFFFFF0) return MDATTN_E_UNSUPPORTED;
  a.total = (int)total;
  a.chunk = (a.total + 7) / 8;
  auto kern = pipe::attn_fwd_bf16_pipe_kernel<QB, NW>;
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, pipe::kLdsBytes) != hipSuccess)
    return MDATTN_E_LAUNCH;
  hipLaunchKernelGGL(kern, dim3(a.chunk * 8), dim3(NW * 64), pipe::kLdsBytes, st, a);
  return launch_status();
}

int launch_fwd_pipe(hipStream_t st, AttnArgs a, int B, int rows_per_wave) {
  if (rows_per_wave == 64) return launch_pipe<2, 4>(st, a, B);
  if (rows_per_wave == 32) return launch_pipe<1, 4>(st, a, B);
  return launch_pipe<1, 8>(st, a, B);
}

}  // namespace mdattn
