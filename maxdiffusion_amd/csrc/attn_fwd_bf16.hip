// Non-causal flash-attention forward for gfx950 (MI355X), bf16 MFMA, head_dim 128.
//
// Work decomposition
//   workgroup  = NW waves, each wave owns 32 query rows  (BM = NW*32 rows); two waves per SIMD
//   K/V tiles  = 64 keys x 128, in a 4-deep LDS ring filled by direct global->LDS loads (no staging
//                registers, no LDS store instructions).  Ring slot t%4 holds K(t) together with V(t-1):
//                both are consumed in the same "period" (two 32-key iterations).  One barrier per
//                period; the loads of slots t+2 and t+3 are in flight while period t runs.
//   S^T = K.Q^T with v_mfma_f32_32x32x16_bf16: A = K rows from LDS (ds_read_b128), B = Q fragment
//                held in registers for the whole kernel.  In the 32x32 accumulator layout every lane
//                then holds 16 keys of ONE query row, so the row sum (and the row max, when needed) are
//                in-lane reductions plus a single swap between the two wave halves, and the reference
//                point / sum / rescale factor are per-lane scalars.
//   O^T += V^T.P^T: the accumulator layout of S^T is already the B-operand layout of the next MFMA
//                (after the bf16 convert), and the A operand V^T comes from the row-major V tile
//                through the transposing LDS read (ds_read_b64_tr_b16).
//   softmax    = exp2 with scale*log2(e) folded into one FMA per logit; f32 state.  A row's reference
//                point m is not its running maximum: it only keeps P, l and O inside the f32 exponent range and
//                moves when a logit exceeds it by about 20 log2 units, which the row's partial sum reveals, so
//                the hot stream computes no maximum at all and the accumulator rescale sits in a cold branch.
//                When the caller's q already carries scale*log2(e) (scale = ln 2: template flag PRE) the FMA goes
//                too: the score chains start from minus the reference point and P is one exp2 away.
//   pipelining = the vector ALU issues through the same port as the MFMAs.  Phases of pure MFMA
//                followed by phases of pure VALU leave the matrix pipe idle half of the time, so the
//                keys are walked in blocks of 32, and in iteration b every wave issues, interleaved in
//                one instruction stream,
//                    matrix pipe : O^T += V^T(b-1).P^T(b-1)  (8 MFMAs)  and  S^T(b+1) = K(b+1).Q^T  (8 MFMAs)
//                    vector ALU  : P(b) = exp2(c*S(b) - c*m), row sums, bf16 convert (3.5 instructions per MFMA,
//                                  2.5 with PRE)
//                    LDS         : the K / V^T fragment of the next MFMA of the same kind
//                PV and QK MFMAs alternate, so no MFMA depends on the one issued just before it.  The
//                loop body is the same for every iteration: the iterations before the first and after
//                the last real block run on fully masked logits (P = 0) instead of being peeled.
//   grid       = 1-D, remapped so that each XCD (workgroup id mod 8) walks a contiguous range of
//                (head, q-tile) pairs: the workgroups resident on one XCD stream the same K/V and
//                share it through that XCD's L2.
#include <type_traits>

#include "mdattn_common.h"

namespace mdattn {

constexpr int kBN = 64;          // keys per tile
constexpr int kD = 128;          // head dim
// LDS tile layouts (elements).  Tiles are filled by direct global->LDS loads.  One wave instruction
// writes 1 KB = one group of 4 rows, row-major; the lane -> global address map is free, so inside a row
// the 16-byte chunks are stored permuted (XOR with the row's position in its group), which replaces
// row padding:
//   K: chunk c of row r sits at chunk position c ^ (r & 3); groups are padded by 64 B.  The 16 lanes a
//      ds_read_b128 serves at once (16 rows, one logical chunk) hit 16 distinct 16-byte bank slots.
//   V: 64-byte segment s of row r sits at segment position s ^ (r & 3).  The 4 rows x 64 B a half-wave
//      reads through ds_read_b64_tr_b16 cover all 64 banks once.
// Every 16 lanes of a load fetch one whole 256-byte row from global memory.
constexpr int kGK = 4 * kD + 32;  // K group stride (1088 B)
constexpr int kGV = 4 * kD;       // V group stride (1024 B)
constexpr int kKTile = (kBN / 4) * kGK;
constexpr int kStage = kKTile + (kBN / 4) * kGV;  // elements per ring stage
// A 16-key partial row sum above this sends the wave to the branch that moves the rows' reference points.  The
// reference point only has to keep P, l and O inside the f32 / bf16 exponent range (the result does not depend on it,
// and bf16's relative precision is the same at every magnitude), so the alarm can sit far out: 2^24 lets a row's
// logits climb 20 log2 units above its reference before anything happens, and leaves 100 binades of headroom.
constexpr float kTrig = 16777216.0f;
constexpr int kS0 = 2;           // first slot of an iteration that touches the block's logits
constexpr int kLA = 1;           // LDS look-ahead: a slot requests the fragment of the kLA-th next MFMA of its kind
                                 // (1, 2 and 3 measure the same)

typedef s16x4 __attribute__((address_space(3))) * lds_s16x4_ptr;
typedef __attribute__((ext_vector_type(8))) short s16x8;

__device__ __forceinline__ bf16x8 read_vt(const __bf16* p0, const __bf16* p1) {
  s16x4 r0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)p0);
  s16x4 r1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)p1);
  s16x8 r = __builtin_shufflevector(r0, r1, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(bf16x8, r);
}

// Epilogue of both schedules for one query row: lane (row, hh) holds, for each 32-wide block db of the head dim, the
// values d = 32 db + 8 g + 4 hh + 0..3 (g = 0..3) of the un-normalised output, `lt` is the row's sum of P and `mc` its
// reference point in log2 units.  Either out = O / lt as bf16 and lse = ln 2 * (mc + log2 lt), or, with a running
// (o_run, lse_run) pair, the LSE-space merge of that result into the pair (ring_attention_kernel.py:1062-1073 of the
// reference, with (0, -1e30) as the neutral start): the attention result of this call never goes to memory.
template <int ND>
__device__ __forceinline__ void store_row(const AttnArgs& a, const f32x16 (&O)[ND], float lt, float mc, int b, int h,
                                          int row, int hh) {
  if (row >= a.Sq) return;
  const int64_t lidx = ((int64_t)b * a.H + h) * a.Sq + row;
  if (a.o_run) {
    const float l2 = lt > 0.f ? (mc + __log2f(lt)) * kLn2 : -INFINITY;
    const float l1 = a.lse_run[lidx];  // both lanes of the row read it before lane hh = 0 writes it back
    const float L = fmaxf(l1, l2);
    float w1 = 0.f, w2 = 0.f;
    if (L > -INFINITY) { w1 = expf(l1 - L); w2 = expf(l2 - L); }
    const float den = w1 + w2;
    const float invd = den > 0.f ? 1.0f / den : 0.f;
    w1 *= invd;
    w2 = lt > 0.f ? w2 * invd / lt : 0.f;
    float* orow = a.o_run + b * a.o_sb + h * a.o_sh + (int64_t)row * a.o_ss + 4 * hh;
#pragma unroll
    for (int db = 0; db < ND; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        float4* p = reinterpret_cast<float4*>(orow + db * 32 + 8 * g);
        float4 r = *p;
        r.x = w1 * r.x + w2 * O[db][4 * g];
        r.y = w1 * r.y + w2 * O[db][4 * g + 1];
        r.z = w1 * r.z + w2 * O[db][4 * g + 2];
        r.w = w1 * r.w + w2 * O[db][4 * g + 3];
        *p = r;
      }
    if (hh == 0) a.lse_run[lidx] = den > 0.f ? L + logf(den) : L;
    return;
  }
  const float inv = lt > 0.f ? 1.0f / lt : 0.f;  // rows whose keys are all excluded return 0
  __bf16* orow = a.out + b * a.o_sb + h * a.o_sh + (int64_t)row * a.o_ss + 4 * hh;
#pragma unroll
  for (int db = 0; db < ND; ++db)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      uint2 u;
      u.x = pack2(O[db][4 * g] * inv, O[db][4 * g + 1] * inv);
      u.y = pack2(O[db][4 * g + 2] * inv, O[db][4 * g + 3] * inv);
      *reinterpret_cast<uint2*>(orow + db * 32 + 8 * g) = u;
    }
  if (a.lse && hh == 0) a.lse[lidx] = (mc + __log2f(lt)) * kLn2;
}

// The same epilogue with whole-row stores, for a wave that may use `stage` (32 rows of HD * 2 + 16 bytes of LDS that
// nobody else touches any more).  store_row writes, per instruction, 16 bytes of each of 32 rows that lie a whole
// token apart; at short key sequences, where the output is a large part of the launch's work, that costs as much as
// the attention itself (75,600 x 40 x 128 outputs: 0.27 ms).  Here the wave's 32 x HD tile is normalised, rounded to
// bf16 and transposed through LDS, and every store instruction then writes 1 KB of whole rows (4 rows of 256 bytes
// at head dim 128).  Same values, same rounding as store_row.
template <int ND>
__device__ __forceinline__ void store_rows_through_lds(const AttnArgs& a, const f32x16 (&O)[ND], float lt, float mc, int b,
                                                       int h, int row0, int lane, char* stage) {
  constexpr int HD = ND * 32;
  constexpr int ROWB = HD * 2 + 16;      // padded row: the 32 lanes of a column write land on 16 different bank groups
  constexpr int LPR = HD * 2 / 16;       // lanes that share a row in the read-back
  constexpr int RPI = 64 / LPR;          // rows per store instruction
  const int l32 = lane & 31, hh = lane >> 5;
  const float inv = lt > 0.f ? 1.0f / lt : 0.f;  // rows whose keys are all excluded return 0
  char* wrow = stage + l32 * ROWB + hh * 8;
#pragma unroll
  for (int db = 0; db < ND; ++db)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      uint2 u;
      u.x = pack2(O[db][4 * g] * inv, O[db][4 * g + 1] * inv);
      u.y = pack2(O[db][4 * g + 2] * inv, O[db][4 * g + 3] * inv);
      *reinterpret_cast<uint2*>(wrow + (db * 32 + g * 8) * 2) = u;
    }
  const int row = row0 + l32;
  if (a.lse && hh == 0 && row < a.Sq) a.lse[((int64_t)b * a.H + h) * a.Sq + row] = (mc + __log2f(lt)) * kLn2;
  // LDS accesses of one wave execute in order: the reads below see the writes above
  __bf16* obase = a.out + b * a.o_sb + h * a.o_sh;
  const int rr = lane / LPR, cc = lane % LPR;
#pragma unroll
  for (int j = 0; j < 32 / RPI; ++j) {
    const int r = j * RPI + rr;
    const uint4 v = *reinterpret_cast<const uint4*>(stage + r * ROWB + cc * 16);
    // streaming store: the output is written once and read by nobody here (1.5 % on the 512-key cross-attention)
    if (row0 + r < a.Sq) st_nt(reinterpret_cast<uint4*>(obase + (int64_t)(row0 + r) * a.o_ss + cc * 8), v);
  }
}

template <int NW, bool PRE>
__global__ __launch_bounds__(NW * 64) void attn_fwd_bf16_kernel(AttnArgs a) {
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  __bf16* smem = reinterpret_cast<__bf16*>(smem_raw);
  constexpr int NT = NW * 64;
  constexpr int BM = NW * 32;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, hh = lane >> 5;

  const int wg = blockIdx.x;
  const int w = (wg & 7) * a.chunk + (wg >> 3);
  if (w >= a.total) return;
  const int bh = w / a.nqt, qt = w - bh * a.nqt;
  const int b = bh / a.H, h = bh - b * a.H;

  const __bf16* qp = a.q + b * a.q_sb + h * a.q_sh;
  const __bf16* kp = a.k + b * a.k_sb + h * a.k_sh;
  const __bf16* vp = a.v + b * a.v_sb + h * a.v_sh;
  const int q0 = qt * BM + wave * 32;
  const int nt = (a.Skv + kBN - 1) / kBN;
  const float c = a.c;

  // ---- Q fragments (B operand of K.Q^T), kept in registers for the whole kernel
  bf16x8 qf[8];
  {
    int row = q0 + l32;
    row = row < a.Sq ? row : a.Sq - 1;
    const __bf16* p = qp + (int64_t)row * a.q_ss + hh * 8;
#pragma unroll
    for (int s = 0; s < 8; ++s) qf[s] = *reinterpret_cast<const bf16x8*>(p + s * 16);
  }

  // ---- direct global -> LDS loads of one ring slot: K(kt) and V(kt-1).  Wave w fills the row groups
  // w, w+NW, ...  Rows outside the sequence re-read the nearest valid row: they only ever meet masked
  // logits / zero probabilities, but must be finite.  Tiles that lie fully inside the sequence use a
  // uniform base plus a lane offset that never changes.
  const int grow = lane >> 4;                                  // row of the group this lane fills
  const int kcol = ((lane & 15) ^ grow) * 8;                   // K: logical chunk stored at this lane's position
  const int vcol = ((lane & 15) ^ (grow << 2)) * 8;            // V: same, segments permuted instead of chunks
  const unsigned kofs = (unsigned)(grow * (int)a.k_ss + kcol) * 2u;    // bytes
  const unsigned vofs = (unsigned)(grow * (int)a.v_ss + vcol) * 2u;
  const unsigned smem_addr = lds_addr_of(smem);
  auto dma = [&](int slot, int kt) __attribute__((always_inline)) {
    const unsigned Ks = smem_addr + (unsigned)(slot * kStage) * 2u;
    const unsigned Vs = Ks + kKTile * 2u;
    if (kt >= 1 && kt * kBN + kBN <= a.Skv) {
      const __bf16* kt0 = kp + (int64_t)(kt * kBN + 4 * wave) * a.k_ss;
      const __bf16* vt0 = vp + (int64_t)((kt - 1) * kBN + 4 * wave) * a.v_ss;
#pragma unroll
      for (int i = 0; i < 16 / NW; ++i) {
        lds_dma16(kt0 + (int64_t)(4 * NW * i) * a.k_ss, kofs, Ks + (unsigned)((wave + NW * i) * kGK) * 2u);
        lds_dma16(vt0 + (int64_t)(4 * NW * i) * a.v_ss, vofs, Vs + (unsigned)((wave + NW * i) * kGV) * 2u);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 16 / NW; ++i) {
        const int g = wave + NW * i;
        int kk = kt * kBN + 4 * g + grow;
        kk = kk < a.Skv ? kk : a.Skv - 1;
        int kvv = (kt - 1) * kBN + 4 * g + grow;
        kvv = kvv < a.Skv ? kvv : a.Skv - 1;
        kvv = kvv > 0 ? kvv : 0;
        lds_dma16(kp + (int64_t)kk * a.k_ss + kcol, Ks + (unsigned)(g * kGK) * 2u);
        lds_dma16(vp + (int64_t)kvv * a.v_ss + vcol, Vs + (unsigned)(g * kGV) * 2u);
      }
    }
  };
  dma(0, 0);
  dma(1, 1);
  dma(2, 2);

  f32x16 O[4];
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) O[db][i] = 0.f;
  float m = -1e30f, l = 0.f;
  float mc = PRE ? 0.f : m * c;  // the rows' reference point in log2 units
  // PRE (scale * log2(e) == 1: the caller's q already carries the factor): the logits need no multiply, and the
  // reference point is subtracted by the MFMA itself, as the start value of every QK accumulator chain.  The
  // first key block then always takes the cold branch, which puts the reference at that block's maximum.
  f32x16 negm;
#pragma unroll
  for (int i = 0; i < 16; ++i) negm[i] = 0.f;

  // lane-constant LDS offsets
  // K fragment j (logical chunk 2j + hh) of row l32 sits at chunk position (2j + hh) ^ (l32 & 3): pair j ^ x1,
  // half hh ^ x0.  Even and odd j get a base each, so that the rest of the offset is a compile-time constant.
  const int kx0 = l32 & 1, kx1 = (l32 >> 1) & 1;
  const int k_base = (l32 >> 2) * kGK + (l32 & 3) * kD + (hh ^ kx0) * 8;
  const int k_off_e = k_base + 16 * kx1, k_off_o = k_base - 16 * kx1;
  // V fragment jv: segment s = jv & 3 of row group 4*(jv >> 2) + hh, row xr of the group; one base per segment
  const int vxr = (lane & 15) >> 2;
  int v_off[4];
#pragma unroll
  for (int sg = 0; sg < 4; ++sg)
    v_off[sg] = kKTile + hh * kGV + vxr * kD + (sg ^ vxr) * 32 + ((lane >> 4) & 1) * 16 + 4 * (lane & 3);

  f32x16 Sa, Sb;        // logits of odd / even blocks
  u32x4 Pa[2], Pb[2];   // probabilities of odd / even blocks (PV B-operand layout, 16 keys each), bf16 pairs
  bf16x8 kfr[4], vfr[4];  // rotating fragment windows
#pragma unroll
  for (int i = 0; i < 16; ++i) { Sa[i] = -INFINITY; Sb[i] = 0.f; }  // block -1: fully masked
#pragma unroll
  for (int i = 0; i < 2; ++i) { Pa[i] = u32x4{0u, 0u, 0u, 0u}; Pb[i] = Pa[i]; }

  // One iteration.  SC holds the logits of block BLK; SN receives those of block BLK+1.
  // KC/KN: K rows of block BLK+1 / BLK+2; VC/VN: V rows of block BLK-1 / BLK.
  // Slot n of the stream: n even -> PV MFMA n/2, n odd -> QK MFMA n/2, each followed by the LDS
  // request for the next MFMA of the same kind, then a share of the softmax of block BLK.  The vector
  // ALU issues through the same port as the MFMAs, so the hot stream carries the bare minimum per pair of
  // logits: two FMAs (none when PRE), two exp2, two adds for the f32 row sum and one bf16 pack.  There is no row
  // max in it: a row's reference point m moves only when a 16-key partial sum of P exceeds kTrig, which also
  // catches the +inf that the first block of a row produces from m = -1e30.  A triggered wave (every row's first
  // block, then almost never) redoes the block's softmax from the logits with the true maximum in a cold branch
  // at the end of the iteration, where no PV MFMA of the previous block is outstanding.
  // The softmax starts at slot kS0: the last QK MFMA of block BLK was issued at slot 15 of the
  // previous iteration, and reading its result earlier stalls the wave's whole stream.
#define MDATTN_ITER(SC, SN, PC, PP, KC, KN, VC, VN, BLK) /* KC.. : base pointers [even j, odd j]; VC.. : [segment] */                                                     \
  {                                                                                                           \
    float lsum = 0.f, pe = 0.f;                                                                               \
    if ((BLK) * 32 + 32 > a.Skv) { /* ragged tail and the virtual blocks past the end: -inf logits */         \
      asm volatile("" ::: "memory");                                                                          \
      const int kv_base = (BLK) * 32 + 4 * hh;                                                                \
      _Pragma("unroll") for (int i = 0; i < 16; ++i)                                                          \
        if (kv_base + 8 * (i >> 2) + (i & 3) >= a.Skv) SC[i] = -INFINITY;                                     \
    }                                                                                                         \
    _Pragma("unroll") for (int n = 0; n < 16; ++n) {                                                          \
      const int j = n >> 1, jn = j + kLA;                                                                     \
      if ((n & 1) == 0) {                                                                                     \
        O[j & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vfr[j & 3], __builtin_bit_cast(bf16x8, PP[j >> 2]), O[j & 3], 0, 0, 0); \
        const __bf16* vsrc = (jn < 8 ? (VC) : (VN))[jn & 3] + ((jn & 7) >> 2) * 4 * kGV;                      \
        vfr[jn & 3] = read_vt(vsrc, vsrc + 2 * kGV);                                                          \
      } else {                                                                                                \
        if (j == 0) {                                                                                         \
          f32x16 z;                                                                                           \
          _Pragma("unroll") for (int i = 0; i < 16; ++i) z[i] = 0.f;                                          \
          SN = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kfr[0], qf[0], PRE ? negm : z, 0, 0, 0);               \
        } else {                                                                                              \
          SN = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kfr[j & 3], qf[j], SN, 0, 0, 0);                       \
        }                                                                                                     \
        kfr[jn & 3] = *reinterpret_cast<const bf16x8*>((jn < 8 ? (KC) : (KN))[jn & 1] + (jn & 7) * 16);       \
      }                                                                                                       \
      const int e0 = n < kS0 ? 0 : ((n - kS0) * 16) / (16 - kS0);                                             \
      const int e1 = n < kS0 ? 0 : ((n + 1 - kS0) * 16) / (16 - kS0);                                         \
      _Pragma("unroll") for (int e = 0; e < 16; ++e) {                                                        \
        if (e >= e0 && e < e1) {                                                                              \
          const float x = __builtin_amdgcn_exp2f(PRE ? SC[e] : __builtin_fmaf(SC[e], c, -mc));                \
          if ((e & 1) == 0) {                                                                                 \
            pe = x;                                                                                           \
            /* pins the work in its slot: otherwise the compiler sinks the softmax below the MFMA stream */  \
            asm volatile("" : "+v"(pe));                                                                      \
          } else {                                                                                            \
            unsigned pk = pack2(pe, x);                                                                       \
            lsum = e == 1 ? pe + x : lsum + (pe + x); /* no add of the initial zero */                        \
            asm volatile("" : "+v"(pk), "+v"(lsum));                                                          \
            PC[e >> 3][(e >> 1) & 3] = pk;                                                                    \
          }                                                                                                   \
        }                                                                                                     \
      }                                                                                                       \
      __builtin_amdgcn_sched_barrier(0);                                                                      \
    }                                                                                                         \
    if (__builtin_expect(__builtin_amdgcn_ballot_w64(!(lsum <= kTrig)) != 0 || (PRE && (BLK) == 0), 0)) {     \
      float mloc = SC[0];                                                                                     \
      _Pragma("unroll") for (int i = 1; i < 16; ++i) mloc = fmaxf(mloc, SC[i]);                               \
      mloc = xhalf_max(mloc);                                                                                 \
      /* every row of a triggered wave moves to its true maximum: right after, the block's sum is at most */  \
      /* 16, so a row can trigger again only when its maximum has grown by another 20 log2 units          */  \
      float alpha;                                                                                            \
      if (PRE) { /* SC and SN hold logits minus the old reference: shift them, and the chains' start value */ \
        const float dm = (BLK) == 0 ? mloc : fmaxf(mloc, 0.f);                                                \
        alpha = (BLK) == 0 ? 0.f : __builtin_amdgcn_exp2f(-dm);                                               \
        mc += dm;                                                                                             \
        _Pragma("unroll") for (int i = 0; i < 16; ++i) { SC[i] -= dm; SN[i] -= dm; negm[i] -= dm; }           \
      } else {                                                                                                \
        const float mnew = fmaxf(m, mloc);                                                                    \
        alpha = __builtin_amdgcn_exp2f((m - mnew) * c); /* exactly 1 for rows that keep m */                  \
        m = mnew;                                                                                             \
        mc = m * c;                                                                                           \
      }                                                                                                       \
      lsum = 0.f;                                                                                             \
      _Pragma("unroll") for (int e = 0; e < 16; e += 2) {                                                     \
        const float x0 = __builtin_amdgcn_exp2f(PRE ? SC[e] : __builtin_fmaf(SC[e], c, -mc));                 \
        const float x1 = __builtin_amdgcn_exp2f(PRE ? SC[e + 1] : __builtin_fmaf(SC[e + 1], c, -mc));         \
        lsum += x0 + x1;                                                                                      \
        PC[e >> 3][(e >> 1) & 3] = pack2(x0, x1);                                                             \
      }                                                                                                       \
      l *= alpha;                                                                                             \
      _Pragma("unroll") for (int db = 0; db < 4; ++db)                                                        \
        _Pragma("unroll") for (int i = 0; i < 16; ++i) O[db][i] *= alpha;                                     \
    }                                                                                                         \
    l += lsum;                                                                                                \
  }

  // ring bookkeeping: period t uses slot t%4 (K(t), V(t-1)) and looks ahead into slot (t+1)%4.  The loop over periods is
  // unrolled four times, one copy per ring slot, so that every fragment address is a lane constant plus a compile-time
  // offset: the stream carries no address arithmetic.
  // fragments the first iteration's first QK / PV MFMA expect in the windows
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): Q fragments and this wave's share of slots 0..2
  __syncthreads();
#pragma unroll
  for (int s = 0; s < kLA; ++s) {
    kfr[s] = *reinterpret_cast<const bf16x8*>(smem + ((s & 1) ? k_off_o : k_off_e) + s * 16);
    const __bf16* vsrc = smem + v_off[s];
    vfr[s] = read_vt(vsrc, vsrc + 2 * kGV);
  }
  const int nfull = a.Skv / kBN;  // tiles that lie fully inside the sequence
  const __bf16* kdma = kp + (int64_t)(3 * kBN + 4 * wave) * a.k_ss;  // this wave's first row group of K(t+3) ...
  const __bf16* vdma = vp + (int64_t)(2 * kBN + 4 * wave) * a.v_ss;  // ... and of V(t+2)
  unsigned kofs_i[16 / NW], vofs_i[16 / NW];                          // lane offsets of its further row groups
#pragma unroll
  for (int i = 0; i < 16 / NW; ++i) {
    kofs_i[i] = kofs + (unsigned)(4 * NW * i * (int)a.k_ss) * 2u;
    vofs_i[i] = vofs + (unsigned)(4 * NW * i * (int)a.v_ss) * 2u;
  }
  auto period = [&](int t, auto slot_c) __attribute__((always_inline)) {
    constexpr int s_cur = decltype(slot_c)::value, s_nxt = (s_cur + 1) & 3, s_fill = (s_cur + 3) & 3;
    // every wave's loads into slot s_nxt (issued two periods ago) have landed once all waves pass the
    // barrier: only the loads of the previous period (2 * 16 / NW per wave) may still be in flight.
    // Slot s_fill was last read in period t-1 and now receives K(t+3), V(t+2).
    __builtin_amdgcn_s_waitcnt(0x0F70 | (32 / NW));
    __syncthreads();
    const __bf16* cur = smem + s_cur * kStage;
    const __bf16* nxt = smem + s_nxt * kStage;
    const __bf16* Kc0[2] = {cur + k_off_e, cur + k_off_o};
    const __bf16* Kc1[2] = {Kc0[0] + 8 * kGK, Kc0[1] + 8 * kGK};
    const __bf16* Kn0[2] = {nxt + k_off_e, nxt + k_off_o};
    const __bf16* Vc0[4] = {cur + v_off[0], cur + v_off[1], cur + v_off[2], cur + v_off[3]};
    const __bf16* Vc1[4] = {Vc0[0] + 8 * kGV, Vc0[1] + 8 * kGV, Vc0[2] + 8 * kGV, Vc0[3] + 8 * kGV};
    const __bf16* Vn0[4] = {nxt + v_off[0], nxt + v_off[1], nxt + v_off[2], nxt + v_off[3]};
    // iteration 2t-1: softmax(2t-1), PV(2t-2), QK(2t)
    MDATTN_ITER(Sa, Sb, Pa, Pb, Kc0, Kc1, Vc0, Vc1, 2 * t - 1)
    // K(t+3) and V(t+2) into slot s_fill, issued here rather than right after the barrier (where all eight
    // waves would queue their loads before their first MFMA).  Tiles inside the sequence: running pointers
    // and constant lane offsets, a handful of scalar instructions per load.
    if (t + 3 < nfull) {
      const unsigned Ks = smem_addr + (unsigned)(s_fill * kStage + wave * kGK) * 2u;
      const unsigned Vs = smem_addr + (unsigned)(s_fill * kStage + kKTile + wave * kGV) * 2u;
#pragma unroll
      for (int i = 0; i < 16 / NW; ++i) {
        lds_dma16(kdma, kofs_i[i], Ks + (unsigned)(NW * i * kGK) * 2u);
        lds_dma16(vdma, vofs_i[i], Vs + (unsigned)(NW * i * kGV) * 2u);
      }
    } else {
      dma(s_fill, t + 3);
    }
    kdma += kBN * a.k_ss;
    vdma += kBN * a.v_ss;
    // iteration 2t: softmax(2t), PV(2t-1), QK(2t+1)
    MDATTN_ITER(Sb, Sa, Pb, Pa, Kc1, Kn0, Vc1, Vn0, 2 * t)
  };
  for (int t = 0; t <= nt; t += 4) {
    period(t, std::integral_constant<int, 0>{});
    if (t + 1 > nt) break;
    period(t + 1, std::integral_constant<int, 1>{});
    if (t + 2 > nt) break;
    period(t + 2, std::integral_constant<int, 2>{});
    if (t + 3 > nt) break;
    period(t + 3, std::integral_constant<int, 3>{});
  }
#undef MDATTN_ITER

  // ---- epilogue: normalise, convert, store; lse = m*scale + ln(l)
  store_row<4>(a, O, xhalf_sum(l), mc, b, h, q0 + l32, hh);
}

#ifndef MDATTN_FLAT_PAIRWISE
#define MDATTN_FLAT_PAIRWISE 1
#endif
#ifndef MDATTN_FLAT_LA128
#define MDATTN_FLAT_LA128 2
#endif
// ---------------------------------------------------------------------------------------------------
// Second schedule: no software pipelining inside a wave.  Four waves per workgroup, 32-key tiles in a
// 3-slot ring (50 KB of LDS) and at most 168 VGPRs, so that three workgroups share a CU and three waves
// share each SIMD: while one wave runs its softmax on the vector ALU the other two keep the matrix
// pipe busy.  Same tile layouts, same fragment reads, same arithmetic as the pipelined kernel.
// Head dim 64 (template HD) uses 128-byte rows: one load instruction fills 8 rows, K chunk c of row r sits at
// position c ^ ((r >> 1) & 7), V chunk c at c ^ 4*((r >> 1) & 1), both unpadded and conflict-free for the
// same two read patterns; its 104-128 VGPRs and 32 KB of LDS (64-key tiles, two 32-key blocks per slot, in a 2-slot
// ring) let four workgroups share a CU (four waves per SIMD: 3 % faster than three at 32 heads x 13,376 tokens, where
// the softmax per MFMA FLOP is twice that of head dim 128).
constexpr int kTS = 32;                               // keys per tile
constexpr int kKTileS = (kTS / 4) * kGK;              // elements
constexpr int kStageS = kKTileS + (kTS / 4) * kGV;    // elements per ring slot
constexpr int kSlotsS = 3;

template <int NW, bool BIAS, int HD, bool PRE>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(HD == 64 ? 4 : 3, HD == 64 ? 4 : 3))) void attn_fwd_bf16_flat_kernel(AttnArgs a) {
  constexpr int NJ = HD / 16;                                    // QK MFMAs per 32-key tile
  constexpr int ND = HD / 32;                                    // 32-wide slabs of d = O accumulators
  // Head dim 64: 64-key tiles (two 32-key blocks per ring slot, the LDS of a 32-key tile at head dim 128) in a 2-slot
  // ring: half the barriers and tile bookkeeping per key of a kernel whose softmax already outweighs its MFMAs.
  constexpr int TS = HD == 128 ? kTS : 64;                       // keys per tile
  constexpr int NB = TS / 32;                                    // 32-key blocks per tile
  constexpr int SLOTS = HD == 128 ? kSlotsS : 2;
  constexpr int KTILE = HD == 128 ? kKTileS : TS * 64;           // elements
  constexpr int QTILE = HD == 128 ? kKTileS : 32 * 64;           // a wave's 32 Q rows, staged like a K tile
  constexpr int TILES = HD == 128 ? kStageS : 2 * TS * 64;       // the K and the V tile of a slot
  // with a bias, a slot also carries the tile's 32 bias values (f32) behind its tiles: a register load inside the
  // loop would be waited for in issue order, i.e. behind the loads of the tile after next
  constexpr int STAGE = TILES + (BIAS ? 128 : 0);  // 64 floats: one per lane of the load that brings them
  constexpr int RPI = HD == 128 ? 4 : 8;                          // rows one load instruction fills
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  __bf16* smem = reinterpret_cast<__bf16*>(smem_raw);
  constexpr int BM = NW * 32;
  constexpr int GPW = (TS / RPI) / NW;  // row groups per wave, tile and tensor

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, hh = lane >> 5;

  const int wg = blockIdx.x;
  const int w = (wg & 7) * a.chunk + (wg >> 3);
  if (w >= a.total) return;
  const int bh = w / a.nqt, qt = w - bh * a.nqt;
  const int b = bh / a.H, h = bh - b * a.H;

  const __bf16* qp = a.q + b * a.q_sb + h * a.q_sh;
  const __bf16* kp = a.k + b * a.k_sb + h * a.k_sh;
  const __bf16* vp = a.v + b * a.v_sb + h * a.v_sh;
  const int q0 = qt * BM + wave * 32;
  const int nt = (a.Skv + TS - 1) / TS;
  const float c = a.c;
  // with a bias the logits are brought to log2 units (scale folded, bias added) right after the MFMAs
  const float cs = BIAS ? 1.0f : c;
  const float* bias_row = BIAS ? a.bias + b * a.bias_sb : nullptr;
  [[maybe_unused]] const int bias_cols = (a.Skv + 31) / 32 * 32;  // entries the caller's bias rows are sure to hold

  bf16x8 qf[NJ];  // filled from LDS below: the wave's 32 Q rows arrive like a K tile, by whole-row loads

  // lane -> (row of the group, logical 16-byte chunk stored at this lane's position)
  const int grow = HD == 128 ? lane >> 4 : lane >> 3;
  const int kcol = HD == 128 ? ((lane & 15) ^ grow) * 8 : ((lane & 7) ^ ((4 * (wave & 1) + (grow >> 1)) & 7)) * 8;
  const int vcol = HD == 128 ? ((lane & 15) ^ (grow << 2)) * 8 : ((lane & 7) ^ (((grow >> 1) & 1) << 2)) * 8;
  constexpr int KGS = HD == 128 ? kGK : 8 * 64;  // group strides in LDS, elements
  constexpr int VGS = HD == 128 ? kGV : 8 * 64;
  const unsigned kofs = (unsigned)(grow * (int)a.k_ss + kcol) * 2u;
  const unsigned vofs = (unsigned)(grow * (int)a.v_ss + vcol) * 2u;
  const unsigned smem_addr = lds_addr_of(smem);
  auto dma = [&](int slot, int kt) __attribute__((always_inline)) {
    const unsigned Ks = smem_addr + (unsigned)(slot * STAGE) * 2u;
    const unsigned Vs = Ks + KTILE * 2u;
    // every wave fetches the same values to the same place (a load more per wave and tile, counted in the loop's
    // s_waitcnt): lane l and lane l + 32 the bias of key l of the tile; the ring runs up to two tiles past the end
    if constexpr (BIAS) {  // (a 64-key tile may reach past the padded bias row, whose length is a multiple of 32)
      int col = (kt < nt ? kt : nt - 1) * TS + (TS == 64 ? lane : l32);
      col = col < bias_cols ? col : bias_cols - 1;
      lds_dma4(bias_row, (unsigned)col * 4u, Ks + TILES * 2u);
    }
    if (kt * TS + TS <= a.Skv) {
      const __bf16* kt0 = kp + (int64_t)(kt * TS + RPI * wave) * a.k_ss;
      const __bf16* vt0 = vp + (int64_t)(kt * TS + RPI * wave) * a.v_ss;
#pragma unroll
      for (int i = 0; i < GPW; ++i) {
        lds_dma16(kt0 + (int64_t)(RPI * NW * i) * a.k_ss, kofs, Ks + (unsigned)((wave + NW * i) * KGS) * 2u);
        lds_dma16(vt0 + (int64_t)(RPI * NW * i) * a.v_ss, vofs, Vs + (unsigned)((wave + NW * i) * VGS) * 2u);
      }
    } else {
#pragma unroll
      for (int i = 0; i < GPW; ++i) {
        const int g = wave + NW * i;
        int kk = kt * TS + RPI * g + grow;
        kk = kk < a.Skv ? kk : a.Skv - 1;
        lds_dma16(kp + (int64_t)kk * a.k_ss + kcol, Ks + (unsigned)(g * KGS) * 2u);
        lds_dma16(vp + (int64_t)kk * a.v_ss + vcol, Vs + (unsigned)(g * VGS) * 2u);
      }
    }
  };

  f32x16 O[ND];
#pragma unroll
  for (int db = 0; db < ND; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) O[db][i] = 0.f;
  float m = -1e30f, l = 0.f;
  float mc = PRE ? 0.f : m * cs;  // the rows' reference point in log2 units
  f32x16 negm;                    // PRE (see the pipelined kernel): start value of every score accumulator chain
#pragma unroll
  for (int i = 0; i < 16; ++i) negm[i] = 0.f;

  // per-lane fragment offsets (elements): K fragment j, V slab sg; kV8 = offset of the second transposing read
  // (rows + 8), kVH = offset of the second 16-key half of the tile
  const int vxr = (lane & 15) >> 2;
  int k_off[NJ], v_off[ND];
  constexpr int kV8 = HD == 128 ? 2 * kGV : 8 * 64, kVH = HD == 128 ? 4 * kGV : 16 * 64;
  if constexpr (HD == 128) {
    const int kx0 = l32 & 1, kx1 = (l32 >> 1) & 1;
    const int k_base = (l32 >> 2) * kGK + (l32 & 3) * kD + (hh ^ kx0) * 8;
#pragma unroll
    for (int j = 0; j < NJ; ++j) k_off[j] = k_base + ((j & 1) ? -16 : 16) * kx1 + j * 16;
#pragma unroll
    for (int sg = 0; sg < ND; ++sg)
      v_off[sg] = KTILE + hh * kGV + vxr * kD + (sg ^ vxr) * 32 + ((lane >> 4) & 1) * 16 + 4 * (lane & 3);
  } else {
    const int kx = (l32 >> 1) & 7, vx = (vxr >> 1) & 1;
#pragma unroll
    for (int j = 0; j < NJ; ++j) k_off[j] = l32 * 64 + (((2 * j + hh) ^ kx) * 8);
#pragma unroll
    for (int sg = 0; sg < ND; ++sg)
      v_off[sg] = KTILE + (4 * hh + vxr) * 64 + (sg ^ vx) * 32 + ((lane >> 4) & 1) * 16 + 4 * (lane & 3);
  }

  // A tile's fragment reads as one stream (per 32-key block: NJ row reads of K, then 2*ND transposing reads of V) with a
  // window of LA fragments running ahead of the MFMAs, pinned by scheduling barriers: left to itself the compiler
  // waits for every read right before its MFMA.
  constexpr int LA = HD == 128 ? MDATTN_FLAT_LA128 : 0;
  constexpr int FPB = NJ + 2 * ND, NFRAG = NB * FPB;
  auto tile = [&](int t, auto slot, auto masked) __attribute__((always_inline)) {  // slot: int or integral_constant
    const __bf16* base = smem + slot * STAGE;
    constexpr int kBlk = 32 * 64;  // a 32-key block of a head-dim-64 tile: 32 rows of 64 elements, in K and in V
    auto frag = [&](int n) __attribute__((always_inline)) {
      const int fb = n / FPB, r = n % FPB;
      if (r < NJ) return *reinterpret_cast<const bf16x8*>(base + k_off[r] + fb * kBlk);
      const __bf16* vsrc = base + v_off[(r - NJ) % ND] + ((r - NJ) / ND) * kVH + fb * kBlk;
      return read_vt(vsrc, vsrc + kV8);
    };
    [[maybe_unused]] bf16x8 win[LA > 0 ? LA : 1];
    if constexpr (LA > 0) {
#pragma unroll
      for (int n = 0; n < LA; ++n) win[n] = frag(n);
    }
#pragma unroll
   for (int blk = 0; blk < NB; ++blk) {
    const bool first = t == 0 && blk == 0;
    // ---- S^T = K.Q^T: one chain of MFMAs; the other waves of the SIMD fill the gaps between them.  A wave in an
    // MFMA phase issues ahead of the SIMD's waves in their softmax phase (1-2 % on short key sequences).
    __builtin_amdgcn_s_setprio(1);
    f32x16 S;
#pragma unroll
    for (int i = 0; i < 16; ++i) S[i] = 0.f;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      if constexpr (LA > 0) {
        const int n = blk * FPB + j;
        S = __builtin_amdgcn_mfma_f32_32x32x16_bf16(win[n % LA], qf[j], (PRE && j == 0) ? negm : S, 0, 0, 0);
        if (n + LA < NFRAG) win[n % LA] = frag(n + LA);
        __builtin_amdgcn_sched_barrier(0);
      } else {
        const bf16x8 kf = *reinterpret_cast<const bf16x8*>(base + k_off[j] + blk * kBlk);
        S = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[j], (PRE && j == 0) ? negm : S, 0, 0, 0);
      }
    }
    if constexpr (BIAS) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const f32x4 bv = *reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(base + TILES) + 32 * blk + 8 * g + 4 * hh);
#pragma unroll
        for (int e = 0; e < 4; ++e) S[4 * g + e] = __builtin_fmaf(S[4 * g + e], c, bv[e] * kLog2e);
      }
    }
    if constexpr (decltype(masked)::value) {
      const int kv_base = t * TS + 32 * blk + 4 * hh;
#pragma unroll
      for (int i = 0; i < 16; ++i)
        if (kv_base + 8 * (i >> 2) + (i & 3) >= a.Skv) S[i] = -INFINITY;
    }
    // ---- online softmax.  The hot path takes no row maximum: P and its sum are formed against the row's
    // current reference point, and only a partial sum above kTrig (a logit far above the reference, or
    // many a little above) sends the wave through the branch that moves every row's reference to its true
    // maximum, rescales the accumulators and redoes the tile's P.
    __builtin_amdgcn_s_setprio(0);
    bf16x8 P[2];
    auto soft = [&](float rf) __attribute__((always_inline)) {
      float lsum = 0.f;
#pragma unroll
      for (int hb = 0; hb < 2; ++hb) {
#if MDATTN_FLAT_PAIRWISE
        // two logits at a time, packed as soon as they exist: 16 f32 probabilities never live at once, which is what
        // leaves this kernel registers for a fragment window
        unsigned pk[4];
#pragma unroll
        for (int e = 0; e < 8; e += 2) {
          const float x0 = __builtin_amdgcn_exp2f(PRE ? S[8 * hb + e] : __builtin_fmaf(S[8 * hb + e], cs, -rf));
          const float x1 = __builtin_amdgcn_exp2f(PRE ? S[8 * hb + e + 1] : __builtin_fmaf(S[8 * hb + e + 1], cs, -rf));
          lsum = (hb == 0 && e == 0) ? x0 : lsum + x0;  // no add of the initial zero
          lsum += x1;
          pk[e >> 1] = pack2(x0, x1);
          asm volatile("" : "+v"(pk[e >> 1]), "+v"(lsum));
        }
        P[hb] = __builtin_bit_cast(bf16x8, u32x4{pk[0], pk[1], pk[2], pk[3]});
#else
        float p[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          p[e] = __builtin_amdgcn_exp2f(PRE ? S[8 * hb + e] : __builtin_fmaf(S[8 * hb + e], cs, -rf));
          lsum += p[e];
        }
        P[hb] = __builtin_bit_cast(bf16x8, pack8(p));
#endif
      }
      return lsum;
    };
    float lsum = soft(mc);
    if (__builtin_expect(__builtin_amdgcn_ballot_w64(!(lsum <= kTrig)) != 0 || (PRE && first), 0)) {
      float mloc = S[0];
#pragma unroll
      for (int i = 1; i < 16; ++i) mloc = fmaxf(mloc, S[i]);
      mloc = xhalf_max(mloc);
      float alpha;
      if constexpr (PRE) {  // S holds logits minus the old reference: shift them and the chains' start value
        const float dm = first ? mloc : fmaxf(mloc, 0.f);
        alpha = first ? 0.f : __builtin_amdgcn_exp2f(-dm);
        mc += dm;
#pragma unroll
        for (int i = 0; i < 16; ++i) { S[i] -= dm; negm[i] -= dm; }
      } else {
        const float mnew = fmaxf(m, mloc);
        alpha = __builtin_amdgcn_exp2f((m - mnew) * cs);
        m = mnew;
        mc = m * cs;
      }
      asm volatile("" : "+v"(alpha));  // keeps the rescale inside this rarely taken branch
      l *= alpha;
#pragma unroll
      for (int db = 0; db < ND; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) O[db][i] *= alpha;
      lsum = soft(mc);
    }
    l += lsum;
    __builtin_amdgcn_s_setprio(1);
    // ---- O^T += V^T.P^T
#pragma unroll
    for (int jv = 0; jv < 2 * ND; ++jv) {
      if constexpr (LA > 0) {
        const int n = blk * FPB + NJ + jv;
        O[jv % ND] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(win[n % LA], P[jv / ND], O[jv % ND], 0, 0, 0);
        if (n + LA < NFRAG) win[n % LA] = frag(n + LA);
        __builtin_amdgcn_sched_barrier(0);
      } else {
        const __bf16* vsrc = base + v_off[jv % ND] + (jv / ND) * kVH + blk * kBlk;
        const bf16x8 vf = read_vt(vsrc, vsrc + kV8);
        O[jv % ND] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, P[jv / ND], O[jv % ND], 0, 0, 0);
      }
    }
   }
  };

  // ---- Q fragments.  A lane's registers hold 16-byte pieces of ONE row, so loading them straight from global memory
  // makes every load instruction touch 32 rows, 32 bytes of each (75,600 x 40 rows: 0.1-0.17 ms per launch).  Instead
  // the wave fetches its 32 rows as a K-shaped tile with the same direct global->LDS loads (whole 256-byte rows per
  // 16 lanes), into a staging area behind ring slot 0 (which receives key tile 0 meanwhile), and reads the fragments
  // with the K fragment offsets.  Each wave stages and reads only its own rows.
  dma(0, 0);
  {
    const unsigned Qs = smem_addr + (unsigned)(STAGE + wave * QTILE) * 2u;
#pragma unroll
    for (int g = 0; g < 32 / RPI; ++g) {
      int row = q0 + RPI * g + grow;
      row = row < a.Sq ? row : a.Sq - 1;
      const int qcol = HD == 128 ? kcol : ((lane & 7) ^ ((4 * (g & 1) + (grow >> 1)) & 7)) * 8;
      lds_dma16(qp + (int64_t)row * a.q_ss + qcol, Qs + (unsigned)(g * KGS) * 2u);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the wave's own Q rows (and its share of tile 0) are in LDS
    const __bf16* qs = smem + STAGE + wave * QTILE;
#pragma unroll
    for (int j = 0; j < NJ; ++j) qf[j] = *reinterpret_cast<const bf16x8*>(qs + k_off[j]);
  }
  __syncthreads();  // every wave holds its fragments: the staging area is ring slots again
  // SLOTS - 1 tiles are requested ahead of the one being worked on
#pragma unroll
  for (int i = 1; i < SLOTS - 1; ++i) dma(i, i);
  auto step = [&](int t, auto slot, int fill) __attribute__((always_inline)) {
    // vmcnt: this wave's share of tile t has landed (the SLOTS - 2 tiles requested after it may still be in flight)
    __builtin_amdgcn_s_waitcnt(0x0F70 | ((SLOTS - 2) * (2 * GPW + (BIAS ? 1 : 0))));
    __syncthreads();                                  // ... and everyone's; slot `fill` (tile t-1) is free
    dma(fill, t + SLOTS - 1);
    tile(t, slot, std::false_type{});
  };
  if constexpr (HD == 64) {
    // Two copies of the loop body, one per ring slot: the slot is a compile-time constant in each, every fragment
    // address a lane constant plus an immediate offset, and the address arithmetic per tile is gone from a kernel that
    // is bound by vector issue (1 % at 32 heads x 13,376 tokens; at head dim 128 the copies cost registers and lose).
    for (int t = 0; t < nt - 1; t += 2) {
      step(t, std::integral_constant<int, 0>{}, 1);
      if (t + 1 >= nt - 1) break;
      step(t + 1, std::integral_constant<int, 1>{}, 0);
    }
  } else {
    int slot = 0, fill = SLOTS - 1;
    for (int t = 0; t < nt - 1; ++t) {
      step(t, slot, fill);
      slot = slot == SLOTS - 1 ? 0 : slot + 1;
      fill = fill == SLOTS - 1 ? 0 : fill + 1;
    }
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();
  tile(nt - 1, (nt - 1) % SLOTS, std::true_type{});

  if (a.o_run) {  // ring step: merged into the f32 carry, row by row
    store_row<ND>(a, O, xhalf_sum(l), mc, b, h, q0 + l32, hh);
  } else {
    static_assert(NW * 32 * (HD * 2 + 16) <= SLOTS * STAGE * 2, "the output staging tiles must fit the ring's LDS");
    __syncthreads();  // every wave has finished reading the ring: its LDS now stages the output tiles
    store_rows_through_lds<ND>(a, O, xhalf_sum(l), mc, b, h, q0, lane, smem_raw + wave * 32 * (HD * 2 + 16));
  }
}

template <int NW, bool BIAS, int HD = 128>
static int launch_flat(hipStream_t st, AttnArgs a, int B) {
  constexpr int BM = NW * 32;
  // the ring, or ring slot 0 plus one K-shaped Q staging tile per wave, whichever is larger
  constexpr int slots = HD == 128 ? kSlotsS : 2;
  constexpr int stage_el = (HD == 128 ? kStageS : 2 * 64 * 64) + (BIAS ? 128 : 0), qtile_el = HD == 128 ? kKTileS : 32 * 64;
  constexpr int lds_bytes = (slots * stage_el > stage_el + NW * qtile_el ? slots * stage_el : stage_el + NW * qtile_el) * 2;
  a.nqt = (a.Sq + BM - 1) / BM;
  const int64_t total = (int64_t)B * a.H * a.nqt;
  if (total > (int64_t)0x7FFFFFF0) return MDATTN_E_UNSUPPORTED;
  a.total = (int)total;
  a.chunk = (a.total + 7) / 8;
  // scale * log2(e) == 1 (to f32 round-off): the caller folded the factor into q; the logits need no multiply.
  // With a key bias the logits are touched after the MFMAs anyway, so that variant keeps its FMA.
  const bool pre = !BIAS && a.c > 1.0f - 1e-6f && a.c < 1.0f + 1e-6f;
  if (pre) MDATTN_LAUNCH((attn_fwd_bf16_flat_kernel<NW, BIAS, HD, !BIAS>), dim3(a.chunk * 8), dim3(NW * 64), lds_bytes, st, a);
  else MDATTN_LAUNCH((attn_fwd_bf16_flat_kernel<NW, BIAS, HD, false>), dim3(a.chunk * 8), dim3(NW * 64), lds_bytes, st, a);
  return launch_status();
}

template <int NW>
static int launch_fwd(hipStream_t st, AttnArgs a, int B) {
  constexpr int BM = NW * 32;
  constexpr int lds_bytes = 4 * kStage * 2;
  a.nqt = (a.Sq + BM - 1) / BM;
  const int64_t total = (int64_t)B * a.H * a.nqt;
  if (total > (int64_t)0x7FFFFFF0) return MDATTN_E_UNSUPPORTED;
  a.total = (int)total;
  a.chunk = (a.total + 7) / 8;
  // scale * log2(e) == 1 (to f32 round-off): the caller folded the factor into q; the logits need no multiply
  const bool pre = a.c > 1.0f - 1e-6f && a.c < 1.0f + 1e-6f;
  auto kern = pre ? attn_fwd_bf16_kernel<NW, true> : attn_fwd_bf16_kernel<NW, false>;
  static LdsOptIn opted[2];
  if (lds_opt_in(opted[pre], reinterpret_cast<const void*>(kern), lds_bytes) != MDATTN_OK) return MDATTN_E_LAUNCH;
  MDATTN_LAUNCH(kern, dim3(a.chunk * 8), dim3(NW * 64), lds_bytes, st, a);
  return launch_status();
}

}  // namespace mdattn

using namespace mdattn;

static int fill_args(AttnArgs& a, const void* q, const void* k, const void* v, void* out, float* lse,
                     int B, int H, int Sq, int Skv, int D,
                     const mdattn_strides* q_strides, const mdattn_strides* k_strides,
                     const mdattn_strides* v_strides, const mdattn_strides* o_strides, float scale) {
  if (!q || !k || !v || !out || B <= 0 || H <= 0 || Sq <= 0 || Skv <= 0 || D <= 0) return MDATTN_E_BADARG;
  if (!q_strides || !k_strides || !v_strides || !o_strides) return MDATTN_E_BADARG;
  if (!(scale > 0.f) || !(scale < 1e30f)) return MDATTN_E_BADARG;
  if (D != kD && D != 64) return MDATTN_E_UNSUPPORTED;
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(out) || (reinterpret_cast<uintptr_t>(lse) & 3u))
    return MDATTN_E_ALIGN;
  if (!strides_ok(q_strides, 8) || !strides_ok(k_strides, 8) || !strides_ok(v_strides, 8) || !strides_ok(o_strides, 8))
    return MDATTN_E_ALIGN;
  if (q_strides->seq < D || k_strides->seq < D || v_strides->seq < D || o_strides->seq < D) return MDATTN_E_BADARG;
  // per-lane byte offsets inside one tile are kept in 32 bits
  if (k_strides->seq >= (1 << 23) || v_strides->seq >= (1 << 23)) return MDATTN_E_UNSUPPORTED;
  a.q = (const __bf16*)q; a.k = (const __bf16*)k; a.v = (const __bf16*)v; a.out = (__bf16*)out; a.lse = lse;
  a.H = H; a.Sq = Sq; a.Skv = Skv;
  a.q_sb = q_strides->batch; a.q_ss = q_strides->seq; a.q_sh = q_strides->head;
  a.k_sb = k_strides->batch; a.k_ss = k_strides->seq; a.k_sh = k_strides->head;
  a.v_sb = v_strides->batch; a.v_ss = v_strides->seq; a.v_sh = v_strides->head;
  a.o_sb = o_strides->batch; a.o_ss = o_strides->seq; a.o_sh = o_strides->head;
  a.c = scale * kLog2e;
  a.bias = nullptr; a.bias_sb = 0;
  a.o_run = nullptr; a.lse_run = nullptr;
  return MDATTN_OK;
}

static int dispatch_fwd(hipStream_t st, const AttnArgs& a, int B, int Sq, int Skv, int D) {
  if (D == 64) return launch_flat<4, false, 64>(st, a, B);  // head dim 64: the flat schedule only

  // Two schedules.  The software-pipelined kernel (8 waves x 32 query rows, two waves per SIMD) is the faster one
  // on long key sequences; its prologue and epilogue (three tiles of look-ahead, one virtual block at each end)
  // weigh on short ones, where the flat kernel (4 waves x 32 rows, three workgroups per CU) wins: measured
  // cross-over between 2048 and 4608 keys.  The flat kernel also yields twice the workgroups on tiny grids.
  // mdattn_set_fwd_schedule (1: pipelined 8 waves, 2: pipelined 4 waves, 3: flat) overrides the choice, for tests.
  int variant = forced_fwd_schedule();
  if (variant == 0) {
    const int64_t wg256 = (int64_t)B * a.H * ((Sq + 255) / 256);
    variant = (Skv <= 3072 || wg256 < 128) ? 3 : 1;
  }
  switch (variant) {
    case 1: return launch_fwd<8>(st, a, B);
    case 2: return launch_fwd<4>(st, a, B);
    case 3: return launch_flat<4, false>(st, a, B);
    default: return MDATTN_E_BADARG;
  }
}

extern "C" int mdattn_fwd_bf16(void* stream, const void* q, const void* k, const void* v, void* out, float* lse,
                               int B, int H, int Sq, int Skv, int D,
                               const mdattn_strides* q_strides, const mdattn_strides* k_strides,
                               const mdattn_strides* v_strides, const mdattn_strides* o_strides, float scale) {
  AttnArgs a;
  const int rc = fill_args(a, q, k, v, out, lse, B, H, Sq, Skv, D, q_strides, k_strides, v_strides, o_strides, scale);
  if (rc != MDATTN_OK) return rc;
  return dispatch_fwd((hipStream_t)stream, a, B, Sq, Skv, D);
}

extern "C" int mdattn_fwd_bf16_merge(void* stream, const void* q, const void* k, const void* v, float* o_run, float* lse_run,
                                     int B, int H, int Sq, int Skv, int D,
                                     const mdattn_strides* q_strides, const mdattn_strides* k_strides,
                                     const mdattn_strides* v_strides, const mdattn_strides* run_strides, float scale) {
  if (!o_run || !lse_run) return MDATTN_E_BADARG;
  if (reinterpret_cast<uintptr_t>(lse_run) & 3u) return MDATTN_E_ALIGN;
  AttnArgs a;
  // o_run stands in for `out` in the checks (16-byte alignment, strides in elements, multiples of 8)
  const int rc = fill_args(a, q, k, v, o_run, nullptr, B, H, Sq, Skv, D, q_strides, k_strides, v_strides, run_strides, scale);
  if (rc != MDATTN_OK) return rc;
  a.out = nullptr;
  a.o_run = o_run;
  a.lse_run = lse_run;
  return dispatch_fwd((hipStream_t)stream, a, B, Sq, Skv, D);
}

extern "C" int mdattn_fwd_bf16_bias(void* stream, const void* q, const void* k, const void* v, void* out, float* lse,
                                    int B, int H, int Sq, int Skv, int D,
                                    const mdattn_strides* q_strides, const mdattn_strides* k_strides,
                                    const mdattn_strides* v_strides, const mdattn_strides* o_strides, float scale,
                                    const float* key_bias, int64_t bias_stride) {
  AttnArgs a;
  const int rc = fill_args(a, q, k, v, out, lse, B, H, Sq, Skv, D, q_strides, k_strides, v_strides, o_strides, scale);
  if (rc != MDATTN_OK) return rc;
  if (!key_bias || bias_stride < ((Skv + kTS - 1) / kTS) * kTS || bias_stride % kTS != 0) return MDATTN_E_BADARG;
  if (!aligned16(key_bias)) return MDATTN_E_ALIGN;
  a.bias = key_bias;
  a.bias_sb = bias_stride;
  if (D == 64) return launch_flat<4, true, 64>((hipStream_t)stream, a, B);
  return launch_flat<4, true>((hipStream_t)stream, a, B);
}
