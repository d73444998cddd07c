// Backward of the non-causal attention forward for gfx950 (MI355X), bf16 MFMA, head_dim 128: dq, dk, dv from
// (q, k, v, out, dout, lse).  With logits s = scale*q.k, p = exp(s - lse), dp = dout.v^T, delta = rowsum(dout*out):
//   dv = p^T dout,   ds = p * (dp - delta),   dq = scale * ds k,   dk = scale * ds^T q.
//
// One kernel body, two passes, no atomics: every gradient is accumulated by the waves that own its rows.
//   dq pass:      "entity" rows = 32 q rows per wave (q and dout fragments in registers), "stream" rows = keys
//                 (k for the scores and for the accumulation, v for dP).
//   dk / dv pass: entity rows = 32 key rows per wave (k and v fragments in registers), stream rows = q rows (q for
//                 the scores and the dk accumulation, dout for dP and the dv accumulation).  S^T and dP^T are formed
//                 once per tile; P feeds the dv accumulators and dS the dk ones: seven matrix products per call
//                 where five are necessary (S and dP are formed in both passes).
// Stream rows are walked in tiles of 32 through a 2-slot LDS ring filled by direct global->LDS loads.
// Per tile, with the forward kernel's layouts and fragment reads:
//   S^T  = stream1 . entity1^T      (A = tile rows by ds_read_b128, B = entity fragments)   lane = entity row
//   dP^T = stream2 . entity2^T
//   W    = exp2(c*S - lse*log2e) [* (dP - delta)]     f32, packed to bf16 in B-operand order (the factor `scale` of
//                                                      dS is applied once, to the finished accumulators)
//   acc^T += stream3^T . W          (A = the tile through the transposing LDS read)
// lse and delta belong to the q rows: per-lane scalars for dq; for dk / dv sixteen values per lane and tile, which
// ride through the ring next to the tile (a register load inside the loop would be waited for in issue order, i.e.
// behind the next tile's loads).  They come from a workspace that a small kernel fills first (-delta and -lse in log2
// units, padded to a multiple of 32 rows with -lse = -inf so that padded q rows get p = 0).  Both are stored negated
// because they start the MFMA chains they are subtracted from: dP^T - delta comes out of the chain, and so does
// S^T - lse when the caller's q already carries scale * log2(e) (the factor c is then 1).
#include <atomic>
#include <mutex>

#include "mdattn_common.h"

namespace mdattn {
namespace {

constexpr int kBT = 32;                  // stream rows per tile
// Tile layouts of the forward's flat schedule (see attn_fwd_bf16.hip).  Head dim 128: groups of 4 rows, row-read
// layout padded by 64 B per group (chunk c of row r at c ^ (r & 3)), transposed-read layout with 64-byte segments at
// s ^ (r & 3).  Head dim 64 (LTX-2's audio stream): 128-byte rows, groups of 8 rows, chunk c at c ^ ((r >> 1) & 7) for
// the row reads and at c ^ 4*((r >> 1) & 1) for the transposing reads, both unpadded.
template <int HD>
struct BwdLayout {
  static constexpr int RPI = HD == 128 ? 4 : 8;                          // rows one load instruction fills
  static constexpr int GA = HD == 128 ? 4 * 128 + 32 : 8 * 64;           // group stride, row-read layout (elements)
  static constexpr int GB = HD == 128 ? 4 * 128 : 8 * 64;                // group stride, transposed-read layout
  static constexpr int TileA = (kBT / RPI) * GA;
  static constexpr int TileB = (kBT / RPI) * GB;
  static constexpr int Stage = 2 * TileA + TileB;                        // elements per ring slot
  static constexpr int V8 = HD == 128 ? 2 * GB : 8 * 64;                 // second transposing read: rows + 8
  static constexpr int VH = HD == 128 ? 4 * GB : 16 * 64;                // second 16-row half of the tile
};

// Per-row f32 values of a stream tile (lse and delta of its q rows, or the bias of its keys) travel through the ring as
// well: 64 floats behind the tiles of a slot.
constexpr int kAuxFloats = 64;
template <int MODE, int HD, bool BIAS>
constexpr int bwd_slot_elems() {  // bf16 elements per ring slot
  return BwdLayout<HD>::Stage + (MODE == 3 ? BwdLayout<HD>::TileB : 0) + ((MODE != 0 || BIAS) ? 2 * kAuxFloats : 0);
}

// Waves per workgroup, 32 entity rows each.  Head dim 128: eight, one workgroup per CU at two waves per SIMD, so that
// the CU's eight waves share one stream ring (half the global->LDS traffic of two workgroups of four; 3-6 % faster).
// Head dim 64: four, three workgroups per CU.
template <int HD>
constexpr int bwd_waves() { return HD == 128 ? 8 : 4; }

typedef s16x4 __attribute__((address_space(3))) * lds_s16x4_ptr_b;
typedef __attribute__((ext_vector_type(8))) short s16x8_b;

__device__ __forceinline__ bf16x8 read_vt_b(const __bf16* p0, const __bf16* p1) {
  s16x4 r0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr_b)p0);
  s16x4 r1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr_b)p1);
  s16x8_b r = __builtin_shufflevector(r0, r1, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(bf16x8, r);
}

struct BwdArgs {
  const __bf16* e1;  // entity tensor of the score contraction
  const __bf16* e2;  // entity tensor of the dP contraction (unused for dv)
  const __bf16* s1;  // stream tensor of the score contraction
  const __bf16* s2;  // stream tensor of the dP contraction (unused for dv)
  const __bf16* s3;  // stream tensor the gradient accumulates with
  __bf16* out;       // gradient of the entity rows
  const __bf16* s4;  // MODE 3: second stream tensor to accumulate with (dout, for dv); s3 is q (for dk)
  __bf16* out2;      // MODE 3: dv
  int64_t s4_sb, s4_ss, s4_sh, o2_sb, o2_ss, o2_sh;
  const float* lse2;   // [B,H,Sp] -lse * log2(e), -inf on padded rows
  const float* delta;  // [B,H,Sp] -rowsum(dout * out)
  int H, Se, Ss, Sp;
  int net, total, chunk;
  int64_t e1_sb, e1_ss, e1_sh, e2_sb, e2_ss, e2_sh;
  int64_t s1_sb, s1_ss, s1_sh, s2_sb, s2_ss, s2_sh, s3_sb, s3_ss, s3_sh;
  int64_t o_sb, o_ss, o_sh;
  float c, scale;
  const float* bias;   // BIAS: additive per-key bias [B, bias_sb] in natural-log units (mdattn_fwd_bf16_bias)
  int64_t bias_sb;
};

// MODE 0: dq (entity = q rows, stream = keys); 3: dk and dv in one pass (entity = key rows, stream = q rows).
// MODE 1 (dk alone) and 2 (dv alone) are the same body with one accumulator set; the library launches 0 and 3.
template <int MODE, int HD, bool BIAS, bool PRE>
__device__ __forceinline__ void attn_bwd_body(const BwdArgs& a) {
  static_assert(!(PRE && BIAS), "a biased logit is touched after the MFMAs anyway");
  extern __shared__ __attribute__((aligned(16))) char smem_raw_b[];
  __bf16* smem = reinterpret_cast<__bf16*>(smem_raw_b);
  constexpr int NW = bwd_waves<HD>();
  constexpr bool HAS2 = MODE != 2;
  constexpr bool BOTH = MODE == 3;
  using L = BwdLayout<HD>;
  constexpr int NJ = HD / 16;   // MFMAs per 32 x 32 block of a contraction over the head dim
  constexpr int ND = HD / 32;   // 32-wide slabs of d = accumulators
  constexpr int kBD = HD, kBGK = L::GA, kBGV = L::GB, kBTileA = L::TileA, kBTileB = L::TileB;
  constexpr int kBStage = bwd_slot_elems<MODE, HD, BIAS>();  // MODE 3: a second transposed-read tile (dout)
  constexpr bool AUX = MODE != 0 || BIAS;
#ifndef MDATTN_BWD_LA
#define MDATTN_BWD_LA 4
#endif
  // fragment look-ahead of the dq pass over its whole read stream (head dim 64, at three waves per SIMD, has room for
  // two: 1 % on one machine, A/B); the merged pass windows its two MFMA phases separately, LA1 and LA3 below
  constexpr int LA = MODE == 0 ? (HD == 128 ? MDATTN_BWD_LA : 2) : 0;
  static_assert(LA == 0 || (HAS2 && !BOTH && LA <= 2 * ND), "the window covers the three-product passes");
#ifndef MDATTN_BWD_LA1
#define MDATTN_BWD_LA1 2
#endif
#ifndef MDATTN_BWD_LA3
#define MDATTN_BWD_LA3 6
#endif
  constexpr int LA3 = BOTH && HD == 128 ? (BIAS ? 4 : MDATTN_BWD_LA3) : 0;
  constexpr int LA1 = BOTH && HD == 128 ? MDATTN_BWD_LA1 : 0;  // merged pass: look-ahead over the chains' row reads only
  constexpr int kBAux = L::Stage + (BOTH ? L::TileB : 0);    // where a slot's f32 values start (elements)

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, hh = lane >> 5;

  const int wg = blockIdx.x;
  const int w = (wg & 7) * a.chunk + (wg >> 3);
  if (w >= a.total) return;
  const int bh = w / a.net, et = w - bh * a.net;
  const int b = bh / a.H, h = bh - b * a.H;
  const int r0 = et * (NW * 32) + wave * 32;
  const int nt = (a.Ss + kBT - 1) / kBT;
  const float c = a.c;

  // ---- entity fragments
  int erow = r0 + l32;
  erow = erow < a.Se ? erow : a.Se - 1;
  bf16x8 ef1[NJ], ef2[NJ];
  {
    const __bf16* p = a.e1 + b * a.e1_sb + h * a.e1_sh + (int64_t)erow * a.e1_ss + hh * 8;
#pragma unroll
    for (int s = 0; s < NJ; ++s) ef1[s] = *reinterpret_cast<const bf16x8*>(p + s * 16);
    if constexpr (HAS2) {
      const __bf16* p2 = a.e2 + b * a.e2_sb + h * a.e2_sh + (int64_t)erow * a.e2_ss + hh * 8;
#pragma unroll
      for (int s = 0; s < NJ; ++s) ef2[s] = *reinterpret_cast<const bf16x8*>(p2 + s * 16);
    }
  }
  const float* lrow = a.lse2 + ((int64_t)b * a.H + h) * a.Sp;
  const float* drow = a.delta + ((int64_t)b * a.H + h) * a.Sp;
  float nlse_e = 0.f, ndelta_e = 0.f;  // the workspace holds both negated
  if constexpr (MODE == 0) {
    nlse_e = lrow[erow];
    ndelta_e = drow[erow];
  }
  // key bias in log2 units: a per-lane scalar when the keys are the entity rows, sixteen values per tile otherwise
  [[maybe_unused]] const float* bias_row = BIAS ? a.bias + b * a.bias_sb : nullptr;
  [[maybe_unused]] float bias_e = 0.f;
  if constexpr (BIAS && MODE != 0) bias_e = bias_row[erow] * kLog2e;

  // ---- direct global -> LDS loads of one stream tile (layouts and lane maps of the forward kernel)
  const __bf16* s1p = a.s1 + b * a.s1_sb + h * a.s1_sh;
  const __bf16* s2p = HAS2 ? a.s2 + b * a.s2_sb + h * a.s2_sh : nullptr;
  const __bf16* s3p = a.s3 + b * a.s3_sb + h * a.s3_sh;
  [[maybe_unused]] const __bf16* s4p = BOTH ? a.s4 + b * a.s4_sb + h * a.s4_sh : nullptr;
  constexpr int RPI = L::RPI;
  const int grow = HD == 128 ? lane >> 4 : lane >> 3;
  // lane -> logical 16-byte chunk stored at this lane's position (a wave fills the row groups wave, wave + NW, ...)
  const int acol = HD == 128 ? ((lane & 15) ^ grow) * 8 : ((lane & 7) ^ ((4 * (wave & 1) + (grow >> 1)) & 7)) * 8;
  const int bcol = HD == 128 ? ((lane & 15) ^ (grow << 2)) * 8 : ((lane & 7) ^ (((grow >> 1) & 1) << 2)) * 8;
  const unsigned smem_addr = lds_addr_of(smem);
  // byte offsets of this lane's chunk from the first row of its row group: the same for every full tile.  The merged
  // pass at head dim 128 has no registers to keep them in (spilled, every reload would wait for the load issued
  // before it): it forms them again per tile from the lane number, a dozen full-rate instructions.
  constexpr bool REFORM = BOTH && HD == 128;
  auto chunk_ofs = [&](int ln, int64_t ss, bool transposed) __attribute__((always_inline)) {
    const int gr = HD == 128 ? ln >> 4 : ln >> 3;
    const int col = transposed ? (HD == 128 ? ((ln & 15) ^ (gr << 2)) * 8 : ((ln & 7) ^ (((gr >> 1) & 1) << 2)) * 8)
                               : (HD == 128 ? ((ln & 15) ^ gr) * 8 : ((ln & 7) ^ ((4 * (wave & 1) + (gr >> 1)) & 7)) * 8);
    return (__umul24((unsigned)gr, (unsigned)ss) + (unsigned)col) * 2u;  // strides are below 2^23
  };
  [[maybe_unused]] const unsigned ofs1 = REFORM ? 0u : chunk_ofs(lane, a.s1_ss, false);
  [[maybe_unused]] const unsigned ofs2 = HAS2 && !REFORM ? chunk_ofs(lane, a.s2_ss, false) : 0u;
  [[maybe_unused]] const unsigned ofs3 = REFORM ? 0u : chunk_ofs(lane, a.s3_ss, true);
  [[maybe_unused]] const unsigned ofs4 = BOTH && !REFORM ? chunk_ofs(lane, a.s4_ss, true) : 0u;
  // wave 0 brings a tile's f32 values: lanes 0-31 the lse of its 32 q rows and lanes 32-63 their delta, or (dq pass)
  // every lane the bias of key lane % 32.  Through LDS because a register load here would be waited for in order
  // behind the next tile's loads.
  [[maybe_unused]] const unsigned ofs_aux =
      MODE != 0 ? (lane < 32 ? 0u : (unsigned)((a.delta - a.lse2) * 4)) + (unsigned)l32 * 4u : (unsigned)l32 * 4u;
  auto dma = [&](int slot, int t) __attribute__((always_inline)) {
    const unsigned A1 = smem_addr + (unsigned)(slot * kBStage) * 2u;
    const unsigned A2 = A1 + kBTileA * 2u;
    const unsigned Bt = A2 + kBTileA * 2u;
    if constexpr (AUX) {
      if (wave == 0) {
        unsigned oa = ofs_aux;
        if constexpr (REFORM) {
          int ln = lane;
          asm volatile("" : "+v"(ln));
          oa = (ln < 32 ? 0u : (unsigned)((a.delta - a.lse2) * 4)) + (unsigned)(ln & 31) * 4u;
        }
        lds_dma4((MODE != 0 ? lrow : bias_row) + t * kBT, oa, A1 + kBAux * 2u);
      }
    }
    if (t * kBT + kBT <= a.Ss) {  // a full tile: uniform row-group bases, one per-lane offset per stream
      unsigned o1 = ofs1, o2 = ofs2, o3 = ofs3, o4 = ofs4;
      if constexpr (REFORM) {
        int ln = lane;
        asm volatile("" : "+v"(ln));  // opaque: keeps the four offsets from being hoisted out of the loop
        o1 = chunk_ofs(ln, a.s1_ss, false);
        o2 = chunk_ofs(ln, a.s2_ss, false);
        o3 = chunk_ofs(ln, a.s3_ss, true);
        o4 = chunk_ofs(ln, a.s4_ss, true);
      }
#pragma unroll
      for (int i = 0; i < (kBT / RPI) / NW; ++i) {
        const int g = wave + NW * i;
        const int64_t r = t * kBT + RPI * g;
        lds_dma16(s1p + r * a.s1_ss, o1, A1 + (unsigned)(g * kBGK) * 2u);
        if constexpr (HAS2) lds_dma16(s2p + r * a.s2_ss, o2, A2 + (unsigned)(g * kBGK) * 2u);
        lds_dma16(s3p + r * a.s3_ss, o3, Bt + (unsigned)(g * kBGV) * 2u);
        if constexpr (BOTH) lds_dma16(s4p + r * a.s4_ss, o4, Bt + (unsigned)(kBTileB + g * kBGV) * 2u);
      }
    } else {  // the ragged last tile: rows past the end repeat the last row
#pragma unroll
      for (int i = 0; i < (kBT / RPI) / NW; ++i) {
        const int g = wave + NW * i;
        int rr = t * kBT + RPI * g + grow;
        rr = rr < a.Ss ? rr : a.Ss - 1;
        lds_dma16(s1p + (int64_t)rr * a.s1_ss + acol, A1 + (unsigned)(g * kBGK) * 2u);
        if constexpr (HAS2) lds_dma16(s2p + (int64_t)rr * a.s2_ss + acol, A2 + (unsigned)(g * kBGK) * 2u);
        lds_dma16(s3p + (int64_t)rr * a.s3_ss + bcol, Bt + (unsigned)(g * kBGV) * 2u);
        if constexpr (BOTH) lds_dma16(s4p + (int64_t)rr * a.s4_ss + bcol, Bt + (unsigned)(kBTileB + g * kBGV) * 2u);
      }
    }
  };

  f32x16 acc[ND];
  [[maybe_unused]] f32x16 acc2[BOTH ? ND : 1];  // MODE 3: dv next to dk
#pragma unroll
  for (int db = 0; db < ND; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      acc[db][i] = 0.f;
      if constexpr (BOTH) acc2[db][i] = 0.f;
    }

  // per-lane fragment offsets (elements)
  int k_off[NJ], v_off[ND];
  const int vxr = (lane & 15) >> 2;
  if constexpr (HD == 128) {
    const int kx0 = l32 & 1, kx1 = (l32 >> 1) & 1;
    const int k_base = (l32 >> 2) * kBGK + (l32 & 3) * kBD + (hh ^ kx0) * 8;
#pragma unroll
    for (int j = 0; j < NJ; ++j) k_off[j] = k_base + ((j & 1) ? -16 : 16) * kx1 + j * 16;
#pragma unroll
    for (int sg = 0; sg < ND; ++sg)
      v_off[sg] = 2 * kBTileA + hh * kBGV + vxr * kBD + (sg ^ vxr) * 32 + ((lane >> 4) & 1) * 16 + 4 * (lane & 3);
  } else {
    const int kx = (l32 >> 1) & 7, vx = (vxr >> 1) & 1;
#pragma unroll
    for (int j = 0; j < NJ; ++j) k_off[j] = l32 * 64 + (((2 * j + hh) ^ kx) * 8);
#pragma unroll
    for (int sg = 0; sg < ND; ++sg)
      v_off[sg] = 2 * kBTileA + (4 * hh + vxr) * 64 + (sg ^ vx) * 32 + ((lane >> 4) & 1) * 16 + 4 * (lane & 3);
  }

  dma(0, 0);
  for (int t = 0; t < nt; ++t) {
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's share of tile t has landed
    __syncthreads();                      // ... and everyone's; the other slot (tile t-1) is free
    if (t + 1 < nt) dma((t + 1) & 1, t + 1);
    const __bf16* base = smem + (t & 1) * kBStage;

    // Start values of the two MFMA chains: -delta for dP^T, so that the chain ends on dP - delta; and, when the
    // logits come out of the MFMAs in log2 units (PRE), -lse for S^T, so that exp2 applies to the chain's result
    // as it is.  Per-lane constants when the q rows are the entity rows, the tile's values from LDS otherwise.
    [[maybe_unused]] const float* aux = reinterpret_cast<const float*>(base + kBAux);
    f32x16 S, dP;
    if constexpr (MODE == 0) {
#pragma unroll
      for (int i = 0; i < 16; ++i) { S[i] = PRE ? nlse_e : 0.f; dP[i] = ndelta_e; }
    } else {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const f32x4 dv = *reinterpret_cast<const f32x4*>(aux + 32 + 8 * g + 4 * hh);
#pragma unroll
        for (int e = 0; e < 4; ++e) dP[4 * g + e] = dv[e];
        if constexpr (PRE) {
          const f32x4 lv = *reinterpret_cast<const f32x4*>(aux + 8 * g + 4 * hh);
#pragma unroll
          for (int e = 0; e < 4; ++e) S[4 * g + e] = lv[e];
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) S[4 * g + e] = 0.f;
        }
      }
    }
    // The tile's fragment reads as one stream: NJ row reads for S^T, NJ for dP^T, then the 2*ND transposing reads
    // of the accumulation.  With LA > 0 a window of LA fragments runs ahead of the MFMAs (pinned by scheduling
    // barriers: left to itself the compiler waits for every read right before its MFMA).
    auto frag = [&](int n) __attribute__((always_inline)) {
      if (n < NJ) return *reinterpret_cast<const bf16x8*>(base + k_off[n]);
      if (n < 2 * NJ) return *reinterpret_cast<const bf16x8*>(base + kBTileA + k_off[n - NJ]);
      const int jv = n - 2 * NJ;
      const __bf16* src = base + v_off[jv % ND] + (jv / ND) * L::VH;
      return read_vt_b(src, src + L::V8);
    };
    [[maybe_unused]] bf16x8 win[LA > 0 ? LA : 1];
    if constexpr (LA > 0) {
#pragma unroll
      for (int n = 0; n < LA; ++n) win[n] = frag(n);
#pragma unroll
      for (int n = 0; n < 2 * NJ; ++n) {
        if (n < NJ) S = __builtin_amdgcn_mfma_f32_32x32x16_bf16(win[n % LA], ef1[n % NJ], S, 0, 0, 0);
        else dP = __builtin_amdgcn_mfma_f32_32x32x16_bf16(win[n % LA], ef2[n % NJ], dP, 0, 0, 0);
        win[n % LA] = frag(n + LA);
        __builtin_amdgcn_sched_barrier(0);
      }
    } else if constexpr (LA1 > 0) {  // a window over the row reads of the two chains only
      bf16x8 w1[LA1];
#pragma unroll
      for (int n = 0; n < LA1; ++n) w1[n] = frag(n);
#pragma unroll
      for (int n = 0; n < 2 * NJ; ++n) {
        if (n < NJ) S = __builtin_amdgcn_mfma_f32_32x32x16_bf16(w1[n % LA1], ef1[n % NJ], S, 0, 0, 0);
        else dP = __builtin_amdgcn_mfma_f32_32x32x16_bf16(w1[n % LA1], ef2[n % NJ], dP, 0, 0, 0);
        if (n + LA1 < 2 * NJ) w1[n % LA1] = frag(n + LA1);
        __builtin_amdgcn_sched_barrier(0);
      }
    } else {
#pragma unroll
      for (int j = 0; j < NJ; ++j) S = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag(j), ef1[j], S, 0, 0, 0);
      if constexpr (HAS2) {
#pragma unroll
        for (int j = 0; j < NJ; ++j) dP = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag(NJ + j), ef2[j], dP, 0, 0, 0);
      }
    }
    // W = P or dS, eight logits (one B operand) at a time
    if constexpr (MODE == 0) {
      if (t == nt - 1) {  // keys past the end of a ragged last tile take no part
        const int sbase = t * kBT + 4 * hh;
#pragma unroll
        for (int i = 0; i < 16; ++i)
          if (sbase + 8 * (i >> 2) + (i & 3) >= a.Ss) S[i] = -INFINITY;
      }
    }
    bf16x8 W[2];
    [[maybe_unused]] bf16x8 Wp[2];  // MODE 3: the probabilities themselves, for dv
#pragma unroll
    for (int hb = 0; hb < 2; ++hb) {
      [[maybe_unused]] float nl[8];  // -lse (log2 units) of each logit's q row, with the key's bias added
      if constexpr (!PRE) {
        if constexpr (MODE == 0) {
#pragma unroll
          for (int e = 0; e < 8; ++e) nl[e] = nlse_e;
          if constexpr (BIAS) {
#pragma unroll
            for (int g = 0; g < 2; ++g) {
              const int col = t * kBT + 8 * (2 * hb + g) + 4 * hh;
              const f32x4 bv = *reinterpret_cast<const f32x4*>(aux + 8 * (2 * hb + g) + 4 * hh);
#pragma unroll
              for (int e = 0; e < 4; ++e)
                nl[4 * g + e] = col + e < a.Ss ? __builtin_fmaf(bv[e], kLog2e, nlse_e) : -INFINITY;  // whatever the padding holds
            }
          }
        } else {
#pragma unroll
          for (int g = 0; g < 2; ++g) {
            const f32x4 lv = *reinterpret_cast<const f32x4*>(aux + 8 * (2 * hb + g) + 4 * hh);
#pragma unroll
            for (int e = 0; e < 4; ++e) nl[4 * g + e] = BIAS ? lv[e] + bias_e : lv[e];
          }
        }
      }
      unsigned wpk[4];
      [[maybe_unused]] unsigned ppk[4];
#pragma unroll
      for (int e = 0; e < 8; e += 2) {
        const float p0 = __builtin_amdgcn_exp2f(PRE ? S[8 * hb + e] : __builtin_fmaf(S[8 * hb + e], c, nl[e]));
        const float p1 = __builtin_amdgcn_exp2f(PRE ? S[8 * hb + e + 1] : __builtin_fmaf(S[8 * hb + e + 1], c, nl[e + 1]));
        // dS without its factor `scale`: applied once, to the accumulators
        wpk[e >> 1] = HAS2 ? pack2(p0 * dP[8 * hb + e], p1 * dP[8 * hb + e + 1]) : pack2(p0, p1);
        if constexpr (BOTH) ppk[e >> 1] = pack2(p0, p1);
      }
      W[hb] = __builtin_bit_cast(bf16x8, u32x4{wpk[0], wpk[1], wpk[2], wpk[3]});
      if constexpr (BOTH) Wp[hb] = __builtin_bit_cast(bf16x8, u32x4{ppk[0], ppk[1], ppk[2], ppk[3]});
    }
    if constexpr (LA3 > 0) {  // merged pass: a window over the transposing reads of both accumulations
      auto frag3 = [&](int n) __attribute__((always_inline)) {
        const int jv = n >> 1;
        const __bf16* src = base + v_off[jv % ND] + (jv / ND) * L::VH + ((n & 1) ? kBTileB : 0);
        return read_vt_b(src, src + L::V8);
      };
      bf16x8 w3[LA3];
#pragma unroll
      for (int n = 0; n < LA3; ++n) w3[n] = frag3(n);
#pragma unroll
      for (int n = 0; n < 4 * ND; ++n) {
        const int jv = n >> 1;
        if (n & 1) acc2[jv % ND] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(w3[n % LA3], Wp[jv / ND], acc2[jv % ND], 0, 0, 0);
        else acc[jv % ND] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(w3[n % LA3], W[jv / ND], acc[jv % ND], 0, 0, 0);
        if (n + LA3 < 4 * ND) w3[n % LA3] = frag3(n + LA3);
        __builtin_amdgcn_sched_barrier(0);
      }
    } else
#pragma unroll
    for (int jv = 0; jv < 2 * ND; ++jv) {
      const __bf16* src = base + v_off[jv % ND] + (jv / ND) * L::VH;
      if constexpr (LA > 0) {
        acc[jv % ND] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(win[(2 * NJ + jv) % LA], W[jv / ND], acc[jv % ND], 0, 0, 0);
        if (jv + LA < 2 * ND) win[(2 * NJ + jv) % LA] = frag(2 * NJ + jv + LA);
        __builtin_amdgcn_sched_barrier(0);
        continue;
      }
      const bf16x8 f = read_vt_b(src, src + L::V8);
      acc[jv % ND] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f, W[jv / ND], acc[jv % ND], 0, 0, 0);
      if constexpr (BOTH) {
        const bf16x8 f2 = read_vt_b(src + kBTileB, src + kBTileB + L::V8);
        acc2[jv % ND] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f2, Wp[jv / ND], acc2[jv % ND], 0, 0, 0);
      }
    }
  }

  const int row = r0 + l32;
  const float osc = HAS2 ? a.scale : 1.0f;  // dq = scale * dS k, dk = scale * dS^T q
  if (row < a.Se) {
    __bf16* orow = a.out + b * a.o_sb + h * a.o_sh + (int64_t)row * a.o_ss + 4 * hh;
#pragma unroll
    for (int db = 0; db < ND; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        uint2 u;
        u.x = pack2(acc[db][4 * g] * osc, acc[db][4 * g + 1] * osc);
        u.y = pack2(acc[db][4 * g + 2] * osc, acc[db][4 * g + 3] * osc);
        *reinterpret_cast<uint2*>(orow + db * 32 + 8 * g) = u;
      }
    if constexpr (BOTH) {
      __bf16* orow2 = a.out2 + b * a.o2_sb + h * a.o2_sh + (int64_t)row * a.o2_ss + 4 * hh;
#pragma unroll
      for (int db = 0; db < ND; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          uint2 u;
          u.x = pack2(acc2[db][4 * g], acc2[db][4 * g + 1]);
          u.y = pack2(acc2[db][4 * g + 2], acc2[db][4 * g + 3]);
          *reinterpret_cast<uint2*>(orow2 + db * 32 + 8 * g) = u;
        }
    }
  }
}

template <int MODE, int HD, bool BIAS, bool PRE>
__global__ __launch_bounds__((bwd_waves<HD>() * 64)) void attn_bwd_kernel(BwdArgs a) {
  attn_bwd_body<MODE, HD, BIAS, PRE>(a);
}
// The dk / dv pass at head dim 128 wants a few registers more than half the register file (128 accumulators, 64 of
// entity fragments, 32 of S and dP): held to two waves per SIMD, which the schedule needs to overlap one wave's
// exponentials with the other's MFMAs; at one wave per SIMD it measured 28 % slower.  Head dim 64 fits three waves
// per SIMD (3 % faster than two).
template <int HD, bool BIAS, bool PRE>
__global__ __launch_bounds__((bwd_waves<HD>() * 64)) __attribute__((amdgpu_waves_per_eu(HD == 64 ? 3 : 2, HD == 64 ? 3 : 2))) void attn_bwd_both_kernel(BwdArgs a) {
  attn_bwd_body<3, HD, BIAS, PRE>(a);
}

// The workspace, both negated (they start the MFMA chains that they are subtracted from):
// delta[b,h,q] = -sum_d dout*out, lse2 = -lse*log2(e); rows q in [Sq, Sp) get delta 0, lse2 -inf.  16 lanes per row
// (head dim 64: the upper 8 stay idle).
__global__ __launch_bounds__(256) void bwd_prep_kernel(const __bf16* out, const __bf16* dout, const float* lse,
                                                       float* lse2, float* delta, int H, int Sq, int Sp, int D,
                                                       int64_t rows, int64_t o_sb, int64_t o_ss, int64_t o_sh) {
  const int64_t r = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
  if (r >= rows) return;
  const int lane = threadIdx.x & 15;
  const int q = (int)(r % Sp);
  const int64_t bh = r / Sp;
  const int h = (int)(bh % H);
  const int64_t b = bh / H;
  float acc = 0.f;
  if (q < Sq && lane * 8 < D) {
    const int64_t off = b * o_sb + (int64_t)q * o_ss + h * o_sh + lane * 8;
    float x[8], y[8];
    unpack8(*reinterpret_cast<const uint4*>(out + off), x);
    unpack8(*reinterpret_cast<const uint4*>(dout + off), y);
#pragma unroll
    for (int j = 0; j < 8; ++j) acc = __builtin_fmaf(x[j], y[j], acc);
  }
  acc = row16_sum(acc);
  if (lane == 0) {
    delta[r] = q < Sq ? -acc : 0.f;
    // padded rows, and rows whose keys were all masked (the forward wrote lse = -inf, out = 0), take no part: p = 0
    const float lv = q < Sq ? lse[bh * Sq + q] : -INFINITY;
    lse2[r] = lv > -INFINITY ? -lv * kLog2e : -INFINITY;
  }
}

template <int MODE, int HD, bool BIAS, bool PRE>
int launch_bwd_as(hipStream_t st, BwdArgs a, int B) {
  constexpr int lds_bytes = 2 * bwd_slot_elems<MODE, HD, BIAS>() * 2;
  constexpr int NW = bwd_waves<HD>();
  a.net = (a.Se + NW * 32 - 1) / (NW * 32);
  const int64_t total = (int64_t)B * a.H * a.net;
  if (total > (int64_t)0x7FFFFFF0) return MDATTN_E_UNSUPPORTED;
  a.total = (int)total;
  a.chunk = (a.total + 7) / 8;
  void (*kern)(BwdArgs);
  if constexpr (MODE == 3) kern = attn_bwd_both_kernel<HD, BIAS, PRE>;
  else kern = attn_bwd_kernel<MODE, HD, BIAS, PRE>;
  static LdsOptIn opted;
  if (lds_opt_in(opted, reinterpret_cast<const void*>(kern), lds_bytes) != MDATTN_OK) return MDATTN_E_LAUNCH;
  MDATTN_LAUNCH(kern, dim3(a.chunk * 8), dim3(NW * 64), lds_bytes, st, a);
  return launch_status();
}

// scale * log2(e) == 1 (to f32 round-off: the caller's q carries the factor, as for the forward): the logits leave the
// MFMAs in log2 units and take -lse as the chain's start value instead of a multiply-add each.
template <int MODE, int HD, bool BIAS>
int launch_bwd(hipStream_t st, const BwdArgs& a, int B) {
  // (not for the merged pass at head dim 128: there the start values come from LDS, a read that the chain's first
  // MFMA then waits for, and the multiply-add version measured 3 % faster)
  if constexpr (!BIAS && !(MODE == 3 && HD == 128)) {
    if (a.c > 1.0f - 1e-6f && a.c < 1.0f + 1e-6f) return launch_bwd_as<MODE, HD, false, true>(st, a, B);
  }
  return launch_bwd_as<MODE, HD, BIAS, false>(st, a, B);
}

template <int MODE>
int launch_bwd_any(hipStream_t st, const BwdArgs& a, int B, int D) {
  if (D == 128) return a.bias ? launch_bwd<MODE, 128, true>(st, a, B) : launch_bwd<MODE, 128, false>(st, a, B);
  return a.bias ? launch_bwd<MODE, 64, true>(st, a, B) : launch_bwd<MODE, 64, false>(st, a, B);
}

}  // namespace
}  // namespace mdattn

using namespace mdattn;

extern "C" int64_t mdattn_bwd_workspace_floats(int B, int H, int Sq) {
  if (B <= 0 || H <= 0 || Sq <= 0) return 0;
  return 2 * (int64_t)B * H * (((int64_t)Sq + 31) / 32 * 32);
}

// Shared body of mdattn_bwd_bf16 and mdattn_bwd_bf16_static: validation, the preparation kernel and the two passes.
static int bwd_run(hipStream_t st, const void* q, const void* k, const void* v, const void* out, const void* dout,
                   const float* lse, void* dq, void* dk, void* dv, float* workspace, int64_t workspace_floats,
                   int B, int H, int Sq, int Skv, int D,
                   const mdattn_strides* q_strides, const mdattn_strides* k_strides,
                   const mdattn_strides* v_strides, const mdattn_strides* o_strides, float scale,
                   const float* key_bias, int64_t bias_stride) {
  if (!q || !k || !v || !out || !dout || !lse || !dq || !dk || !dv || !workspace) return MDATTN_E_BADARG;
  if (key_bias) {
    if (bias_stride < ((int64_t)Skv + 31) / 32 * 32 || bias_stride % 32 != 0) return MDATTN_E_BADARG;
    if (!aligned16(key_bias)) return MDATTN_E_ALIGN;
  }
  if (B <= 0 || H <= 0 || Sq <= 0 || Skv <= 0 || D <= 0) return MDATTN_E_BADARG;
  if (!q_strides || !k_strides || !v_strides || !o_strides) return MDATTN_E_BADARG;
  if (!(scale > 0.f) || !(scale < 1e30f)) return MDATTN_E_BADARG;
  if (D != 128 && D != 64) return MDATTN_E_UNSUPPORTED;
  if (workspace_floats < mdattn_bwd_workspace_floats(B, H, Sq)) return MDATTN_E_BADARG;
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(out) || !aligned16(dout) || !aligned16(dq) ||
      !aligned16(dk) || !aligned16(dv) || !aligned16(workspace) || (reinterpret_cast<uintptr_t>(lse) & 3u))
    return MDATTN_E_ALIGN;
  if (!strides_ok(q_strides, 8) || !strides_ok(k_strides, 8) || !strides_ok(v_strides, 8) || !strides_ok(o_strides, 8))
    return MDATTN_E_ALIGN;
  if (q_strides->seq < D || k_strides->seq < D || v_strides->seq < D || o_strides->seq < D) return MDATTN_E_BADARG;
  // every tensor is streamed by one of the passes with 32-bit byte offsets inside a row group
  if (q_strides->seq >= (1 << 23) || k_strides->seq >= (1 << 23) || v_strides->seq >= (1 << 23) || o_strides->seq >= (1 << 23))
    return MDATTN_E_UNSUPPORTED;

  const int Sp = (Sq + 31) / 32 * 32;
  float* lse2 = workspace;
  float* delta = workspace + (int64_t)B * H * Sp;
  const int64_t rows = (int64_t)B * H * Sp;
  if ((rows + 15) / 16 > 0x7FFFFFFF || rows >= (1 << 29)) return MDATTN_E_UNSUPPORTED;  // delta - lse2 as a 32-bit byte offset
  MDATTN_LAUNCH(bwd_prep_kernel, dim3((unsigned)((rows + 15) / 16)), dim3(256), 0, st, (const __bf16*)out,
                     (const __bf16*)dout, lse, lse2, delta, H, Sq, Sp, D, rows, o_strides->batch, o_strides->seq, o_strides->head);
  if (launch_status() != MDATTN_OK) return MDATTN_E_LAUNCH;

  BwdArgs a;
  a.lse2 = lse2; a.delta = delta; a.H = H; a.Sp = Sp; a.c = scale * kLog2e; a.scale = scale;
  a.bias = key_bias; a.bias_sb = bias_stride;
  auto set = [](int64_t& sb, int64_t& ss, int64_t& sh, const mdattn_strides* s) { sb = s->batch; ss = s->seq; sh = s->head; };
  // dq: entity q / dout, stream k (scores), v (dP), k (accumulate)
  a.e1 = (const __bf16*)q; a.e2 = (const __bf16*)dout; a.s1 = (const __bf16*)k; a.s2 = (const __bf16*)v; a.s3 = (const __bf16*)k;
  a.out = (__bf16*)dq; a.Se = Sq; a.Ss = Skv;
  set(a.e1_sb, a.e1_ss, a.e1_sh, q_strides); set(a.e2_sb, a.e2_ss, a.e2_sh, o_strides);
  set(a.s1_sb, a.s1_ss, a.s1_sh, k_strides); set(a.s2_sb, a.s2_ss, a.s2_sh, v_strides); set(a.s3_sb, a.s3_ss, a.s3_sh, k_strides);
  set(a.o_sb, a.o_ss, a.o_sh, q_strides);
  int rc = launch_bwd_any<0>(st, a, B, D);
  if (rc != MDATTN_OK) return rc;
  // dk and dv in one pass: entity k / v, stream q (scores, and accumulate for dk), dout (dP, and accumulate for dv)
  a.e1 = (const __bf16*)k; a.e2 = (const __bf16*)v; a.s1 = (const __bf16*)q; a.s2 = (const __bf16*)dout; a.s3 = (const __bf16*)q;
  a.s4 = (const __bf16*)dout;
  a.out = (__bf16*)dk; a.out2 = (__bf16*)dv; a.Se = Skv; a.Ss = Sq;
  set(a.e1_sb, a.e1_ss, a.e1_sh, k_strides); set(a.e2_sb, a.e2_ss, a.e2_sh, v_strides);
  set(a.s1_sb, a.s1_ss, a.s1_sh, q_strides); set(a.s2_sb, a.s2_ss, a.s2_sh, o_strides); set(a.s3_sb, a.s3_ss, a.s3_sh, q_strides);
  set(a.s4_sb, a.s4_ss, a.s4_sh, o_strides);
  set(a.o_sb, a.o_ss, a.o_sh, k_strides); set(a.o2_sb, a.o2_ss, a.o2_sh, v_strides);
  return launch_bwd_any<3>(st, a, B, D);
}


extern "C" int mdattn_bwd_bf16(void* stream, const void* q, const void* k, const void* v, const void* out, const void* dout,
                               const float* lse, void* dq, void* dk, void* dv, float* workspace, int64_t workspace_floats,
                               int B, int H, int Sq, int Skv, int D,
                               const mdattn_strides* q_strides, const mdattn_strides* k_strides,
                               const mdattn_strides* v_strides, const mdattn_strides* o_strides, float scale) {
  return bwd_run((hipStream_t)stream, q, k, v, out, dout, lse, dq, dk, dv, workspace, workspace_floats, B, H, Sq, Skv, D,
                 q_strides, k_strides, v_strides, o_strides, scale, nullptr, 0);
}

extern "C" int mdattn_bwd_bf16_bias(void* stream, const void* q, const void* k, const void* v, const void* out, const void* dout,
                                    const float* lse, void* dq, void* dk, void* dv, float* workspace, int64_t workspace_floats,
                                    int B, int H, int Sq, int Skv, int D,
                                    const mdattn_strides* q_strides, const mdattn_strides* k_strides,
                                    const mdattn_strides* v_strides, const mdattn_strides* o_strides, float scale,
                                    const float* key_bias, int64_t bias_stride) {
  if (!key_bias) return MDATTN_E_BADARG;
  return bwd_run((hipStream_t)stream, q, k, v, out, dout, lse, dq, dk, dv, workspace, workspace_floats, B, H, Sq, Skv, D,
                 q_strides, k_strides, v_strides, o_strides, scale, key_bias, bias_stride);
}

// ---------------------------------------------------------------------------------------------------
// mdattn_bwd_bf16_static: the same backward for callers that cannot allocate (HIP graph capture, serving loops that
// forbid hipMalloc).  The workspace (-lse in log2 units and -delta, one float each per padded query row) lives in a
// file-scope device array instead of a caller's buffer.  Every GPU holds its own copy of the array at its own
// address: that address is looked up once per device with hipGetSymbolAddress and kept; host code never uses the
// array's name as a pointer.  bwd_prep_kernel writes every element the passes read, so nothing has to be cleared
// between calls; calls that overlap on one GPU share the array and race.
static __device__ __align__(256) float scratch[MDATTN_BWD_STATIC_MAX_FLOATS];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
std::atomic<float*> g_scratch_ptr[kMaxDevices];

// Device address of `scratch` on the current device (looked up on the first call per device), or nullptr.
float* scratch_on_current_device() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  float* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (p) return p;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  p = g_scratch_ptr[dev].load(std::memory_order_relaxed);
  if (p) return p;
  void* sym = nullptr;
  if (hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch)) != hipSuccess || !sym) {
    (void)hipGetLastError();
    return nullptr;
  }
  p = static_cast<float*>(sym);
  g_scratch_ptr[dev].store(p, std::memory_order_release);
  return p;
}
}  // namespace

// Also the warm-up of the static entry point: looks the array's address up for the current device (which may make the
// runtime load the code object and place the array), so that a later mdattn_bwd_bf16_static call -- under graph
// capture, say -- finds it resolved.  Without a GPU the lookup fails quietly.
extern "C" int64_t mdattn_bwd_static_max_floats(void) {
  (void)scratch_on_current_device();
  return MDATTN_BWD_STATIC_MAX_FLOATS;
}

extern "C" int mdattn_bwd_bf16_static(void* stream, const void* q, const void* k, const void* v, const void* out,
                                      const void* dout, const float* lse, void* dq, void* dk, void* dv,
                                      int B, int H, int Sq, int Skv, int D,
                                      const mdattn_strides* q_strides, const mdattn_strides* k_strides,
                                      const mdattn_strides* v_strides, const mdattn_strides* o_strides, float scale) {
  if (B <= 0 || H <= 0 || Sq <= 0) return MDATTN_E_BADARG;
  const int64_t need = mdattn_bwd_workspace_floats(B, H, Sq);
  if (need > (int64_t)MDATTN_BWD_STATIC_MAX_FLOATS) return MDATTN_E_TOOBIG;
  float* ws = scratch_on_current_device();
  if (!ws) return MDATTN_E_LAUNCH;
  return bwd_run((hipStream_t)stream, q, k, v, out, dout, lse, dq, dk, dv, ws, need, B, H, Sq, Skv, D,
                 q_strides, k_strides, v_strides, o_strides, scale, nullptr, 0);
}
