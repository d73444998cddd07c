// Non-causal flash-attention forward for gfx950 (MI355X) on fp8-e4m3 (OCP) operands, head_dim 128 (described below)
// or 64 (template HD: one QK MFMA per 32-key block, two slabs of d, 64-byte rows; the differences are noted in place).
//
// Same decomposition as the bf16 kernel, on v_mfma_f32_32x32x64_f8f6f4 (K = 64 per instruction, twice
// the bf16 rate):
//   workgroup  = NW waves x 32 query rows, three workgroups per CU (three waves per SIMD overlap each other's MFMA
//                and softmax phases); keys walked in tiles of 64 through a 3-slot LDS ring filled by direct
//                global->LDS loads (no staging registers), the loads of tile t+2 issued at the top of iteration t.
//   S^T = K.Q^T  two 32-key blocks per tile, two MFMAs each (d = 0..63, 64..127).  A = K rows from LDS (unpadded
//                rows of head_dim bytes, 16-byte chunks XOR-permuted by the row), B = the wave's Q fragment,
//                resident in registers.  A and B use the same k-slot order, so a lane simply holds 32 contiguous
//                bytes of its row.
//   softmax      in f32 on the logits a lane holds for its query row, against a per-row reference point that is not
//                the running maximum: it moves (cold branch: tile maximum - kPOff = 3, so that e4m3's normal range
//                covers probabilities down to 2^-9 of the maximum) only when a lane's partial sum of P over the
//                tile passes 448, e4m3's largest value.  MODE 0: q_scale*k_scale*scale*log2(e) folded into the
//                exp2 argument, one multiply-add per logit.  MODE 1 (that product is a power of two): the scale
//                rides in the MFMAs' block-scale operand and the chains start at minus the reference, P is one
//                exp2 away.  MODE 2: no exponentials either (see kCodeOne).  Which of MODE 0 and MODE 1/2 applies
//                depends on scales that live in device memory: one kernel holds both bodies and takes a
//                wave-uniform branch on the scales it reads.
//   O^T += V^T.P^T  one MFMA per 32-wide slab of d with all 64 keys of the tile as K.  P goes from the
//                accumulator layout to the B operand by the e4m3 convert alone (operand byte s = value
//                s%16 of block s/16).  V^T comes from the row-major V tile through ds_read_b64_tr_b8:
//                within 16 lanes, lane i receives as byte e the element i%8 of the 8-byte chunk whose
//                address lane 2e + i/8 supplies, so each lane points at one key row and one 8-byte
//                column chunk, and every lane ends up with 8 keys of its own d.  The V tile's 16-byte chunks are
//                XOR-permuted by row bits 1 and 3, which makes the 8 rows x 32 B a half-wave reads hit 64
//                distinct banks.
//   key bias     (BIAS) the tile's 64 bias values ride through the LDS ring with the tile (a register load inside
//                the loop would be waited for in issue order, behind the loads of the tile after next); tiles whose
//                bias is all zero (every tile but the last few, for a padding mask) skip the bias code.  The bias
//                joins the logits right after the MFMAs: divided by the logit scale in MODE 0 (the multiply per
//                logit then carries it), in log2 units in MODE 1.
//   epilogue     O * v_scale / l, bf16; lse = ln2 * (reference + log2 l).
#include <type_traits>

#include "mdattn_common.h"

namespace mdattn {
namespace {

constexpr int kBN8 = 64;                                  // keys per tile
constexpr int kSlots8 = 3;                                // LDS ring depth
// K and V rows sit in LDS with a stride of head_dim bytes (chunks permuted, not padded): 2 * 64 * HD bytes per stage
constexpr float kPOff = 3.0f;                             // P = exp2(logit - max + kPOff) at a fresh maximum
// Softmax without exponentials (MODE 2).  An e4m3 byte read as an integer is a piecewise-linear log2 of its value:
// code = 8 * (exponent + 7) + mantissa.  So the QK MFMAs are made to deliver x' = 8 * (logit - ref) + 56 (block scale
// times 8, start value 56 - 8 ref), and v_cvt_pk_u8_f32 (round to nearest even, saturating at 0) turns x' straight
// into the operand byte: P~ = e4m3(code), equal to 2^(logit - ref) at every power of two and up to 6 % above it in
// between (mean ratio 1.0404, against e4m3's own rounding noise of the same size).  The row sum is taken over the
// decoded bytes (by an MFMA of the operand against ones), so O / l stays a properly normalised average; the lse carries the mean ratio as a constant.
constexpr float kCodeOne = 56.0f;                         // the byte of P~ = 1
constexpr float kCodeBiasLog2 = 0.0570814f;               // log2 of the mean of P~ / 2^x over a binade
constexpr float kPTrig = 448.0f;                          // a lane's partial row sum over one tile above this (e4m3's largest
                                                          // value) sends the wave to the rescale branch

typedef __attribute__((ext_vector_type(2))) int i32x2;
typedef i32x2 __attribute__((address_space(3))) * lds_i32x2_ptr;

struct Fp8Args {
  const uint8_t* q;
  const uint8_t* k;
  const uint8_t* v;
  __bf16* out;
  float* lse;
  const float* q_scale;
  const float* k_scale;
  const float* v_scale;
  int H, Sq, Skv;
  int nqt, total, chunk;
  int64_t q_sb, q_ss, q_sh;
  int64_t k_sb, k_ss, k_sh;
  int64_t v_sb, v_ss, v_sh;
  int64_t o_sb, o_ss, o_sh;
  float c;  // scale * log2(e)
  const float* bias;   // BIAS: additive per-key bias [B, bias_sb], natural-log units (-inf excludes a key)
  int64_t bias_sb;
};

// Register budget: three waves per SIMD (<= 168 VGPRs); four at head dim 64 (<= 128 VGPRs, 24 KB of LDS: 1-4 % faster).  The kernel is bound by the vector ALU (softmax)
// and by latencies a single wave cannot hide, so the third wave per SIMD is worth more than registers.
// BIAS (MODE 0 and 1): an additive per-key bias (a key padding mask), see the header.
template <int NW, int MODE, bool BIAS, int HD>
__device__ __forceinline__ void fp8_body(const Fp8Args& a, const float c, char* smem8) {
  static_assert(!BIAS || MODE != 2, "the key bias keeps exact exponentials");
  static_assert(HD == 128 || HD == 64, "head dim");
  constexpr int kKS8 = HD, kVS8 = HD;                 // row strides in LDS, bytes
  constexpr int kTiles8 = kBN8 * kKS8 + kBN8 * kVS8;  // the K and the V tile of a stage
  constexpr int kStage8 = kTiles8 + (BIAS ? 4 * kBN8 : 0);  // bytes per LDS stage; BIAS: + the tile's 64 bias values (f32)
  constexpr int NJ = HD / 64;                         // QK MFMAs (K = 64) per 32-key block
  constexpr int NSL = HD / 32;                        // 32-wide slabs of d = O accumulators
  constexpr bool PRE = MODE != 0;    // the logit scale is a power of two and rides in the MFMAs' block scale
  constexpr bool CODE = MODE == 2;   // ... and P is formed without exp2: see kCodeOne
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

  const uint8_t* qp = a.q + b * a.q_sb + h * a.q_sh;
  const uint8_t* kp = a.k + b * a.k_sb + h * a.k_sh;
  const uint8_t* vp = a.v + b * a.v_sb + h * a.v_sh;
  const int q0 = qt * BM + wave * 32;
  const int nt = (a.Skv + kBN8 - 1) / kBN8;
  [[maybe_unused]] const float* bias_row = BIAS ? a.bias + b * a.bias_sb : nullptr;
  [[maybe_unused]] const float bias_mul = PRE ? kLog2e : kLog2e / c;  // natural-log bias -> log2 units (MODE 1) or units of the raw products
  [[maybe_unused]] const int bias_cols = (a.Skv + 31) / 32 * 32;      // entries the caller's bias rows are sure to hold

  // ---- Q fragments: lane (row l32, half hh) holds bytes 64*j + 32*hh .. +31 of its row
  i32x8 qf[NJ];
  {
    int row = q0 + l32;
    row = row < a.Sq ? row : a.Sq - 1;
    const uint8_t* p = qp + (int64_t)row * a.q_ss + hh * 32;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const u32x4 lo = *reinterpret_cast<const u32x4*>(p + j * 64);
      const u32x4 hi = *reinterpret_cast<const u32x4*>(p + j * 64 + 16);
      qf[j] = i32x8{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
    }
  }

  // ---- direct global -> LDS loads of one K/V tile (no staging registers, no LDS store instructions).
  // One wave instruction writes 1 KB = 8 rows, row-major; inside a row the 16-byte chunks are stored
  // permuted, which replaces padding: K chunk c of row r sits at position c ^ ((r >> 1) & 7), V chunk c at
  // c ^ 2*(((r >> 1) & 1) + 2*((r >> 3) & 1)).  Every 8 lanes fetch one whole 128-byte row.  Wave w fills
  // the row groups w, w+NW, ...  Rows past the end re-read the last valid row: they only ever meet
  // masked logits (P = 0), and every e4m3 code the quantiser emits is finite.
  // Head dim 64: one instruction writes 16 rows of 64 bytes, every 4 lanes one row; K chunk c of row r sits at
  // c ^ ((r >> 2) & 3), V chunk c at c ^ 2*((r >> 3) & 1): conflict-free for the same two read patterns.
  constexpr int RPI = 1024 / HD;                               // rows one load instruction fills
  constexpr int CPR = HD / 16;                                 // 16-byte chunks per row
  constexpr int GPW = (kBN8 / RPI) / NW;                       // row groups per wave, tile and tensor
  static_assert(GPW >= 1, "a wave fills at least one row group per tile");
  const int grow = lane / CPR;                                 // row of the group this lane fills
  // the row's permutation key (groups w, w+NW of head dim 128 have the same parity; head dim 64 needs the row in its group only)
  const int kx_fill = HD == 128 ? (4 * (wave & 1) + (grow >> 1)) & 7 : (grow >> 2) & 3;
  const int vx_fill = HD == 128 ? 2 * (((grow >> 1) & 1) + 2 * (wave & 1)) : 2 * ((grow >> 3) & 1);
  const unsigned kofs = (unsigned)(grow * (int)a.k_ss + (((lane & (CPR - 1)) ^ kx_fill) * 16));
  const unsigned vofs = (unsigned)(grow * (int)a.v_ss + (((lane & (CPR - 1)) ^ vx_fill) * 16));
  const unsigned smem_addr = lds_addr_of(smem8);
  auto dma = [&](int slot, int kt) __attribute__((always_inline)) {
    const unsigned Ks = smem_addr + (unsigned)(slot * kStage8);
    const unsigned Vs = Ks + kBN8 * kKS8;
    if constexpr (BIAS) {
      // every wave fetches the same 64 values to the same place (one load more per wave and tile, counted in the loop's
      // s_waitcnt); the ring runs up to two tiles past the end, and a tile may reach past the padded bias row
      int col = (kt < nt ? kt : nt - 1) * kBN8 + lane;
      col = col < bias_cols ? col : bias_cols - 1;
      lds_dma4(bias_row, (unsigned)col * 4u, Ks + kTiles8);
    }
    if (kt * kBN8 + kBN8 <= a.Skv) {
      const uint8_t* kt0 = kp + (int64_t)(kt * kBN8 + RPI * wave) * a.k_ss;
      const uint8_t* vt0 = vp + (int64_t)(kt * kBN8 + RPI * wave) * a.v_ss;
#pragma unroll
      for (int i = 0; i < GPW; ++i) {
        lds_dma16(kt0 + (int64_t)(RPI * NW * i) * a.k_ss, kofs, Ks + (unsigned)((wave + NW * i) * RPI * kKS8));
        lds_dma16(vt0 + (int64_t)(RPI * NW * i) * a.v_ss, vofs, Vs + (unsigned)((wave + NW * i) * RPI * kVS8));
      }
    } else {
#pragma unroll
      for (int i = 0; i < GPW; ++i) {
        const int g = wave + NW * i;
        int kk = kt * kBN8 + RPI * g + grow;
        kk = kk < a.Skv ? kk : a.Skv - 1;
        lds_dma16(kp + (int64_t)kk * a.k_ss + (((lane & (CPR - 1)) ^ kx_fill) * 16), Ks + (unsigned)(g * RPI * kKS8));
        lds_dma16(vp + (int64_t)kk * a.v_ss + (((lane & (CPR - 1)) ^ vx_fill) * 16), Vs + (unsigned)(g * RPI * kVS8));
      }
    }
  };

  f32x16 O[NSL];
#pragma unroll
  for (int sl = 0; sl < NSL; ++sl)
#pragma unroll
    for (int i = 0; i < 16; ++i) O[sl][i] = 0.f;
  // When the whole logit scale c is a power of two (power-of-two q and k scales from the quantiser, the softmax
  // scale already inside q), the MFMAs apply it through their block-scale operand and start every logit chain at
  // minus the row's reference point: the logits arrive in log2 units relative to it and the softmax needs no
  // multiply.  The reference then starts at 0 and the first tile always takes the branch that sets it.
  const int sexp = (int)(__float_as_uint(c) >> 23) + (CODE ? 3 : 0);  // E8M0 code of c (of 8 c when the logits come in code units)
  float ref = PRE ? 0.f : -1e30f, l = 0.f;           // reference point of P (log2 units), per-lane partial row sum
  [[maybe_unused]] bool fresh = true;                // PRE with a key bias: the row has not met a finite logit yet
  f32x16 negref;
#pragma unroll
  for (int i = 0; i < 16; ++i) negref[i] = CODE ? kCodeOne : 0.f;

  // lane-constant LDS offsets (bytes)
  // K fragment (d half j, 16-byte half i) of row l32 is logical chunk 4j + 2hh + i
  int k_off[NJ][2];
#pragma unroll
  for (int j = 0; j < NJ; ++j)
#pragma unroll
    for (int i = 0; i < 2; ++i)
      k_off[j][i] = l32 * kKS8 + (((4 * j + 2 * hh + i) ^ (HD == 128 ? (l32 >> 1) & 7 : (l32 >> 2) & 3)) * 16);
  int v_off[NSL];
  {
    const int e = (lane & 15) >> 1;
    const int rowl = 8 * (e >> 2) + 4 * hh + (e & 3);
    // the 32-byte slab's permutation key: row bits 1 and 3 (head dim 128), row bit 3 (head dim 64)
    const int fl = HD == 128 ? ((e >> 1) & 1) + 2 * ((e >> 2) & 1) : (e >> 2) & 1;
    const int cl = 2 * ((lane >> 4) & 1) + (lane & 1);
#pragma unroll
    for (int sl = 0; sl < NSL; ++sl) v_off[sl] = kBN8 * kKS8 + rowl * kVS8 + 32 * (sl ^ fl) + 8 * cl;
  }

  auto tile = [&](int t, int slot, auto masked) __attribute__((always_inline)) {
    const char* Ks = smem8 + slot * kStage8;
    // A key padding mask is zero on all but the last tiles: lane l looks at the bias of key l of the tile, and a tile
    // without any non-zero bias (one LDS read, one compare, one wave-uniform branch per block) skips the bias code.
    [[maybe_unused]] bool has_bias = false;
    if constexpr (BIAS) has_bias = __builtin_amdgcn_ballot_w64(reinterpret_cast<const float*>(Ks + kTiles8)[lane] != 0.f) != 0;
    // ---- S^T = K.Q^T for one 32-key block
    auto qk = [&](f32x16& S, int blk, const char* Kb) __attribute__((always_inline)) {
      i32x8 kf[NJ];
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const u32x4 lo = *reinterpret_cast<const u32x4*>(Kb + k_off[j][0] + blk * 32 * kKS8);
        const u32x4 hi = *reinterpret_cast<const u32x4*>(Kb + k_off[j][1] + blk * 32 * kKS8);
        kf[j] = i32x8{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
      }
      if constexpr (PRE) {  // logits in log2 units minus the reference point, straight out of the MFMAs
        S = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(kf[0], qf[0], negref, 0, 0, 0, 127, 0, sexp);
        if constexpr (NJ == 2) S = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(kf[1], qf[1], S, 0, 0, 0, 127, 0, sexp);
      } else {
        f32x16 z;
#pragma unroll
        for (int i = 0; i < 16; ++i) z[i] = 0.f;
        S = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(kf[0], qf[0], z, 0, 0, 0, 0, 0, 0);
        if constexpr (NJ == 2) S = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(kf[1], qf[1], S, 0, 0, 0, 0, 0, 0);
      }
      // the keys' bias joins the products after the MFMAs: in log2 units (MODE 1) or divided by the logit scale (MODE 0)
      if (BIAS && has_bias) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const f32x4 bv = *reinterpret_cast<const f32x4*>(Kb + kTiles8 + (32 * blk + 8 * g + 4 * hh) * 4);
#pragma unroll
          for (int e = 0; e < 4; ++e) S[4 * g + e] = __builtin_fmaf(bv[e], bias_mul, S[4 * g + e]);
        }
      }
      if constexpr (decltype(masked)::value) {
        const int kbase = t * kBN8 + 4 * hh + 32 * blk;
#pragma unroll
        for (int i = 0; i < 16; ++i)
          if (kbase + 8 * (i >> 2) + (i & 3) >= a.Skv) S[i] = -INFINITY;
      }
    };
    // ---- P = exp2(c*S - ref), f32 row sum, e4m3 pack in B-operand order.  The hot path takes no row
    // maximum: P is formed against the current reference point, and only a lane's sum over the tile (32 of the
    // row's 64 probabilities) beyond e4m3's largest value, so possibly one probability beyond it, sends the wave
    // through the branch that moves every row's reference to its true maximum - kPOff, rescales the accumulators
    // and redoes the tile's logits and P.  Right after a move such a sum is at most 32 * 2^kPOff = 256, so even a
    // row of equal logits triggers again only when its level has grown by 0.8 log2 units.  The two 32-key blocks
    // of the tile are taken one after the other, so that only 16 logits per lane are alive at a time.
    i32x8 pk;
    float ls;
    unsigned hib = 0;  // MODE 2: OR of the operand dwords; a byte above 127 is a logit beyond e4m3's range
    auto soft = [&](const f32x16& S, int blk, float rf) __attribute__((always_inline)) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        if constexpr (CODE) {
          unsigned u = __float_as_uint(S[4 * g]);  // any defined value: all four bytes are written below
          u = __builtin_amdgcn_cvt_pk_u8_f32(S[4 * g], 0, u);
          u = __builtin_amdgcn_cvt_pk_u8_f32(S[4 * g + 1], 1, u);
          u = __builtin_amdgcn_cvt_pk_u8_f32(S[4 * g + 2], 2, u);
          u = __builtin_amdgcn_cvt_pk_u8_f32(S[4 * g + 3], 3, u);
          hib |= u;
          pk[4 * blk + g] = (int)u;
        } else {
          float p[4];
#pragma unroll
          for (int x = 0; x < 4; ++x) p[x] = __builtin_amdgcn_exp2f(PRE ? S[4 * g + x] : __builtin_fmaf(S[4 * g + x], c, -rf));
          ls += (p[0] + p[1]) + (p[2] + p[3]);
          int u = __builtin_bit_cast(int, p[0]);  // any defined value: both halves are written below, in place
          u = __builtin_amdgcn_cvt_pk_fp8_f32(p[0], p[1], u, false);
          u = __builtin_amdgcn_cvt_pk_fp8_f32(p[2], p[3], u, true);
          pk[4 * blk + g] = u;
        }
      }
    };
    ls = 0.f;
#pragma unroll
    for (int blk = 0; blk < 2; ++blk) {
      f32x16 S;
      qk(S, blk, Ks);
      soft(S, blk, ref);
      if (PRE) __builtin_amdgcn_sched_barrier(0);  // keeps the second block's logits from being hoisted over the first's softmax
    }
    // MODE 2: the row sum of the tile's 64 operand bytes comes from the matrix pipe, one more MFMA per tile (ones . P~:
    // every output row holds the sums, over both halves of the row's keys) instead of two decodes and four adds per
    // four logits (1.3 % faster at head dim 128, 6 % at 64).  A byte 0x7F still poisons the sum with its NaN.
    auto rowsum = [&]() __attribute__((always_inline)) {
      // the ones as FP4 (E2M1: 1.0 = 0b0010), the operand bytes as e4m3: the instruction takes the two formats
      // independently, and a lane's 32 FP4 ones are four registers where e4m3 ones are eight
      const int one8 = 0x22222222;  // eight E2M1 ones
      const i32x8 ones = {one8, one8, one8, one8, 0, 0, 0, 0};
      f32x16 z;
#pragma unroll
      for (int i = 0; i < 16; ++i) z[i] = 0.f;
      z = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(ones, pk, z, 4, 0, 0, 0, 0, 0);
      return z[0];
    };
    if constexpr (CODE) ls = rowsum();
    // (a byte 0x7F decodes to NaN and poisons the sum; bytes above it are caught by their top bit)
    // PRE: a row's reference is set by the first tile in which it meets a finite logit: tile 0, unless a key bias
    // excludes all of that tile's keys (`fresh` then stays set and the row tries again on the next tile)
    if (__builtin_expect(__builtin_amdgcn_ballot_w64(!(ls <= (CODE ? 3.0e38f : kPTrig)) || (hib & 0x80808080u) != 0u || (PRE && BIAS && fresh)) != 0 ||
                         (PRE && !BIAS && t == 0), 0)) {
      // The logits are recomputed rather than kept: the hot path holds them only while it forms P.
      int zero = 0;
      asm volatile("" : "+s"(zero));  // an address the compiler cannot match with the hot path's: no reuse of its logits
      float mx = -INFINITY;
#pragma unroll
      for (int blk = 0; blk < 2; ++blk) {
        f32x16 S;
        qk(S, blk, Ks + zero);
#pragma unroll
        for (int i = 0; i < 16; ++i) mx = fmaxf(mx, S[i]);
      }
      float alpha;
      if constexpr (PRE) {  // the logits are relative to the old reference (MODE 2: in code units, 56 at the reference)
        mx = xhalf_max(mx);
        if constexpr (CODE) mx = (mx - kCodeOne) * 0.125f;
        float dm;
        if constexpr (BIAS) {
          const bool first = fresh && mx > -INFINITY;
          dm = first ? mx - kPOff : (fresh ? 0.f : fmaxf(mx - kPOff, 0.f));
          alpha = fresh ? 0.f : __builtin_amdgcn_exp2f(-dm);
          fresh = fresh && !first;
        } else {
          dm = t == 0 ? mx - kPOff : fmaxf(mx - kPOff, 0.f);
          alpha = t == 0 ? 0.f : __builtin_amdgcn_exp2f(-dm);
        }
        ref += dm;
#pragma unroll
        for (int i = 0; i < 16; ++i) negref[i] = CODE ? kCodeOne - 8.0f * ref : -ref;
      } else {
        mx = xhalf_max(mx) * c;
        const float nref = fmaxf(ref, mx - kPOff);
        alpha = __builtin_amdgcn_exp2f(ref - nref);
        ref = nref;
      }
      asm volatile("" : "+v"(alpha));  // keeps the rescale inside this rarely taken branch
      l *= alpha;
#pragma unroll
      for (int sl = 0; sl < NSL; ++sl)
#pragma unroll
        for (int i = 0; i < 16; ++i) O[sl][i] *= alpha;
      // once more against the new reference points
      asm volatile("" : "+s"(zero));
      ls = 0.f;
      hib = 0u;
#pragma unroll
      for (int blk = 0; blk < 2; ++blk) {
        f32x16 S;
        qk(S, blk, Ks + zero);
        soft(S, blk, ref);
      }
      if constexpr (CODE) ls = rowsum();
    }
    l += ls;
    // ---- O^T += V^T.P^T
    // The V^T operand of slab sl + 1 is requested before the MFMA of slab sl is issued (the 16 registers of the logits
    // are free by now), pinned by scheduling barriers: the compiler's own order reads each operand into one
    // buffer and waits for it right before its MFMA.
    auto vfrag = [&](int sl) __attribute__((always_inline)) {
      const char* vsrc = Ks + v_off[sl];
      const i32x2 r0 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_i32x2_ptr)(vsrc));
      const i32x2 r1 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_i32x2_ptr)(vsrc + 16 * kVS8));
      const i32x2 r2 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_i32x2_ptr)(vsrc + 32 * kVS8));
      const i32x2 r3 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_i32x2_ptr)(vsrc + 48 * kVS8));
      return i32x8{r0[0], r0[1], r1[0], r1[1], r2[0], r2[1], r3[0], r3[1]};
    };
    i32x8 vw[2];
    vw[0] = vfrag(0);
#pragma unroll
    for (int sl = 0; sl < NSL; ++sl) {
      if (sl + 1 < NSL) vw[(sl + 1) & 1] = vfrag(sl + 1);
      __builtin_amdgcn_sched_barrier(0);
      O[sl] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(vw[sl & 1], pk, O[sl], 0, 0, 0, 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // Ring of kSlots8 tiles: the loads of tile t+2 are issued at the top of iteration t, so at the top of
  // iteration t only the 2*GPW loads of tile t+1 may still be in flight once tile t is needed.
  dma(0, 0);
  dma(1, 1);
  int slot = 0, fill = 2;
  for (int t = 0; t < nt - 1; ++t) {
    __builtin_amdgcn_s_waitcnt(0x0F70 | (2 * GPW + (BIAS ? 1 : 0)));  // vmcnt: this wave's share of tile t has landed
    __syncthreads();                                  // ... and everyone's; slot `fill` (tile t-1) is free
    dma(fill, t + 2);
    tile(t, slot, std::false_type{});
    slot = slot == kSlots8 - 1 ? 0 : slot + 1;
    fill = fill == kSlots8 - 1 ? 0 : fill + 1;
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();
  tile(nt - 1, slot, std::true_type{});

  // ---- epilogue
  __bf16* op = a.out + b * a.o_sb + h * a.o_sh;
  const float lt = CODE ? l : xhalf_sum(l);  // MODE 2: the MFMA already summed both halves of the row's keys
  const float inv = lt > 0.f ? a.v_scale[0] / lt : 0.f;  // rows whose keys are all excluded return 0 (and lse = -inf)
  const int row = q0 + l32;
  if (row < a.Sq) {
    __bf16* orow = op + (int64_t)row * a.o_ss + 4 * hh;
#pragma unroll
    for (int sl = 0; sl < NSL; ++sl)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        uint2 u;
        u.x = pack2(O[sl][4 * g] * inv, O[sl][4 * g + 1] * inv);
        u.y = pack2(O[sl][4 * g + 2] * inv, O[sl][4 * g + 3] * inv);
        *reinterpret_cast<uint2*>(orow + sl * 32 + 8 * g) = u;
      }
    if (a.lse && hh == 0) a.lse[((int64_t)b * a.H + h) * a.Sq + row] = (ref + __log2f(lt) - (CODE ? kCodeBiasLog2 : 0.f)) * kLn2;
  }
}

// One kernel for both kinds of logit scale: c = scale * log2(e) * q_scale * k_scale is read on the device (the scales
// are results of the quantiser, the host never sees them), and every wave takes the same branch: the body without a
// multiply per logit when c is a power of two (PMODE 1: exp2; 2: the byte-grid softmax), the general body otherwise.
// The two bodies are never live together, so the kernel's register count is the larger of the two.
template <int NW, int PMODE, bool BIAS, int HD>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(HD == 64 ? 4 : 3, HD == 64 ? 4 : 3))) void attn_fwd_fp8_kernel(Fp8Args a) {
  extern __shared__ __attribute__((aligned(16))) char smem8[];
  const float c = a.c * a.q_scale[0] * a.k_scale[0];
  const unsigned cbits = __builtin_amdgcn_readfirstlane(__float_as_uint(c));
  const bool c_pow2 = (cbits & 0x007FFFFFu) == 0u && cbits > 0x00800000u && cbits < 0x7F000000u;
  if (c_pow2) fp8_body<NW, PMODE, BIAS, HD>(a, c, smem8);
  else fp8_body<NW, 0, BIAS, HD>(a, c, smem8);
}

template <int NW, int HD>
int launch_fwd8(hipStream_t st, Fp8Args a, int B, int softmax_mode) {
  constexpr int BM = NW * 32;
  const int lds_bytes = kSlots8 * (2 * kBN8 * HD + (a.bias ? 4 * kBN8 : 0));
  a.nqt = (a.Sq + BM - 1) / BM;
  const int64_t total = (int64_t)B * a.H * a.nqt;
  if (total > (int64_t)0x7FFFFFF0) return MDATTN_E_UNSUPPORTED;
  a.total = (int)total;
  a.chunk = (a.total + 7) / 8;
  const dim3 grid(a.chunk * 8), block(NW * 64);
  if (a.bias) MDATTN_LAUNCH((attn_fwd_fp8_kernel<NW, 1, true, HD>), grid, block, lds_bytes, st, a);
  else if (softmax_mode == MDATTN_FP8_SOFTMAX_BYTE_GRID) MDATTN_LAUNCH((attn_fwd_fp8_kernel<NW, 2, false, HD>), grid, block, lds_bytes, st, a);
  else MDATTN_LAUNCH((attn_fwd_fp8_kernel<NW, 1, false, HD>), grid, block, lds_bytes, st, a);
  return launch_status();
}

}  // namespace
}  // namespace mdattn

using namespace mdattn;

static int fp8_run(void* stream, const void* q8, const void* k8, const void* v8, void* out, float* lse,
                   int B, int H, int Sq, int Skv, int D,
                   const mdattn_strides* q_strides, const mdattn_strides* k_strides,
                   const mdattn_strides* v_strides, const mdattn_strides* o_strides, float scale,
                   const float* q_scale, const float* k_scale, const float* v_scale, int softmax_mode,
                   const float* key_bias, int64_t bias_stride) {
  if (softmax_mode != MDATTN_FP8_SOFTMAX_EXP2 && softmax_mode != MDATTN_FP8_SOFTMAX_BYTE_GRID) return MDATTN_E_BADARG;
  if (!q8 || !k8 || !v8 || !out || !q_scale || !k_scale || !v_scale) return MDATTN_E_BADARG;
  if (B <= 0 || H <= 0 || Sq <= 0 || Skv <= 0 || D <= 0) return MDATTN_E_BADARG;
  if (!q_strides || !k_strides || !v_strides || !o_strides) return MDATTN_E_BADARG;
  if (!(scale > 0.f) || !(scale < 1e30f)) return MDATTN_E_BADARG;
  if (D != 128 && D != 64) return MDATTN_E_UNSUPPORTED;
  if (!aligned16(q8) || !aligned16(k8) || !aligned16(v8) || !aligned16(out) || (reinterpret_cast<uintptr_t>(lse) & 3u) ||
      (reinterpret_cast<uintptr_t>(q_scale) & 3u) || (reinterpret_cast<uintptr_t>(k_scale) & 3u) ||
      (reinterpret_cast<uintptr_t>(v_scale) & 3u))
    return MDATTN_E_ALIGN;
  // fp8 rows are read in 16-byte pieces, bf16 output rows written in 8-byte pieces
  if (!strides_ok(q_strides, 16) || !strides_ok(k_strides, 16) || !strides_ok(v_strides, 16) || !strides_ok(o_strides, 8))
    return MDATTN_E_ALIGN;
  if (q_strides->seq < D || k_strides->seq < D || v_strides->seq < D || o_strides->seq < D) return MDATTN_E_BADARG;
  // per-lane byte offsets inside one 64-row tile are kept in 32 bits
  if (k_strides->seq >= (1 << 24) || v_strides->seq >= (1 << 24)) return MDATTN_E_UNSUPPORTED;

  Fp8Args a;
  a.q = (const uint8_t*)q8; a.k = (const uint8_t*)k8; a.v = (const uint8_t*)v8; a.out = (__bf16*)out; a.lse = lse;
  a.q_scale = q_scale; a.k_scale = k_scale; a.v_scale = v_scale;
  a.H = H; a.Sq = Sq; a.Skv = Skv;
  a.q_sb = q_strides->batch; a.q_ss = q_strides->seq; a.q_sh = q_strides->head;
  a.k_sb = k_strides->batch; a.k_ss = k_strides->seq; a.k_sh = k_strides->head;
  a.v_sb = v_strides->batch; a.v_ss = v_strides->seq; a.v_sh = v_strides->head;
  a.o_sb = o_strides->batch; a.o_ss = o_strides->seq; a.o_sh = o_strides->head;
  a.c = scale * kLog2e;
  if (a.c > 1.0f - 1e-6f && a.c < 1.0f + 1e-6f) a.c = 1.0f;  // scale = ln 2: the caller's q carries the softmax scale
  a.bias = key_bias;
  a.bias_sb = bias_stride;
  if (key_bias) {
    if (bias_stride < ((int64_t)Skv + 31) / 32 * 32 || bias_stride % 32 != 0) return MDATTN_E_BADARG;
    if (!aligned16(key_bias)) return MDATTN_E_ALIGN;
  }
  hipStream_t st = (hipStream_t)stream;
  // Four waves per workgroup (three workgroups per CU) measured faster than eight at every shape tried.
  return D == 128 ? launch_fwd8<4, 128>(st, a, B, softmax_mode) : launch_fwd8<4, 64>(st, a, B, softmax_mode);
}


extern "C" int mdattn_fwd_fp8(void* stream, const void* q8, const void* k8, const void* v8, void* out, float* lse,
                              int B, int H, int Sq, int Skv, int D,
                              const mdattn_strides* q_strides, const mdattn_strides* k_strides,
                              const mdattn_strides* v_strides, const mdattn_strides* o_strides, float scale,
                              const float* q_scale, const float* k_scale, const float* v_scale, int softmax_mode) {
  return fp8_run(stream, q8, k8, v8, out, lse, B, H, Sq, Skv, D, q_strides, k_strides, v_strides, o_strides, scale, q_scale,
                 k_scale, v_scale, softmax_mode, nullptr, 0);
}

extern "C" int mdattn_fwd_fp8_bias(void* stream, const void* q8, const void* k8, const void* v8, void* out, float* lse,
                                   int B, int H, int Sq, int Skv, int D,
                                   const mdattn_strides* q_strides, const mdattn_strides* k_strides,
                                   const mdattn_strides* v_strides, const mdattn_strides* o_strides, float scale,
                                   const float* q_scale, const float* k_scale, const float* v_scale,
                                   const float* key_bias, int64_t bias_stride) {
  if (!key_bias) return MDATTN_E_BADARG;
  return fp8_run(stream, q8, k8, v8, out, lse, B, H, Sq, Skv, D, q_strides, k_strides, v_strides, o_strides, scale, q_scale,
                 k_scale, v_scale, MDATTN_FP8_SOFTMAX_EXP2, key_bias, bias_stride);
}
