// Shared device/host helpers for the gfx950 kernels behind mdattn.h.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "mdattn.h"

namespace mdattn {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(8))) float f32x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(2))) unsigned u32x2;
typedef __attribute__((ext_vector_type(4))) unsigned u32x4;
typedef __attribute__((ext_vector_type(8))) int i32x8;

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// max over the two lanes l and l^32 (the two halves of a wave64).
__device__ __forceinline__ float xhalf_max(float x) {
  u32x2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float xhalf_sum(float x) {
  u32x2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Butterfly sum over each aligned group of 16 lanes, on the VALU's DPP path.
__device__ __forceinline__ float row16_sum(float x) {
  x += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(x), 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
  x += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(x), 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
  x += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(x), 0x141, 0xF, 0xF, true));  // row_half_mirror
  x += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(x), 0x140, 0xF, 0xF, true));  // row_mirror
  return x;
}

__device__ __forceinline__ float bf16_bits_to_f32(unsigned short b) { return __uint_as_float(((unsigned)b) << 16); }

// 8 bf16 packed in a uint4 -> 8 floats.
__device__ __forceinline__ void unpack8(const uint4& u, float* f) {
  f[0] = __uint_as_float(u.x << 16); f[1] = __uint_as_float(u.x & 0xFFFF0000u);
  f[2] = __uint_as_float(u.y << 16); f[3] = __uint_as_float(u.y & 0xFFFF0000u);
  f[4] = __uint_as_float(u.z << 16); f[5] = __uint_as_float(u.z & 0xFFFF0000u);
  f[6] = __uint_as_float(u.w << 16); f[7] = __uint_as_float(u.w & 0xFFFF0000u);
}

// two floats -> packed bf16 pair (round-to-nearest-even; gfx950 has a native convert).
__device__ __forceinline__ unsigned pack2(float a, float b) {
  f32x2 v = {a, b};
  bf16x2 r = __builtin_convertvector(v, bf16x2);
  return __builtin_bit_cast(unsigned, r);
}
__device__ __forceinline__ uint4 pack8(const float* f) {
  uint4 u;
  u.x = pack2(f[0], f[1]); u.y = pack2(f[2], f[3]); u.z = pack2(f[4], f[5]); u.w = pack2(f[6], f[7]);
  return u;
}

// streaming (non-temporal) 16-byte accesses for data touched exactly once
__device__ __forceinline__ uint4 ld_nt(const uint4* p) {
  const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ float4 ld_nt(const float4* p) {
  const f32x4 v = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p));
  return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void st_nt(uint4* p, const uint4& u) {
  const u32x4 v = {u.x, u.y, u.z, u.w};
  __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p));
}

// Direct global -> LDS load of 16 bytes per lane: lane i's bytes land at lds_addr + 16*i (the LDS base
// travels in M0).  Written as inline assembly so that the loads stay asynchronous: the compiler cannot
// tell which LDS bytes such a load writes and would otherwise wait for it before the next LDS read.
// The statement writes M0 and says so, so the compiler never keeps a value of its own in M0 across it.
// The kernels track these loads themselves with s_waitcnt vmcnt.
__device__ __forceinline__ void lds_dma16(const void* base, unsigned byte_off, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_addr), "v"(byte_off), "s"(base) : "memory", "m0");
}
__device__ __forceinline__ void lds_dma16(const void* addr, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(lds_addr), "v"(addr) : "memory", "m0");
}
// The 4-byte form: lane i's dword lands at lds_addr + 4*i.
__device__ __forceinline__ void lds_dma4(const void* base, unsigned byte_off, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dword %1, %2" : : "s"(lds_addr), "v"(byte_off), "s"(base) : "memory", "m0");
}
__device__ __forceinline__ unsigned lds_addr_of(const void* p) {
  return (unsigned)(uintptr_t)(const void __attribute__((address_space(3)))*)p;
}

// Arguments of the attention-forward kernels (element strides; head_dim contiguous).
struct AttnArgs {
  const __bf16* q;
  const __bf16* k;
  const __bf16* v;
  __bf16* out;
  float* lse;
  int H, Sq, Skv;
  int nqt, total, chunk;
  int64_t q_sb, q_ss, q_sh;
  int64_t k_sb, k_ss, k_sh;
  int64_t v_sb, v_ss, v_sh;
  int64_t o_sb, o_ss, o_sh;
  float c;  // scale * log2(e)
  const float* bias;   // optional additive per-key bias [B, bias_sb] (natural-log units), flat kernel only
  int64_t bias_sb;
  float* o_run;    // when set: no `out`; the result is merged in LSE space into this f32 carry (strides o_s*, in floats)
  float* lse_run;  // ... and into its lse [B,H,Sq]
};



inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline bool strides_ok(const mdattn_strides* s, int64_t mult) {
  return s && s->batch % mult == 0 && s->seq % mult == 0 && s->head % mult == 0 && s->seq > 0 && s->head > 0 && s->batch >= 0;
}
// Every kernel launch of the library goes through MDATTN_LAUNCH and is followed by launch_status().  hipGetLastError()
// returns (and clears) the last error of ANY earlier HIP call on the calling thread, so an error that the caller's own
// code left pending would otherwise surface here as MDATTN_E_LAUNCH of a launch that went fine: MDATTN_LAUNCH reads
// the pending error first.  That clears it: a caller who wants to see its own sticky error has to read it before
// calling into the library.
#define MDATTN_LAUNCH(...)         \
  do {                             \
    (void)hipGetLastError();       \
    hipLaunchKernelGGL(__VA_ARGS__); \
  } while (0)
inline int launch_status() { return hipGetLastError() == hipSuccess ? MDATTN_OK : MDATTN_E_LAUNCH; }

// A kernel that needs more dynamic LDS than the default limit has to opt in with hipFuncSetAttribute, once per
// kernel and device: one LdsOptIn per kernel instance remembers the devices that have been told.
struct LdsOptIn {
  std::atomic<uint64_t> devices{0};
};
inline int lds_opt_in(LdsOptIn& flag, const void* kernel, int lds_bytes) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return MDATTN_E_LAUNCH;
  const uint64_t bit = 1ull << dev;
  if (flag.devices.load(std::memory_order_acquire) & bit) return MDATTN_OK;
  if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes) != hipSuccess) return MDATTN_E_LAUNCH;
  flag.devices.fetch_or(bit, std::memory_order_release);
  return MDATTN_OK;
}

// Schedule forced by mdattn_set_fwd_schedule (0: chosen by shape).
int forced_fwd_schedule();

}  // namespace mdattn
