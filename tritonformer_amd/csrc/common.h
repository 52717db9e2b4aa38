// Shared device helpers for the gfx950 kernels: 16-bit types, 16-byte vector
// access, wave64 reductions and MFMA wrappers.  gfx950 only, wave size 64.
#pragma once
#include <type_traits>
#include <utility>
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/tritonformer_amd.h"

namespace tfa {

typedef _Float16 f16;
typedef __bf16 bf16;

typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

template <typename T> struct Vec;
template <> struct Vec<f16> { typedef f16x8 v8; typedef f16x4 v4; };
template <> struct Vec<bf16> { typedef bf16x8 v8; typedef bf16x4 v4; };

template <typename T> __device__ __forceinline__ float to_f32(T v) { return (float)v; }
template <typename T> __device__ __forceinline__ T from_f32(float v) { return (T)v; }

// ---- wave64 reductions (butterfly over cross-lane shuffles) ---------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// ---- 16-byte global access -------------------------------------------------
__device__ __forceinline__ u32x4 ld16(const void* p) { return *reinterpret_cast<const u32x4*>(p); }
// Large data that a kernel reads exactly once (the logits of the cross-entropy passes, 0.8 GB): a
// streaming (non-temporal) load, which leaves the caches to what is used again -- forward 195 ->
// 150 us, backward 305 -> 273 us inside the training step.  No difference for the 34-67 MB inputs
// of the normalisation, conversion and reduce passes, which keep plain loads.
__device__ __forceinline__ u32x4 ld16_stream(const void* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
}
// Result stores that cover whole cache lines (a wave writes complete 128-byte row segments) are
// written through L2 at once (device scope) instead of staying dirty in the cache: a kernel then
// ends with less left to write back, and the write traffic runs beside its remaining work
// instead of in a burst after it (0.3-0.7 ms of a 27 ms training step of the 410M model).  Stores
// that fill a line piecewise over several instructions must NOT use these: written through, every
// piece becomes a partial-line write (the same step 2 ms slower with the attention results stored
// this way).  The compiler does not see a store inside an asm statement, so the wait states that
// a store needs before a VALU instruction may overwrite its data registers are part of the
// statement.
__device__ __forceinline__ void st16(void* p, u32x4 v) {
  asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ void st8(void* p, u32x2 v) {
  asm volatile("global_store_dwordx2 %0, %1, off sc1\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
}
// any 8- or 16-byte vector value
template <typename V> __device__ __forceinline__ void store_out(void* p, const V& v) {
  static_assert(sizeof(V) == 8 || sizeof(V) == 16, "8- or 16-byte values");
  if constexpr (sizeof(V) == 16) st16(p, __builtin_bit_cast(u32x4, v));
  else st8(p, __builtin_bit_cast(u32x2, v));
}

template <typename T> __device__ __forceinline__ void unpack8(u32x4 raw, float (&out)[8]) {
  typename Vec<T>::v8 h = __builtin_bit_cast(typename Vec<T>::v8, raw);
#pragma unroll
  for (int i = 0; i < 8; ++i) out[i] = (float)h[i];
}
template <typename T> __device__ __forceinline__ u32x4 pack8(const float (&in)[8]) {
  typename Vec<T>::v8 h;
#pragma unroll
  for (int i = 0; i < 8; ++i) h[i] = (T)in[i];
  return __builtin_bit_cast(u32x4, h);
}

// ---- MFMA 32x32x16, D(32x32 fp32) += A(32x16) * B(16x32) ------------------
// Lane l supplies A[l%32][(l/32)*8 .. +8] and B[(l/32)*8 .. +8][l%32];
// result register r of lane l is D[(r/4)*8 + (l/32)*4 + r%4][l%32].
__device__ __forceinline__ f32x16 mfma32(f16x8 a, f16x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

// ---- LDS access ------------------------------------------------------------
typedef __attribute__((address_space(3))) void lds_void;

__device__ __forceinline__ u32x4 lds_ld16(const char* base, int byte_off) {
  return *reinterpret_cast<const u32x4*>(base + byte_off);
}
__device__ __forceinline__ void lds_st16(char* base, int byte_off, u32x4 v) {
  *reinterpret_cast<u32x4*>(base + byte_off) = v;
}
// Transposing 8-byte LDS read: within each group of 16 lanes, lane i supplies
// the address of 4 consecutive 16-bit elements; viewing the 16 loads as a
// 4x16 matrix (row = i/4, 4 columns per lane), lane j receives column j.
__device__ __forceinline__ u32x2 lds_ld8_tr(const char* base, int byte_off) {
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
  s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(base + byte_off));
  return __builtin_bit_cast(u32x2, v);
}

// ---- LDS reads as volatile asm ---------------------------------------------
// The compiler neither reorders these nor waits for them (and does not make them
// wait for direct-to-LDS global loads it cannot tell apart), so a kernel decides
// how far ahead of their consumers they run.  Every consumer must sit behind
// lds_wait<N>(reg): it waits until at most N later LDS operations are outstanding
// and is tied to the register, so the consumer cannot be scheduled above it.
// A register that was requested must always be waited for before it dies.
__device__ __forceinline__ uint32_t lds_address(const char* p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)p;
}
template <int OFF> __device__ __forceinline__ void lds_read128_at(u32x4& dst, uint32_t addr) {
  static_assert(OFF >= 0, "offset");
  constexpr int IMM = OFF < 65536 ? OFF : OFF % 32768;  // the instruction's offset field is 16 bits
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr + (uint32_t)(OFF - IMM)), "n"(IMM));
}
template <int OFF> __device__ __forceinline__ void lds_read64_tr_at(u32x2& dst, uint32_t addr) {
  static_assert(OFF >= 0, "offset");
  constexpr int IMM = OFF < 65536 ? OFF : OFF % 32768;  // the instruction's offset field is 16 bits
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(dst) : "v"(addr + (uint32_t)(OFF - IMM)), "n"(IMM));
}
template <int OFF> __device__ __forceinline__ void lds_read64_at(u32x2& dst, uint32_t addr) {
  static_assert(OFF >= 0, "offset");
  constexpr int IMM = OFF < 65536 ? OFF : OFF % 32768;  // the instruction's offset field is 16 bits
  asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(dst) : "v"(addr + (uint32_t)(OFF - IMM)), "n"(IMM));
}
template <int OFF> __device__ __forceinline__ void lds_read_u16_at(uint32_t& dst, uint32_t addr) {
  static_assert(OFF >= 0, "offset");
  constexpr int IMM = OFF < 65536 ? OFF : OFF % 32768;
  asm volatile("ds_read_u16 %0, %1 offset:%2" : "=v"(dst) : "v"(addr + (uint32_t)(OFF - IMM)), "n"(IMM));
}
template <int N, typename R> __device__ __forceinline__ void lds_wait(R& reg) {
  static_assert(N >= 0 && N <= 15, "lgkmcnt is 4 bits");
  asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(reg) : "n"(N));
}

// Orders every later use of `reg` after the preceding lds_wait (volatile asm statements keep
// their order): for registers that were requested before the one the wait names and so have
// landed with it.  Emits no instruction.
template <typename R> __device__ __forceinline__ void lds_tie(R& reg) { asm volatile("" : "+v"(reg)); }

// s_waitcnt vmcnt(n) with the other counters unconstrained (gfx9 encoding).
template <int N> __device__ __forceinline__ void wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

// f(std::integral_constant<int, 0>{}), ..., f(std::integral_constant<int, N-1>{})
template <typename F, int... I> __device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F> __device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

inline int ceil_div(int64_t a, int64_t b) { return (int)((a + b - 1) / b); }

// CUs and XCDs of the current device, read from the runtime once per device and kept (the only
// state this library holds besides the scratch array of the allocation-free entry point).  Falls
// back to the MI355X figures if the runtime does not answer.
struct DeviceShape { int cus, xcds; };
DeviceShape device_shape();

}  // namespace tfa
