// Row-wise helpers shared by the bandwidth-bound kernels: 16-byte chunks of a
// row converted to fp32, for 16-bit and 32-bit element types.
#pragma once
#include "common.h"

namespace tfa {

template <typename T> struct Chunk {  // 16-bit types: 8 elements per 16 bytes
  static constexpr int N = 8;
  static __device__ __forceinline__ void load(const T* p, float (&v)[8]) { unpack8<T>(ld16(p), v); }
  static __device__ __forceinline__ void load_stream(const T* p, float (&v)[8]) { unpack8<T>(ld16_stream(p), v); }
  static __device__ __forceinline__ void store(T* p, const float (&v)[8]) { st16(p, pack8<T>(v)); }
};
template <> struct Chunk<float> {
  static constexpr int N = 4;
  static __device__ __forceinline__ void load(const float* p, float (&v)[4]) {
    f32x4 r = *reinterpret_cast<const f32x4*>(p);
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = r[i];
  }
  static __device__ __forceinline__ void load_stream(const float* p, float (&v)[4]) {
    f32x4 r = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p));
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = r[i];
  }
  static __device__ __forceinline__ void store(float* p, const float (&v)[4]) {
    f32x4 r;
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = v[i];
    store_out(p, r);
  }
};

// 8 consecutive elements as fp32; TP = a 16-bit type or float (fp32 master parameters are
// read as they are, no 16-bit copy is made first).
template <typename TP> __device__ __forceinline__ void load8(const TP* p, float (&v)[8]) { Chunk<TP>::load(p, v); }
template <> __device__ __forceinline__ void load8<float>(const float* p, float (&v)[8]) {
  float a[4], b[4];
  Chunk<float>::load(p, a);
  Chunk<float>::load(p + 4, b);
#pragma unroll
  for (int i = 0; i < 4; ++i) { v[i] = a[i]; v[4 + i] = b[i]; }
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// True when rows of `n` elements of T starting at p with leading dimension ld
// can be read as whole 16-byte chunks.
template <typename T> inline bool row_vectorizable(const void* p, int64_t n, int64_t ld) {
  const int per = 16 / (int)sizeof(T);
  return aligned16(p) && (n % per == 0) && (ld % per == 0);
}

#define TF_CHECK_LAUNCH()                                      \
  do {                                                         \
    if (hipGetLastError() != hipSuccess) return TF_ELAUNCH;    \
  } while (0)

}  // namespace tfa
