// Column sums (bias gradient) and the ReLU gradient mask for gfx950; both are
// HBM-bound streaming kernels with 16-byte accesses.
#include <atomic>
#include "rowops.h"

namespace tfa {

// Scratch of the allocation-free column sum (tf_colsum_noalloc): the first-stage partial sums live
// here instead of in a buffer the caller brings.  One copy per GPU the library runs on, held until
// the process ends.  In host code the array's name is only a handle for hipGetSymbolAddress; the
// device address it yields is what kernels and copies are given.
constexpr int64_t kNoAllocScratchBytes = 4 << 20;
static __device__ __align__(256) float scratch[kNoAllocScratchBytes / sizeof(float)];

constexpr int kCsColsPerBlock = 256;  // 32 lanes x 8 elements
constexpr int kCsSlices = 8;          // row slices per workgroup

static int colsum_groups(int64_t rows, int64_t cols) {
  const int64_t col_blocks = (cols + kCsColsPerBlock - 1) / kCsColsPerBlock;
  int64_t want = (2048 + col_blocks - 1) / col_blocks;  // aim for ~2048 workgroups
  const int64_t max_groups = (rows + 4 * kCsSlices - 1) / (4 * kCsSlices);  // >= 4 rows per slice
  if (want > max_groups) want = max_groups;
  if (want < 1) want = 1;
  return (int)want;
}

// grid (col_blocks, groups).  Thread (slice, lane32) sums 8 adjacent columns
// over rows  group_begin + slice, + 8, ...; slices are combined through LDS.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void colsum_partial(int64_t rows, int cols, const T* __restrict__ x, int64_t ldx,
                                                       float* __restrict__ partial, int rows_per_group) {
  __shared__ float red[kCsSlices][kCsColsPerBlock];
  const int lane32 = threadIdx.x & 31;
  const int slice = threadIdx.x >> 5;
  const int col0 = blockIdx.x * kCsColsPerBlock + lane32 * 8;
  const int64_t rbeg = (int64_t)blockIdx.y * rows_per_group;
  int64_t rend = rbeg + rows_per_group;
  if (rend > rows) rend = rows;
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  if (VEC) {
    if (col0 < cols) {
      for (int64_t r = rbeg + slice; r < rend; r += kCsSlices) {
        float v[8];
        Chunk<T>::load(x + r * ldx + col0, v);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] += v[e];
      }
    }
  } else {
    for (int64_t r = rbeg + slice; r < rend; r += kCsSlices) {
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (col0 + e < cols) acc[e] += (float)x[r * ldx + col0 + e];
    }
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) red[slice][lane32 * 8 + e] = acc[e];
  __syncthreads();
  const int c = blockIdx.x * kCsColsPerBlock + threadIdx.x;
  if (c < cols) {
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < kCsSlices; ++k) s += red[k][threadIdx.x];
    partial[(int64_t)blockIdx.y * cols + c] = s;
  }
}

// Second stage: out[c] = sum over groups of partial[g][c], in a fixed order.  A workgroup takes 32
// columns; its 8 slices of 32 lanes each add up every 8th group (independent loads in flight
// instead of one dependent chain per column), then the slices are combined through LDS.
template <typename T>
__global__ __launch_bounds__(256) void colsum_final(int groups, int cols, const float* __restrict__ partial,
                                                     T* __restrict__ out) {
  __shared__ float red[8][32];
  const int lane32 = threadIdx.x & 31, slice = threadIdx.x >> 5;
  const int c = blockIdx.x * 32 + lane32;
  float s0 = 0.f, s1 = 0.f;
  if (c < cols) {
    int g = slice;
    for (; g + 8 < groups; g += 16) {
      s0 += partial[(int64_t)g * cols + c];
      s1 += partial[(int64_t)(g + 8) * cols + c];
    }
    if (g < groups) s0 += partial[(int64_t)g * cols + c];
  }
  red[slice][lane32] = s0 + s1;
  __syncthreads();
  if (slice == 0 && c < cols) {
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < 8; ++k) s += red[k][lane32];
    out[c] = (T)s;
  }
}

template <typename T, bool VEC>
__global__ __launch_bounds__(256) void relu_mask_kernel(int64_t rows, int cols, const T* __restrict__ grad,
                                                         int64_t ldg, const T* __restrict__ act, int64_t lda,
                                                         T* __restrict__ out, int64_t ldo) {
  if (VEC) {
    const int cpr = cols >> 3;
    const int64_t total = rows * cpr;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
      const int64_t r = i / cpr;
      const int c = (int)(i - r * cpr) * 8;
      float g[8], a[8];
      Chunk<T>::load(grad + r * ldg + c, g);
      Chunk<T>::load(act + r * lda + c, a);
#pragma unroll
      for (int e = 0; e < 8; ++e) g[e] = a[e] > 0.f ? g[e] : 0.f;
      Chunk<T>::store(out + r * ldo + c, g);
    }
  } else {
    const int64_t total = rows * cols;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
      const int64_t r = i / cols;
      const int c = (int)(i - r * cols);
      out[r * ldo + c] = (float)act[r * lda + c] > 0.f ? grad[r * ldg + c] : (T)0.f;
    }
  }
}

template <typename T>
static int colsum_launch(hipStream_t st, int64_t rows, int64_t cols, const void* x, int64_t ldx, void* out,
                         bool out_f32, float* partial) {
  const int groups = colsum_groups(rows, cols);
  const int rpg = (int)((rows + groups - 1) / groups);
  const dim3 grid((unsigned)ceil_div(cols, kCsColsPerBlock), (unsigned)groups), block(256);
  if (row_vectorizable<T>(x, cols, ldx))
    colsum_partial<T, true><<<grid, block, 0, st>>>(rows, (int)cols, (const T*)x, ldx, partial, rpg);
  else
    colsum_partial<T, false><<<grid, block, 0, st>>>(rows, (int)cols, (const T*)x, ldx, partial, rpg);
  TF_CHECK_LAUNCH();
  if (out_f32) colsum_final<float><<<dim3(ceil_div(cols, 32)), block, 0, st>>>(groups, (int)cols, partial, (float*)out);
  else colsum_final<T><<<dim3(ceil_div(cols, 32)), block, 0, st>>>(groups, (int)cols, partial, (T*)out);
  TF_CHECK_LAUNCH();
  return TF_OK;
}

template <typename T>
static int relu_mask_launch(hipStream_t st, int64_t rows, int64_t cols, const void* grad, int64_t ldg,
                            const void* act, int64_t lda, void* out, int64_t ldo) {
  const bool vec =
      row_vectorizable<T>(grad, cols, ldg) && row_vectorizable<T>(act, cols, lda) && row_vectorizable<T>(out, cols, ldo);
  const int64_t work = vec ? rows * (cols / 8) : rows * cols;
  int64_t blocks = (work + 255) / 256;
  if (blocks > 256 * 32) blocks = 256 * 32;
  if (blocks < 1) blocks = 1;
  if (vec)
    relu_mask_kernel<T, true><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(rows, (int)cols, (const T*)grad, ldg,
                                                                            (const T*)act, lda, (T*)out, ldo);
  else
    relu_mask_kernel<T, false><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(rows, (int)cols, (const T*)grad, ldg,
                                                                             (const T*)act, lda, (T*)out, ldo);
  TF_CHECK_LAUNCH();
  return TF_OK;
}

// ---------------------------------------------------------------------------
// Convert up to four (rows, cols) matrices to 16 bits, side by side in one matrix.
// ---------------------------------------------------------------------------
struct PackSources { const void* p[4]; };

template <typename TI, typename TO, bool VEC>
__global__ __launch_bounds__(256) void cast_pack(PackSources src, int count, int64_t rows, int cols, int64_t ld_src,
                                                  TO* __restrict__ dst, int64_t ld_dst) {
  const int per_row = VEC ? cols >> 3 : cols;  // work items per source row
  const int64_t total = rows * count * per_row;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int c = (int)(i % per_row);
    const int64_t rj = i / per_row;
    const int j = (int)(rj % count);
    const int64_t r = rj / count;
    const TI* s = (const TI*)src.p[j] + r * ld_src;
    TO* d = dst + r * ld_dst + (int64_t)j * cols;
    if (VEC) {
      float v[8];
      load8<TI>(s + c * 8, v);
      Chunk<TO>::store(d + c * 8, v);
    } else {
      d[c] = (TO)(float)s[c];
    }
  }
}

template <typename TI, typename TO>
static int cast_pack_launch(hipStream_t st, int count, int64_t rows, int64_t cols, const void* const* srcs,
                            int64_t ld_src, void* dst, int64_t ld_dst) {
  PackSources ps = {};
  bool vec = cols % 8 == 0 && ld_src % 8 == 0 && ld_dst % 8 == 0 && aligned16(dst);
  for (int j = 0; j < count; ++j) { ps.p[j] = srcs[j]; vec = vec && aligned16(srcs[j]); }
  const int64_t items = rows * count * (vec ? cols / 8 : cols);
  int64_t blocks = (items + 255) / 256;
  if (blocks > 8192) blocks = 8192;
  if (vec) cast_pack<TI, TO, true><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(ps, count, rows, (int)cols, ld_src, (TO*)dst, ld_dst);
  else cast_pack<TI, TO, false><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(ps, count, rows, (int)cols, ld_src, (TO*)dst, ld_dst);
  TF_CHECK_LAUNCH();
  return TF_OK;
}

}  // namespace tfa

using namespace tfa;

extern "C" int64_t tf_colsum_partial_bytes(int64_t rows, int64_t cols) {
  if (rows <= 0 || cols <= 0) return 0;
  return (int64_t)colsum_groups(rows, cols) * cols * (int64_t)sizeof(float);
}

extern "C" int tf_colsum(void* stream, int dtype, int out_dtype, int64_t rows, int64_t cols, const void* x,
                         int64_t ldx, void* out, float* partial, int64_t partial_bytes) {
  if (!x || !out) return TF_EINVAL;
  if (rows <= 0 || cols <= 0 || cols > (1 << 30) || ldx < cols) return TF_EINVAL;
  if (dtype != TF_F16 && dtype != TF_BF16) return TF_EDTYPE;
  if (out_dtype != dtype && out_dtype != TF_F32) return TF_EDTYPE;
  if (!partial || partial_bytes < tf_colsum_partial_bytes(rows, cols)) return TF_EWORKSPACE;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == TF_F16) return colsum_launch<f16>(st, rows, cols, x, ldx, out, out_dtype == TF_F32, partial);
  return colsum_launch<bf16>(st, rows, cols, x, ldx, out, out_dtype == TF_F32, partial);
}

// Device address of `scratch` on the current device, looked up once per device (with that device
// current) and kept.  Returns null if the runtime refuses.
static float* noalloc_scratch() {
  constexpr int kMaxDevices = 64;
  static std::atomic<float*> ptrs[kMaxDevices];
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  float* p = ptrs[dev].load(std::memory_order_acquire);
  if (!p) {
    void* addr = nullptr;
    if (hipGetSymbolAddress(&addr, HIP_SYMBOL(scratch)) != hipSuccess || !addr) {
      (void)hipGetLastError();
      return nullptr;
    }
    p = static_cast<float*>(addr);
    ptrs[dev].store(p, std::memory_order_release);  // every thread finds the same address
  }
  return p;
}

extern "C" int64_t tf_colsum_noalloc_max_partial_bytes(void) { return kNoAllocScratchBytes; }

extern "C" int tf_colsum_noalloc(void* stream, int dtype, int out_dtype, int64_t rows, int64_t cols, const void* x,
                                 int64_t ldx, void* out) {
  if (!x || !out) return TF_EINVAL;
  if (rows <= 0 || cols <= 0 || cols > (1 << 30) || ldx < cols) return TF_EINVAL;
  if (dtype != TF_F16 && dtype != TF_BF16) return TF_EDTYPE;
  if (out_dtype != dtype && out_dtype != TF_F32) return TF_EDTYPE;
  if (tf_colsum_partial_bytes(rows, cols) > kNoAllocScratchBytes) return TF_EWORKSPACE;  // beyond the fixed scratch
  float* partial = noalloc_scratch();
  if (!partial) return TF_ELAUNCH;
  hipStream_t st = (hipStream_t)stream;
  // every partial sum the second stage reads is written by the first stage of the same call:
  // nothing has to start at zero, whatever an earlier (larger) call left behind
  if (dtype == TF_F16) return colsum_launch<f16>(st, rows, cols, x, ldx, out, out_dtype == TF_F32, partial);
  return colsum_launch<bf16>(st, rows, cols, x, ldx, out, out_dtype == TF_F32, partial);
}

extern "C" int tf_relu_mask(void* stream, int dtype, int64_t rows, int64_t cols, const void* grad, int64_t ldg,
                            const void* act, int64_t lda, void* out, int64_t ldo) {
  if (!grad || !act || !out) return TF_EINVAL;
  if (rows < 0 || cols <= 0 || cols > (1 << 30) || ldg < cols || lda < cols || ldo < cols) return TF_EINVAL;
  if (rows == 0) return TF_OK;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == TF_F16) return relu_mask_launch<f16>(st, rows, cols, grad, ldg, act, lda, out, ldo);
  if (dtype == TF_BF16) return relu_mask_launch<bf16>(st, rows, cols, grad, ldg, act, lda, out, ldo);
  return TF_EDTYPE;
}

extern "C" int tf_cast_pack(void* stream, int src_dtype, int dst_dtype, int count, int64_t rows, int64_t cols,
                            const void* const* srcs, int64_t ld_src, void* dst, int64_t ld_dst) {
  if (!srcs || !dst || count < 1 || count > 4) return TF_EINVAL;
  for (int j = 0; j < count; ++j)
    if (!srcs[j]) return TF_EINVAL;
  if (rows < 0 || cols <= 0 || cols > (1 << 30) || ld_src < cols || ld_dst < count * cols) return TF_EINVAL;
  if (dst_dtype != TF_F16 && dst_dtype != TF_BF16) return TF_EDTYPE;
  if (src_dtype != TF_F32 && src_dtype != dst_dtype) return TF_EDTYPE;
  if (rows == 0) return TF_OK;
  hipStream_t st = (hipStream_t)stream;
  if (dst_dtype == TF_F16)
    return src_dtype == TF_F32 ? cast_pack_launch<float, f16>(st, count, rows, cols, srcs, ld_src, dst, ld_dst)
                               : cast_pack_launch<f16, f16>(st, count, rows, cols, srcs, ld_src, dst, ld_dst);
  return src_dtype == TF_F32 ? cast_pack_launch<float, bf16>(st, count, rows, cols, srcs, ld_src, dst, ld_dst)
                             : cast_pack_launch<bf16, bf16>(st, count, rows, cols, srcs, ld_src, dst, ld_dst);
}
