// Cross-entropy forward/backward for gfx950.  HBM-bound: the forward streams
// each logits row once (online max / sum-of-exp in the log2 domain), the
// backward streams it once more and writes the gradient, already multiplied by
// the upstream per-row gradient.
#include "rowops.h"

namespace tfa {

constexpr int kCeThreads = 256;

// v_exp_f32 as it is: the library exp2f wraps the same instruction in a range check and a rescaling
// (five instructions more per element) that only matter for results below 2^-126, which are
// flushed to zero here -- terms that change neither a sum of exponentials whose largest term is 1
// nor a 16-bit gradient.
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

struct MaxSum {
  float m;  // running max of x*log2e
  float s;  // running sum of exp2(x*log2e - m)
};
__device__ __forceinline__ MaxSum combine(MaxSum a, MaxSum b) {
  const float m = fmaxf(a.m, b.m);
  MaxSum r;
  r.m = m;
  // exp2f(-inf - finite) = 0; both -inf only when both are empty (s = 0).
  r.s = (m == -INFINITY) ? 0.f : a.s * exp2f(a.m - m) + b.s * exp2f(b.m - m);
  return r;
}

__device__ __forceinline__ MaxSum block_combine(MaxSum v, MaxSum* smem) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    MaxSum other;
    other.m = __shfl_xor(v.m, o, 64);
    other.s = __shfl_xor(v.s, o, 64);
    v = combine(v, other);
  }
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) smem[wave] = v;
  __syncthreads();
  MaxSum r = smem[0];
#pragma unroll
  for (int w = 1; w < kCeThreads / 64; ++w) r = combine(r, smem[w]);
  return r;
}

// Row r of the (rows, V) problem lives at (r / inner) * outer + (r % inner) * ld: with
// inner = S-1, ld = V, outer = S*V these are the rows of a (B, S, V) tensor without the
// last position of every sequence, i.e. the shifted logits read in place.
struct RowMap {
  int64_t ld, outer;
  int inner;
  __device__ __forceinline__ int64_t at(int64_t r) const { return (r / inner) * outer + (r % inner) * ld; }
};

template <typename T, bool VEC>
__global__ __launch_bounds__(kCeThreads) void ce_fwd(int V, const T* __restrict__ logits, RowMap map,
                                                      const int64_t* __restrict__ labels, T* __restrict__ loss,
                                                      float* __restrict__ lse) {
  __shared__ MaxSum smem[kCeThreads / 64];
  const int64_t row = blockIdx.x;
  const T* xr = logits + map.at(row);
  MaxSum acc = {-INFINITY, 0.f};
  if (VEC) {
    const int nchunk = V >> 3;
    constexpr int U = 4;  // 16-byte loads in flight per thread
    for (int c0 = threadIdx.x; c0 < nchunk; c0 += U * kCeThreads) {
      u32x4 raw[U];
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (c0 + u * kCeThreads < nchunk) raw[u] = ld16_stream(xr + (c0 + u * kCeThreads) * 8);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (c0 + u * kCeThreads >= nchunk) break;
        float v[8];
        unpack8<T>(raw[u], v);
        float cm = v[0];
#pragma unroll
        for (int e = 1; e < 8; ++e) cm = fmaxf(cm, v[e]);
        cm *= kLog2e;
        if (cm > acc.m) { acc.s *= exp2f(acc.m - cm); acc.m = cm; }
        float part = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) part += fast_exp2(v[e] * kLog2e - acc.m);
        acc.s += part;
      }
    }
  } else {
    for (int c = threadIdx.x; c < V; c += kCeThreads) {
      const float t = (float)xr[c] * kLog2e;
      if (t > acc.m) { acc.s *= exp2f(acc.m - t); acc.m = t; }
      acc.s += exp2f(t - acc.m);
    }
  }
  const MaxSum tot = block_combine(acc, smem);
  if (threadIdx.x == 0) {
    const float l = (tot.m + log2f(tot.s)) * kLn2;  // natural-log logsumexp
    lse[row] = l;
    const int64_t lab = labels[row];
    const float xl = (lab >= 0 && lab < V) ? (float)xr[lab] : 0.f;
    loss[row] = (T)(l - xl);
  }
}

// Forward for rows that fit into the registers of one workgroup (V <= 8 * NCH * kCeThreads): a
// thread requests all of its NCH 16-byte chunks at once -- NCH loads in flight instead of four --
// takes the row maximum first and then the sum of exponentials, both from registers.
// GRAD: the same pass also writes (softmax(row) - onehot(label)) * grad_scale to the row of
// `dlogits` -- the row is still in registers once its log-sum-exp is known, so the gradient of
// the loss with respect to the logits costs one write instead of a second read-and-write pass.
template <typename T, int NCH, bool GRAD>
__global__ __launch_bounds__(kCeThreads) void ce_fwd_regs(int V, const T* __restrict__ logits, RowMap map,
                                                           const int64_t* __restrict__ labels, T* __restrict__ loss,
                                                           float* __restrict__ lse, T* __restrict__ dlogits,
                                                           RowMap dmap, float grad_scale) {
  __shared__ float red[2][kCeThreads / 64];
  const int64_t row = blockIdx.x;
  const T* xr = logits + map.at(row);
  const int nchunk = V >> 3;
  u32x4 raw[NCH];
#pragma unroll
  for (int u = 0; u < NCH; ++u) {
    const int c = threadIdx.x + u * kCeThreads;
    if (c < nchunk) raw[u] = ld16_stream(xr + c * 8);
  }
  float m = -INFINITY;
#pragma unroll
  for (int u = 0; u < NCH; ++u) {
    if (threadIdx.x + u * kCeThreads < nchunk) {
      float v[8];
      unpack8<T>(raw[u], v);
#pragma unroll
      for (int e = 0; e < 8; ++e) m = fmaxf(m, v[e]);
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) red[0][wave] = m;
  __syncthreads();
  m = red[0][0];
#pragma unroll
  for (int w = 1; w < kCeThreads / 64; ++w) m = fmaxf(m, red[0][w]);
  const float m2 = m * kLog2e;
  float s = 0.f;
#pragma unroll
  for (int u = 0; u < NCH; ++u) {
    if (threadIdx.x + u * kCeThreads < nchunk) {
      float v[8];
      unpack8<T>(raw[u], v);
      float part = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) part += fast_exp2(v[e] * kLog2e - m2);
      s += part;
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
  if ((threadIdx.x & 63) == 0) red[1][wave] = s;
  __syncthreads();
  float tot = red[1][0];
#pragma unroll
  for (int w = 1; w < kCeThreads / 64; ++w) tot += red[1][w];
  const float l = (m2 + log2f(tot)) * kLn2;  // natural-log logsumexp
  // back to the log2 domain exactly as the backward kernel does from the stored value: the
  // gradient written here equals the one ce_bwd would produce, bit for bit
  const float l2 = l * kLog2e;
  const int64_t lab = labels[row];
  if (threadIdx.x == 0) {
    lse[row] = l;
    const float xl = (lab >= 0 && lab < V) ? (float)xr[lab] : 0.f;
    loss[row] = (T)(l - xl);
  }
  if constexpr (GRAD) {
    T* dr = dlogits + dmap.at(row);
    const int lab_chunk = (lab >= 0 && lab < V) ? (int)(lab >> 3) : -1;
#pragma unroll
    for (int u = 0; u < NCH; ++u) {
      const int c = threadIdx.x + u * kCeThreads;
      if (c < nchunk) {
        float v[8];
        unpack8<T>(raw[u], v);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = fast_exp2(v[e] * kLog2e - l2);
        if (c == lab_chunk) {
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] -= (e == (int)(lab & 7)) ? 1.0f : 0.0f;
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] *= grad_scale;
        Chunk<T>::store(dr + c * 8, v);
      }
    }
  }
}

template <typename T, bool VEC>
__global__ __launch_bounds__(kCeThreads) void ce_bwd(int V, const T* __restrict__ logits, RowMap map,
                                                      const int64_t* __restrict__ labels,
                                                      const float* __restrict__ lse, const T* __restrict__ gout,
                                                      int64_t gstride, T* __restrict__ dlogits, RowMap dmap) {
  const int64_t row = blockIdx.x;
  const T* xr = logits + map.at(row);
  T* dr = dlogits + dmap.at(row);
  const float l2 = lse[row] * kLog2e;
  const float g = (float)gout[row * gstride];
  const int lab = (int)labels[row];
  if (VEC) {
    const int nchunk = V >> 3;
    for (int c = threadIdx.x; c < nchunk; c += kCeThreads) {
      float v[8];
      Chunk<T>::load_stream(xr + c * 8, v);
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = fast_exp2(v[e] * kLog2e - l2);
      if ((lab >> 3) == c) {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] -= (e == (lab & 7)) ? 1.0f : 0.0f;
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] *= g;
      Chunk<T>::store(dr + c * 8, v);
    }
  } else {
    for (int c = threadIdx.x; c < V; c += kCeThreads) {
      float p = exp2f((float)xr[c] * kLog2e - l2);
      if (c == lab) p -= 1.0f;
      dr[c] = (T)(p * g);
    }
  }
}

template <typename T>
static int ce_fwd_launch(hipStream_t st, int64_t rows, int64_t V, const void* logits, RowMap map,
                         const int64_t* labels, void* loss, float* lse) {
  const dim3 grid((unsigned)rows), block(kCeThreads);
  const RowMap none = {0, 0, 1};
  if (row_vectorizable<T>(logits, V, map.ld) && map.outer % 8 == 0) {
    const int64_t per_thread = (V / 8 + kCeThreads - 1) / kCeThreads;  // 16-byte chunks per thread
#define CE_REGS(NCH) \
  ce_fwd_regs<T, NCH, false><<<grid, block, 0, st>>>((int)V, (const T*)logits, map, labels, (T*)loss, lse, nullptr, none, 0.f)
    if (per_thread <= 8) CE_REGS(8);
    else if (per_thread <= 16) CE_REGS(16);
    else if (per_thread <= 25) CE_REGS(25);
    else ce_fwd<T, true><<<grid, block, 0, st>>>((int)V, (const T*)logits, map, labels, (T*)loss, lse);
#undef CE_REGS
  } else
    ce_fwd<T, false><<<grid, block, 0, st>>>((int)V, (const T*)logits, map, labels, (T*)loss, lse);
  TF_CHECK_LAUNCH();
  return TF_OK;
}

template <typename T>
static int ce_bwd_launch(hipStream_t st, int64_t rows, int64_t V, const void* logits, RowMap map,
                         const int64_t* labels, const float* lse, const void* gout, int64_t gstride,
                         void* dlogits, RowMap dmap) {
  const dim3 grid((unsigned)rows), block(kCeThreads);
  if (row_vectorizable<T>(logits, V, map.ld) && row_vectorizable<T>(dlogits, V, dmap.ld) && map.outer % 8 == 0 &&
      dmap.outer % 8 == 0)
    ce_bwd<T, true><<<grid, block, 0, st>>>((int)V, (const T*)logits, map, labels, lse, (const T*)gout, gstride,
                                            (T*)dlogits, dmap);
  else
    ce_bwd<T, false><<<grid, block, 0, st>>>((int)V, (const T*)logits, map, labels, lse, (const T*)gout, gstride,
                                             (T*)dlogits, dmap);
  TF_CHECK_LAUNCH();
  return TF_OK;
}

// Forward that also leaves (softmax - onehot) * grad_scale in dlogits: one kernel when the row fits
// the registers of a workgroup and both matrices can be accessed in 16-byte chunks, else the forward
// followed by the backward kernel with `scale_dev` (one value of T in device memory holding
// grad_scale) as the upstream gradient of every row -- the same values either way.
template <typename T>
static int ce_fwd_grad_launch(hipStream_t st, int64_t rows, int64_t V, const void* logits, RowMap map,
                              const int64_t* labels, void* loss, float* lse, void* dlogits, RowMap dmap,
                              float grad_scale, const void* scale_dev) {
  const dim3 grid((unsigned)rows), block(kCeThreads);
  const int64_t per_thread = (V / 8 + kCeThreads - 1) / kCeThreads;
  if (row_vectorizable<T>(logits, V, map.ld) && map.outer % 8 == 0 && row_vectorizable<T>(dlogits, V, dmap.ld) &&
      dmap.outer % 8 == 0 && per_thread <= 25) {
#define CE_REGS(NCH)                                                                                               \
  ce_fwd_regs<T, NCH, true><<<grid, block, 0, st>>>((int)V, (const T*)logits, map, labels, (T*)loss, lse, (T*)dlogits, \
                                                    dmap, grad_scale)
    if (per_thread <= 8) CE_REGS(8);
    else if (per_thread <= 16) CE_REGS(16);
    else CE_REGS(25);
#undef CE_REGS
    TF_CHECK_LAUNCH();
    return TF_OK;
  }
  if (!scale_dev) return TF_EINVAL;
  const int rc = ce_fwd_launch<T>(st, rows, V, logits, map, labels, loss, lse);
  if (rc != TF_OK) return rc;
  return ce_bwd_launch<T>(st, rows, V, logits, map, labels, lse, scale_dev, 0, dlogits, dmap);
}

}  // namespace tfa

using namespace tfa;

static bool make_map(RowMap& m, int64_t rows, int64_t V, int64_t ld, int64_t inner, int64_t outer) {
  if (inner <= 0) { inner = rows > 0 ? rows : 1; outer = 0; }
  if (ld < V || inner > 0x7fffffff || outer < 0 || (inner < rows && outer < (inner - 1) * ld + V)) return false;
  m.ld = ld; m.outer = outer; m.inner = (int)inner;
  return true;
}

extern "C" int tf_cross_entropy_fwd(void* stream, int dtype, int64_t rows, int64_t V, const void* logits,
                                    int64_t ld, int64_t inner_rows, int64_t outer_stride, const int64_t* labels,
                                    void* loss, float* lse) {
  if (!logits || !labels || !loss || !lse) return TF_EINVAL;
  if (rows < 0 || rows > 0x7fffffff || V <= 0 || V > (1 << 30)) return TF_EINVAL;
  RowMap map;
  if (!make_map(map, rows, V, ld, inner_rows, outer_stride)) return TF_EINVAL;
  if (rows == 0) return TF_OK;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == TF_F16) return ce_fwd_launch<f16>(st, rows, V, logits, map, labels, loss, lse);
  if (dtype == TF_BF16) return ce_fwd_launch<bf16>(st, rows, V, logits, map, labels, loss, lse);
  return TF_EDTYPE;
}

extern "C" int tf_cross_entropy_bwd(void* stream, int dtype, int64_t rows, int64_t V, const void* logits,
                                    int64_t ld, int64_t inner_rows, int64_t outer_stride, const int64_t* labels,
                                    const float* lse, const void* gout, int64_t gout_stride, void* dlogits,
                                    int64_t ldd, int64_t outer_stride_d) {
  if (!logits || !labels || !lse || !gout || !dlogits) return TF_EINVAL;
  if (rows < 0 || rows > 0x7fffffff || V <= 0 || V > (1 << 30) || gout_stride < 0) return TF_EINVAL;
  RowMap map, dmap;
  if (!make_map(map, rows, V, ld, inner_rows, outer_stride)) return TF_EINVAL;
  if (!make_map(dmap, rows, V, ldd, inner_rows, outer_stride_d)) return TF_EINVAL;
  if (rows == 0) return TF_OK;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == TF_F16)
    return ce_bwd_launch<f16>(st, rows, V, logits, map, labels, lse, gout, gout_stride, dlogits, dmap);
  if (dtype == TF_BF16)
    return ce_bwd_launch<bf16>(st, rows, V, logits, map, labels, lse, gout, gout_stride, dlogits, dmap);
  return TF_EDTYPE;
}

extern "C" int tf_cross_entropy_fwd_grad(void* stream, int dtype, int64_t rows, int64_t V, const void* logits,
                                         int64_t ld, int64_t inner_rows, int64_t outer_stride, const int64_t* labels,
                                         void* loss, float* lse, void* dlogits, int64_t ldd, int64_t outer_stride_d,
                                         float grad_scale, const void* grad_scale_dev) {
  if (!logits || !labels || !loss || !lse || !dlogits) return TF_EINVAL;
  if (rows < 0 || rows > 0x7fffffff || V <= 0 || V > (1 << 30)) return TF_EINVAL;
  RowMap map, dmap;
  if (!make_map(map, rows, V, ld, inner_rows, outer_stride)) return TF_EINVAL;
  if (!make_map(dmap, rows, V, ldd, inner_rows, outer_stride_d)) return TF_EINVAL;
  if (dtype != TF_F16 && dtype != TF_BF16) return TF_EDTYPE;
  if (rows == 0) return TF_OK;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == TF_F16)
    return ce_fwd_grad_launch<f16>(st, rows, V, logits, map, labels, loss, lse, dlogits, dmap, grad_scale, grad_scale_dev);
  return ce_fwd_grad_launch<bf16>(st, rows, V, logits, map, labels, loss, lse, dlogits, dmap, grad_scale, grad_scale_dev);
}
