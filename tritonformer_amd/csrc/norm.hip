// LayerNorm forward/backward and row softmax forward/backward for gfx950.
// All four are HBM-bound: one wave64 owns one row, holds it in registers as
// 16-byte chunks (chunk c of the row belongs to lane c % 64), and reduces with
// cross-lane shuffles, so every element is read from HBM exactly once.
#include "rowops.h"

namespace tfa {

constexpr int kRowsPerBlock = 4;  // 4 waves per workgroup, one row each
#ifndef TF_LN_FWD_ROWS
#define TF_LN_FWD_ROWS 2
#endif
constexpr int kLnFwdRowsPerWave = TF_LN_FWD_ROWS;  // rows a wave of the forward kernel walks (with the next one in flight)

// ---------------------------------------------------------------------------
// LayerNorm forward.  NV = 16-byte chunks per lane (row length <= NV*64*8).
// ---------------------------------------------------------------------------
// With ADD the normalised row is s = x + res, rounded to T and also written to `sum`
// (the residual stream after the addition); the statistics are those of the rounded s,
// so the result equals an addition kernel followed by the plain forward.
template <typename T, typename TP, int NV, bool ADD>
__global__ __launch_bounds__(256) void ln_fwd_vec(int64_t rows, int d, const T* __restrict__ x, int64_t ldx,
                                                   const T* __restrict__ res, int64_t ldres,
                                                   T* __restrict__ sum, int64_t ldsum,
                                                   const TP* __restrict__ gamma, const TP* __restrict__ beta,
                                                   float eps, T* __restrict__ y, int64_t ldy,
                                                   float* __restrict__ mean_out, float* __restrict__ rstd_out) {
  // Wave w of workgroup b walks rows (b*4 + w) + k*4*grid.  The raw chunks of the wave's next row
  // are requested before the cross-lane sums of the current one, so that the reads of one row run
  // beside the reductions and the stores of the row before: with one row per wave and every wave
  // of the launch resident at once, the whole launch reads first and writes afterwards, and
  // neither half of the memory system's time is used by the other.
  // The add + LayerNorm instantiation must give the bits of an addition followed by the plain one:
  // no contraction left to the compiler (it may fuse differently per instantiation), the fused
  // operations are spelled out.
#pragma clang fp contract(off)
  const int lane = threadIdx.x & 63;
  const int nchunk = d >> 3;
  const int64_t stride = (int64_t)gridDim.x * kRowsPerBlock;
  u32x4 raw_x[NV], raw_r[ADD ? NV : 1];
  auto fetch = [&](int64_t row) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int c = lane + i * 64;
      if (c < nchunk) {
        raw_x[i] = ld16(x + row * ldx + c * 8);
        if (ADD) raw_r[i] = ld16(res + row * ldres + c * 8);
      }
    }
  };
  int64_t row = (int64_t)blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6);
  if (row < rows) fetch(row);
  for (; row < rows; row += stride) {
    float v[NV][8];
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int c = lane + i * 64;
      if (c < nchunk) {
        unpack8<T>(raw_x[i], v[i]);
        if (ADD) {
          float r[8];
          unpack8<T>(raw_r[i], r);
#pragma unroll
          for (int e = 0; e < 8; ++e) v[i][e] += r[e];
          const u32x4 packed = pack8<T>(v[i]);
          st16(sum + row * ldsum + c * 8, packed);
          unpack8<T>(packed, v[i]);
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) s += v[i][e];
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[i][e] = 0.f;
      }
    }
    if (row + stride < rows) fetch(row + stride);
    const float mean = wave_sum(s) / (float)d;
    float q = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      if (lane + i * 64 < nchunk) {
#pragma unroll
        for (int e = 0; e < 8; ++e) { const float t = v[i][e] - mean; q = __builtin_fmaf(t, t, q); }
      }
    }
    const float var = wave_sum(q) / (float)d;
    const float rstd = 1.0f / sqrtf(var + eps);
    if (lane == 0) { mean_out[row] = mean; rstd_out[row] = rstd; }
    T* yr = y + row * ldy;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int c = lane + i * 64;
      if (c < nchunk) {
        // (gamma and beta are fetched per row: held in registers across the rows a wave walks they
        // cost a wave of occupancy, 98 against 86 VGPRs, and the kernel 0.5 us at d = 1024)
        float g[8], b[8], o[8];
        load8<TP>(gamma + c * 8, g);
        load8<TP>(beta + c * 8, b);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          o[e] = __builtin_fmaf((v[i][e] - mean) * rstd, g[e], b[e]);
          // the fp32 value is pinned before the rounding to 16 bits: left alone, the compiler turns
          // some of these into v_fma_mix*_f16 (one rounding straight to 16 bits) and others not,
          // differently per instantiation, and the two forms differ in one element in 50 000
          asm("" : "+v"(o[e]));
        }
        Chunk<T>::store(yr + c * 8, o);
      }
    }
  }
}

// Any row length / alignment: scalar loads, three passes over the row (the
// second and third come from cache).
template <typename T, typename TP, bool ADD>
__global__ __launch_bounds__(256) void ln_fwd_any(int64_t rows, int d, const T* __restrict__ x, int64_t ldx,
                                                   const T* __restrict__ res, int64_t ldres,
                                                   T* __restrict__ sum, int64_t ldsum,
                                                   const TP* __restrict__ gamma, const TP* __restrict__ beta,
                                                   float eps, T* __restrict__ y, int64_t ldy,
                                                   float* __restrict__ mean_out, float* __restrict__ rstd_out) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6);
  if (row >= rows) return;
  const T* xr = x + row * ldx;
  if (ADD) {
    // every lane re-reads only the columns it wrote itself
    T* sr = sum + row * ldsum;
    for (int c = lane; c < d; c += 64) sr[c] = (T)((float)xr[c] + (float)res[row * ldres + c]);
    xr = sr;
  }
  float s = 0.f;
  for (int c = lane; c < d; c += 64) s += (float)xr[c];
  const float mean = wave_sum(s) / (float)d;
  float q = 0.f;
  for (int c = lane; c < d; c += 64) { const float t = (float)xr[c] - mean; q += t * t; }
  const float rstd = 1.0f / sqrtf(wave_sum(q) / (float)d + eps);
  if (lane == 0) { mean_out[row] = mean; rstd_out[row] = rstd; }
  T* yr = y + row * ldy;
  for (int c = lane; c < d; c += 64)
    yr[c] = (T)__builtin_fmaf(((float)xr[c] - mean) * rstd, (float)gamma[c], (float)beta[c]);
}

// ---------------------------------------------------------------------------
// LayerNorm backward.  Wave w of workgroup b walks rows (b*4 + w) + k*4*grid.
// dx is written per row; dgamma/dbeta partial sums stay in registers, are
// summed over the 4 waves through LDS and land in partial[b][0|1][d].
// The raw 16-byte chunks of the wave's next row are requested before the
// cross-lane sums of the current row, so a wave always has loads in flight.
// With ADD, dsum (the gradient that reaches the normalised tensor by another
// path, e.g. along a residual stream) is added to dx before the rounding.
// ---------------------------------------------------------------------------
template <typename T, typename TP, int NV, bool ADD>
__global__ __launch_bounds__(256) void ln_bwd_vec(int64_t rows, int d, const T* __restrict__ dy, int64_t lddy,
                                                   const T* __restrict__ dsum, int64_t lddsum,
                                                   const T* __restrict__ x, int64_t ldx,
                                                   const TP* __restrict__ gamma, const float* __restrict__ mean,
                                                   const float* __restrict__ rstd, T* __restrict__ dx,
                                                   int64_t lddx, float* __restrict__ partial) {
  extern __shared__ float red[];  // [4][d], and behind it [d] for gamma when G_LDS
  // Wide rows (NV >= 4) keep gamma in LDS as fp32 and read a chunk where it is used: held in registers its
  // 8 * NV values pushed the kernel past 256 registers, one wave per SIMD and one workgroup per CU, so that
  // the 512 workgroups of a launch ran in two turns (d = 2048: 23.4 us per launch with it, 67 MB).
  constexpr bool G_LDS = NV >= 4;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int nchunk = d >> 3;
  float* const gam = red + 4 * d;
  float g[G_LDS ? 1 : NV][8], dg[NV][8], db[NV][8];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = lane + i * 64;
#pragma unroll
    for (int e = 0; e < 8; ++e) { dg[i][e] = 0.f; db[i][e] = 0.f; }
    if constexpr (!G_LDS) {
#pragma unroll
      for (int e = 0; e < 8; ++e) g[i][e] = 0.f;
      if (c < nchunk) load8<TP>(gamma + c * 8, g[i]);
    }
  }
  if constexpr (G_LDS) {
    for (int c = threadIdx.x; c < nchunk; c += 256) {
      float gv[8];
      load8<TP>(gamma + c * 8, gv);
#pragma unroll
      for (int e = 0; e < 8; ++e) gam[c * 8 + e] = gv[e];
    }
    __syncthreads();
  }
  const float inv_d = 1.0f / (float)d;
  const int64_t stride = (int64_t)gridDim.x * kRowsPerBlock;
  u32x4 raw_x[NV], raw_dy[NV], raw_ds[ADD ? NV : 1];
  float mu_next = 0.f, rs_next = 0.f;
  auto fetch = [&](int64_t row) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int c = lane + i * 64;
      if (c < nchunk) {
        raw_x[i] = ld16(x + row * ldx + c * 8);
        raw_dy[i] = ld16(dy + row * lddy + c * 8);
        if (ADD) raw_ds[i] = ld16(dsum + row * lddsum + c * 8);
      }
    }
    mu_next = mean[row];
    rs_next = rstd[row];
  };
  int64_t row = (int64_t)blockIdx.x * kRowsPerBlock + wave;
  if (row < rows) fetch(row);
  for (; row < rows; row += stride) {
    const float mu = mu_next, rs = rs_next;
    float xh[NV][8], gd[NV][8], ds[ADD ? NV : 1][8];
    float s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int c = lane + i * 64;
      if (c < nchunk) {
        float xv[8], dv[8], gl[8];
        unpack8<T>(raw_x[i], xv);
        unpack8<T>(raw_dy[i], dv);
        if (ADD) unpack8<T>(raw_ds[i], ds[i]);
#pragma unroll
        for (int e = 0; e < 8; ++e) gl[e] = G_LDS ? gam[c * 8 + e] : g[G_LDS ? 0 : i][e];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          xh[i][e] = (xv[e] - mu) * rs;
          gd[i][e] = dv[e] * gl[e];
          s1 += gd[i][e] * xh[i][e];
          s2 += gd[i][e];
          dg[i][e] += dv[e] * xh[i][e];
          db[i][e] += dv[e];
        }
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) { xh[i][e] = 0.f; gd[i][e] = 0.f; }
      }
    }
    if (row + stride < rows) fetch(row + stride);
    const float c1 = wave_sum(s1) * inv_d;
    const float c2 = wave_sum(s2) * inv_d;
    T* dxr = dx + row * lddx;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int c = lane + i * 64;
      if (c < nchunk) {
        float o[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          o[e] = (gd[i][e] - xh[i][e] * c1 - c2) * rs;
          if (ADD) o[e] += ds[i][e];
        }
        Chunk<T>::store(dxr + c * 8, o);
      }
    }
  }
  // cross-wave reduction, dgamma then dbeta, through one [4][d] LDS buffer
  float* pout = partial + (int64_t)blockIdx.x * 2 * d;
#pragma unroll
  for (int which = 0; which < 2; ++which) {
    __syncthreads();
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int c = lane + i * 64;
      if (c < nchunk) {
#pragma unroll
        for (int e = 0; e < 8; ++e) red[wave * d + c * 8 + e] = which ? db[i][e] : dg[i][e];
      }
    }
    __syncthreads();
    for (int c = threadIdx.x; c < d; c += 256)
      pout[which * d + c] = red[c] + red[d + c] + red[2 * d + c] + red[3 * d + c];
  }
}

template <typename T, typename TP, bool ADD>
__global__ __launch_bounds__(256) void ln_bwd_any(int64_t rows, int d, const T* __restrict__ dy, int64_t lddy,
                                                   const T* __restrict__ dsum, int64_t lddsum,
                                                   const T* __restrict__ x, int64_t ldx,
                                                   const TP* __restrict__ gamma, const float* __restrict__ mean,
                                                   const float* __restrict__ rstd, T* __restrict__ dx,
                                                   int64_t lddx, float* __restrict__ partial) {
  // One workgroup per slice of rows; every thread owns columns tid, tid+256, ...
  // so the dgamma/dbeta partials need no cross-thread reduction; the per-row
  // sums are reduced per wave, with all 4 waves walking the same row.
  __shared__ float sred[2][4];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const float inv_d = 1.0f / (float)d;
  float* pout = partial + (int64_t)blockIdx.x * 2 * d;
  for (int c = threadIdx.x; c < d; c += 256) { pout[c] = 0.f; pout[d + c] = 0.f; }
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const float mu = mean[row], rs = rstd[row];
    const T* xr = x + row * ldx;
    const T* dyr = dy + row * lddy;
    float s1 = 0.f, s2 = 0.f;
    for (int c = threadIdx.x; c < d; c += 256) {
      const float xh = ((float)xr[c] - mu) * rs, dv = (float)dyr[c], gd = dv * (float)gamma[c];
      s1 += gd * xh;
      s2 += gd;
      pout[c] += dv * xh;
      pout[d + c] += dv;
    }
    s1 = wave_sum(s1);
    s2 = wave_sum(s2);
    __syncthreads();
    if (lane == 0) { sred[0][wave] = s1; sred[1][wave] = s2; }
    __syncthreads();
    const float c1 = (sred[0][0] + sred[0][1] + sred[0][2] + sred[0][3]) * inv_d;
    const float c2 = (sred[1][0] + sred[1][1] + sred[1][2] + sred[1][3]) * inv_d;
    T* dxr = dx + row * lddx;
    for (int c = threadIdx.x; c < d; c += 256) {
      const float xh = ((float)xr[c] - mu) * rs, gd = (float)dyr[c] * (float)gamma[c];
      float o = (gd - xh * c1 - c2) * rs;
      if (ADD) o += (float)dsum[row * lddsum + c];
      dxr[c] = (T)o;
    }
  }
}

// Second stage over partial viewed as a [nparts][2d] matrix (dgamma columns then
// dbeta columns): workgroup = 16 columns x 16 row slices, slices summed in a
// fixed order through LDS.  Four independent running sums per thread keep
// several loads in flight.
template <typename T>
__global__ __launch_bounds__(256) void ln_bwd_reduce(int nparts, int d, const float* __restrict__ partial,
                                                      T* __restrict__ dgamma, T* __restrict__ dbeta) {
  __shared__ float red[16][17];
  const int cl = threadIdx.x & 15, slice = threadIdx.x >> 4;
  const int col = blockIdx.x * 16 + cl;  // 0 .. 2d-1
  float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
  if (col < 2 * d) {
    const float* src = partial + col;
    const int64_t ld = 2 * (int64_t)d;
    int p = slice;
    for (; p + 48 < nparts; p += 64) {
      a0 += src[(int64_t)p * ld];
      a1 += src[(int64_t)(p + 16) * ld];
      a2 += src[(int64_t)(p + 32) * ld];
      a3 += src[(int64_t)(p + 48) * ld];
    }
    for (; p < nparts; p += 16) a0 += src[(int64_t)p * ld];
  }
  red[slice][cl] = (a0 + a1) + (a2 + a3);
  __syncthreads();
  if (slice == 0 && col < 2 * d) {
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < 16; ++k) s += red[k][cl];
    if (col < d) dgamma[col] = (T)s;
    else dbeta[col - d] = (T)s;
  }
}

// The same second stage for the partial sums of several LayerNorms in one launch (blockIdx.y = LayerNorm):
// the parameter gradients of a whole backward pass, whose partial sums were left in place by the row passes.
constexpr int kLnReduceBatch = 64;
struct LnReduceItem {
  const float* partial;
  void* dgamma;
  void* dbeta;
  int parts;
};
struct LnReduceBatch { LnReduceItem it[kLnReduceBatch]; };
template <typename T>
__global__ __launch_bounds__(256) void ln_bwd_reduce_batch(LnReduceBatch batch, int d) {
  __shared__ float red[16][17];
  const LnReduceItem r = batch.it[blockIdx.y];
  const int cl = threadIdx.x & 15, slice = threadIdx.x >> 4;
  const int col = blockIdx.x * 16 + cl;  // 0 .. 2d-1
  float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
  if (col < 2 * d) {
    const float* src = r.partial + col;
    const int64_t ld = 2 * (int64_t)d;
    int p = slice;
    for (; p + 48 < r.parts; p += 64) {
      a0 += src[(int64_t)p * ld];
      a1 += src[(int64_t)(p + 16) * ld];
      a2 += src[(int64_t)(p + 32) * ld];
      a3 += src[(int64_t)(p + 48) * ld];
    }
    for (; p < r.parts; p += 16) a0 += src[(int64_t)p * ld];
  }
  red[slice][cl] = (a0 + a1) + (a2 + a3);
  __syncthreads();
  if (slice == 0 && col < 2 * d) {
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < 16; ++k) s += red[k][cl];
    if (col < d) ((T*)r.dgamma)[col] = (T)s;
    else ((T*)r.dbeta)[col - d] = (T)s;
  }
}

// ---------------------------------------------------------------------------
// Softmax (T = f16 / bf16 / float).  NV chunks of Chunk<T>::N elements per lane.
// ---------------------------------------------------------------------------
template <typename T, int NV>
__global__ __launch_bounds__(256) void softmax_fwd_vec(int64_t rows, int cols, const T* __restrict__ x,
                                                        int64_t ldx, T* __restrict__ y, int64_t ldy) {
  constexpr int N = Chunk<T>::N;
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int nchunk = cols / N;
  const T* xr = x + row * ldx;
  float v[NV][N];
  float m = -INFINITY;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = lane + i * 64;
    if (c < nchunk) {
      Chunk<T>::load(xr + c * N, v[i]);
#pragma unroll
      for (int e = 0; e < N; ++e) m = fmaxf(m, v[i][e]);
    }
  }
  m = wave_max(m);
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    if (lane + i * 64 < nchunk) {
#pragma unroll
      for (int e = 0; e < N; ++e) { v[i][e] = exp2f((v[i][e] - m) * kLog2e); s += v[i][e]; }
    }
  }
  const float inv = 1.0f / wave_sum(s);
  T* yr = y + row * ldy;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = lane + i * 64;
    if (c < nchunk) {
#pragma unroll
      for (int e = 0; e < N; ++e) v[i][e] *= inv;
      Chunk<T>::store(yr + c * N, v[i]);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void softmax_fwd_any(int64_t rows, int cols, const T* __restrict__ x,
                                                        int64_t ldx, T* __restrict__ y, int64_t ldy) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6);
  if (row >= rows) return;
  const T* xr = x + row * ldx;
  float m = -INFINITY;
  for (int c = lane; c < cols; c += 64) m = fmaxf(m, (float)xr[c]);
  m = wave_max(m);
  float s = 0.f;
  for (int c = lane; c < cols; c += 64) s += exp2f(((float)xr[c] - m) * kLog2e);
  const float inv = 1.0f / wave_sum(s);
  T* yr = y + row * ldy;
  for (int c = lane; c < cols; c += 64) yr[c] = (T)(exp2f(((float)xr[c] - m) * kLog2e) * inv);
}

template <typename T, int NV>
__global__ __launch_bounds__(256) void softmax_bwd_vec(int64_t rows, int cols, const T* __restrict__ dy,
                                                        int64_t lddy, const T* __restrict__ y, int64_t ldy,
                                                        T* __restrict__ dx, int64_t lddx) {
  constexpr int N = Chunk<T>::N;
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int nchunk = cols / N;
  float yv[NV][N], gv[NV][N];
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = lane + i * 64;
    if (c < nchunk) {
      Chunk<T>::load(y + row * ldy + c * N, yv[i]);
      Chunk<T>::load(dy + row * lddy + c * N, gv[i]);
#pragma unroll
      for (int e = 0; e < N; ++e) s += yv[i][e] * gv[i][e];
    }
  }
  s = wave_sum(s);
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = lane + i * 64;
    if (c < nchunk) {
      float o[N];
#pragma unroll
      for (int e = 0; e < N; ++e) o[e] = yv[i][e] * (gv[i][e] - s);
      Chunk<T>::store(dx + row * lddx + c * N, o);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void softmax_bwd_any(int64_t rows, int cols, const T* __restrict__ dy,
                                                        int64_t lddy, const T* __restrict__ y, int64_t ldy,
                                                        T* __restrict__ dx, int64_t lddx) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6);
  if (row >= rows) return;
  float s = 0.f;
  for (int c = lane; c < cols; c += 64) s += (float)y[row * ldy + c] * (float)dy[row * lddy + c];
  s = wave_sum(s);
  for (int c = lane; c < cols; c += 64)
    dx[row * lddx + c] = (T)((float)y[row * ldy + c] * ((float)dy[row * lddy + c] - s));
}

// ---------------------------------------------------------------------------
// Long rows (beyond the 512 chunks a single wave holds: vocabulary-sized rows): one workgroup of 16
// waves per row, the row in registers as NV 16-byte chunks per thread (chunk c of thread t:
// t + 1024 c), wave sums merged through LDS.  Every element is read once and written once, as in
// the wave-per-row kernels.
// ---------------------------------------------------------------------------
constexpr int kLongRowThreads = 1024;
// all-reduce of one value per thread over the workgroup; `slot` distinguishes consecutive uses
template <bool MAX> __device__ __forceinline__ float block_reduce16(float v, float* red, int slot) {
  v = MAX ? wave_max(v) : wave_sum(v);
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) red[slot * 16 + wave] = v;
  __syncthreads();
  float r = red[slot * 16];
#pragma unroll
  for (int w = 1; w < 16; ++w) r = MAX ? fmaxf(r, red[slot * 16 + w]) : r + red[slot * 16 + w];
  return r;
}

template <typename T> __device__ __forceinline__ void chunk_floats(u32x4 raw, float (&v)[Chunk<T>::N]) {
  if constexpr (sizeof(T) == 2) unpack8<T>(raw, v);
  else {
    const f32x4 f = __builtin_bit_cast(f32x4, raw);
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = f[i];
  }
}
// (exponentials of non-positive arguments: v_exp_f32 as it is, without the library wrapper's range
// handling -- results below 2^-126 become zero, which is what they round to in the sum anyway)
template <typename T, int NV>
__global__ __launch_bounds__(kLongRowThreads) void softmax_fwd_long(int cols, const T* __restrict__ x, int64_t ldx,
                                                                    T* __restrict__ y, int64_t ldy) {
  constexpr int N = Chunk<T>::N;
  __shared__ float red[32];
  const int64_t row = blockIdx.x;
  const int nchunk = cols / N;
  const T* xr = x + row * ldx;
  float v[NV][N];
  float m = -INFINITY;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = threadIdx.x + i * kLongRowThreads;
    if (c < nchunk) {
      chunk_floats<T>(ld16_stream(xr + c * N), v[i]);
#pragma unroll
      for (int e = 0; e < N; ++e) m = fmaxf(m, v[i][e]);
    }
  }
  m = block_reduce16<true>(m, red, 0);
  const float shift = -m * kLog2e;
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    if ((int)threadIdx.x + i * kLongRowThreads < nchunk) {
#pragma unroll
      for (int e = 0; e < N; ++e) { v[i][e] = __builtin_amdgcn_exp2f(__builtin_fmaf(v[i][e], kLog2e, shift)); s += v[i][e]; }
    }
  }
  const float inv = 1.0f / block_reduce16<false>(s, red, 1);
  T* yr = y + row * ldy;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = threadIdx.x + i * kLongRowThreads;
    if (c < nchunk) {
#pragma unroll
      for (int e = 0; e < N; ++e) v[i][e] *= inv;
      Chunk<T>::store(yr + c * N, v[i]);
    }
  }
}

// y and dy stay in registers as the raw 16-byte chunks (converted where they are used: as floats, 16-bit
// rows would need twice the registers); with HOLD_DY false dy is read a second time instead (from the
// cache: a row is a few hundred KB), for rows whose two operands do not fit the 128 registers of a thread.
template <typename T, int NV, bool HOLD_DY>
__global__ __launch_bounds__(kLongRowThreads) void softmax_bwd_long(int cols, const T* __restrict__ dy, int64_t lddy,
                                                                    const T* __restrict__ y, int64_t ldy,
                                                                    T* __restrict__ dx, int64_t lddx) {
  constexpr int N = Chunk<T>::N;
  __shared__ float red[16];
  const int64_t row = blockIdx.x;
  const int nchunk = cols / N;
  u32x4 ry[NV], rg[HOLD_DY ? NV : 1];
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = threadIdx.x + i * kLongRowThreads;
    if (c < nchunk) {
      ry[i] = ld16_stream(y + row * ldy + c * N);
      const u32x4 g = HOLD_DY ? ld16_stream(dy + row * lddy + c * N) : ld16(dy + row * lddy + c * N);
      if (HOLD_DY) rg[i] = g;
      float yv[N], gv[N];
      chunk_floats<T>(ry[i], yv);
      chunk_floats<T>(g, gv);
#pragma unroll
      for (int e = 0; e < N; ++e) s += yv[e] * gv[e];
    }
  }
  s = block_reduce16<false>(s, red, 0);
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = threadIdx.x + i * kLongRowThreads;
    if (c < nchunk) {
      float yv[N], gv[N], o[N];
      chunk_floats<T>(ry[i], yv);
      chunk_floats<T>(HOLD_DY ? rg[i] : ld16(dy + row * lddy + c * N), gv);
#pragma unroll
      for (int e = 0; e < N; ++e) o[e] = yv[e] * (gv[e] - s);
      Chunk<T>::store(dx + row * lddx + c * N, o);
    }
  }
}
// chunks per thread of the long-row kernels for a row of `nchunk` chunks (0: beyond them)
template <typename T> static int pick_long_nv(int64_t nchunk) {
  if (nchunk <= 4 * kLongRowThreads) return 4;
  if (nchunk <= 8 * kLongRowThreads) return 8;
  if (nchunk <= 16 * kLongRowThreads && sizeof(T) == 4) return 16;  // 65536 elements of either width
  return 0;
}

// ---------------------------------------------------------------------------
// host dispatch
// ---------------------------------------------------------------------------
static int pick_nv(int64_t nchunk) {
  if (nchunk <= 64) return 1;
  if (nchunk <= 128) return 2;
  if (nchunk <= 256) return 4;
  if (nchunk <= 512) return 8;
  return 0;
}

template <typename T, typename TP, bool ADD>
static int ln_fwd_launch(hipStream_t st, int64_t rows, int64_t d, const void* x, int64_t ldx, const void* res,
                         int64_t ldres, void* sum, int64_t ldsum, const void* gamma, const void* beta, float eps,
                         void* y, int64_t ldy, float* mean, float* rstd) {
  const dim3 grid((unsigned)ceil_div(rows, kRowsPerBlock)), block(256);
  bool vec = row_vectorizable<T>(x, d, ldx) && row_vectorizable<T>(y, d, ldy) && aligned16(gamma) && aligned16(beta);
  if (ADD) vec = vec && row_vectorizable<T>(res, d, ldres) && row_vectorizable<T>(sum, d, ldsum);
  const int nv = vec ? pick_nv(d / 8) : 0;
  // the row-walking kernel: kLnFwdRowsPerWave rows per wave once there are enough rows to fill the chip
  int64_t walkers = ceil_div(rows, kRowsPerBlock * kLnFwdRowsPerWave);
  const int64_t fill = (int64_t)device_shape().cus * 4;
  if (walkers < fill) walkers = ceil_div(rows, kRowsPerBlock) < fill ? ceil_div(rows, kRowsPerBlock) : fill;
  const dim3 wgrid((unsigned)walkers);
#define LN_FWD(NV)                                                                                             \
  ln_fwd_vec<T, TP, NV, ADD><<<wgrid, block, 0, st>>>(rows, (int)d, (const T*)x, ldx, (const T*)res, ldres, (T*)sum, \
                                                     ldsum, (const TP*)gamma, (const TP*)beta, eps, (T*)y, ldy, mean, \
                                                     rstd)
  switch (nv) {
    case 1: LN_FWD(1); break;
    case 2: LN_FWD(2); break;
    case 4: LN_FWD(4); break;
    case 8: LN_FWD(8); break;
    default:
      ln_fwd_any<T, TP, ADD><<<grid, block, 0, st>>>(rows, (int)d, (const T*)x, ldx, (const T*)res, ldres, (T*)sum,
                                                     ldsum, (const TP*)gamma, (const TP*)beta, eps, (T*)y, ldy, mean,
                                                     rstd);
  }
#undef LN_FWD
  TF_CHECK_LAUNCH();
  return TF_OK;
}

static int ln_bwd_parts(int64_t rows) {
  int64_t g = (rows + kRowsPerBlock - 1) / kRowsPerBlock;
  return (int)(g < 512 ? g : 512);
}

template <typename T, typename TP, bool ADD>
static int ln_bwd_launch(hipStream_t st, int64_t rows, int64_t d, const void* dy, int64_t lddy, const void* dsum,
                         int64_t lddsum, const void* x, int64_t ldx, const void* gamma, const float* mean,
                         const float* rstd, void* dx, int64_t lddx, void* dgamma, void* dbeta, float* partial) {
  const int parts = ln_bwd_parts(rows);
  bool vec = row_vectorizable<T>(x, d, ldx) && row_vectorizable<T>(dy, d, lddy) && row_vectorizable<T>(dx, d, lddx) &&
             aligned16(gamma);
  if (ADD) vec = vec && row_vectorizable<T>(dsum, d, lddsum);
  const int nv = vec ? pick_nv(d / 8) : 0;
  const size_t lds = (size_t)(nv >= 4 ? 5 : 4) * d * sizeof(float);  // wide rows keep gamma there too
#define LN_BWD(NV)                                                                                                \
  ln_bwd_vec<T, TP, NV, ADD><<<dim3(parts), dim3(256), lds, st>>>(rows, (int)d, (const T*)dy, lddy, (const T*)dsum,   \
                                                                  lddsum, (const T*)x, ldx, (const TP*)gamma, mean, \
                                                                  rstd, (T*)dx, lddx, partial)
  switch (nv) {
    case 1: LN_BWD(1); break;
    case 2: LN_BWD(2); break;
    case 4: LN_BWD(4); break;
    case 8: LN_BWD(8); break;
    default:
      ln_bwd_any<T, TP, ADD><<<dim3(parts), dim3(256), 0, st>>>(rows, (int)d, (const T*)dy, lddy, (const T*)dsum,
                                                                lddsum, (const T*)x, ldx, (const TP*)gamma, mean,
                                                                rstd, (T*)dx, lddx, partial);
  }
#undef LN_BWD
  TF_CHECK_LAUNCH();
  if (!dgamma) return TF_OK;  // the partial sums stay where they are, for tf_layernorm_param_grads
  ln_bwd_reduce<TP><<<dim3(ceil_div(2 * d, 16)), dim3(256), 0, st>>>(parts, (int)d, partial, (TP*)dgamma, (TP*)dbeta);
  TF_CHECK_LAUNCH();
  return TF_OK;
}

template <typename T>
static int softmax_fwd_launch(hipStream_t st, int64_t rows, int64_t cols, const void* x, int64_t ldx, void* y,
                              int64_t ldy) {
  const dim3 grid((unsigned)ceil_div(rows, kRowsPerBlock)), block(256);
  const bool vec = row_vectorizable<T>(x, cols, ldx) && row_vectorizable<T>(y, cols, ldy);
  const int nv = vec ? pick_nv(cols / Chunk<T>::N) : 0;
#define SM_FWD(NV) softmax_fwd_vec<T, NV><<<grid, block, 0, st>>>(rows, (int)cols, (const T*)x, ldx, (T*)y, ldy)
  switch (nv) {
    case 1: SM_FWD(1); break;
    case 2: SM_FWD(2); break;
    case 4: SM_FWD(4); break;
    case 8: SM_FWD(8); break;
    default: {
      const int lnv = vec && rows <= 0x7fffffff ? pick_long_nv<T>(cols / Chunk<T>::N) : 0;
      const dim3 lgrid((unsigned)rows), lblock(kLongRowThreads);
      if (lnv == 4) softmax_fwd_long<T, 4><<<lgrid, lblock, 0, st>>>((int)cols, (const T*)x, ldx, (T*)y, ldy);
      else if (lnv == 8) softmax_fwd_long<T, 8><<<lgrid, lblock, 0, st>>>((int)cols, (const T*)x, ldx, (T*)y, ldy);
      else if (lnv == 16 && sizeof(T) == 4) softmax_fwd_long<float, 16><<<lgrid, lblock, 0, st>>>((int)cols, (const float*)x, ldx, (float*)y, ldy);
      else softmax_fwd_any<T><<<grid, block, 0, st>>>(rows, (int)cols, (const T*)x, ldx, (T*)y, ldy);
    }
  }
#undef SM_FWD
  TF_CHECK_LAUNCH();
  return TF_OK;
}

template <typename T>
static int softmax_bwd_launch(hipStream_t st, int64_t rows, int64_t cols, const void* dy, int64_t lddy,
                              const void* y, int64_t ldy, void* dx, int64_t lddx) {
  const dim3 grid((unsigned)ceil_div(rows, kRowsPerBlock)), block(256);
  const bool vec =
      row_vectorizable<T>(dy, cols, lddy) && row_vectorizable<T>(y, cols, ldy) && row_vectorizable<T>(dx, cols, lddx);
  const int nv = vec ? pick_nv(cols / Chunk<T>::N) : 0;
#define SM_BWD(NV) \
  softmax_bwd_vec<T, NV><<<grid, block, 0, st>>>(rows, (int)cols, (const T*)dy, lddy, (const T*)y, ldy, (T*)dx, lddx)
  switch (nv) {
    case 1: SM_BWD(1); break;
    case 2: SM_BWD(2); break;
    case 4: SM_BWD(4); break;
    case 8: SM_BWD(8); break;
    default: {
      const int lnv = vec && rows <= 0x7fffffff ? pick_long_nv<T>(cols / Chunk<T>::N) : 0;
      const dim3 lgrid((unsigned)rows), lblock(kLongRowThreads);
#define SM_BWD_LONG(TT, NV, HOLD) \
  softmax_bwd_long<TT, NV, HOLD><<<lgrid, lblock, 0, st>>>((int)cols, (const TT*)dy, lddy, (const TT*)y, ldy, (TT*)dx, lddx)
      if (lnv == 4) SM_BWD_LONG(T, 4, true);
      else if (lnv == 8) SM_BWD_LONG(T, 8, true);
      else if (lnv == 16 && sizeof(T) == 4) SM_BWD_LONG(float, 16, false);
      else softmax_bwd_any<T><<<grid, block, 0, st>>>(rows, (int)cols, (const T*)dy, lddy, (const T*)y, ldy, (T*)dx, lddx);
#undef SM_BWD_LONG
    }
  }
#undef SM_BWD
  TF_CHECK_LAUNCH();
  return TF_OK;
}

static bool bad_rows(int64_t rows, int64_t n, int64_t ld) {
  return rows < 0 || n <= 0 || n > (1 << 30) || ld < n || rows > (int64_t)kRowsPerBlock * 0x7fffffff;
}

}  // namespace tfa

using namespace tfa;

template <bool ADD>
static int ln_fwd_entry(void* stream, int dtype, int param_dtype, int64_t rows, int64_t d, const void* x, int64_t ldx,
                        const void* res, int64_t ldres, void* sum, int64_t ldsum, const void* gamma,
                        const void* beta, float eps, void* y, int64_t ldy, float* mean, float* rstd) {
  if (!x || !gamma || !beta || !y || !mean || !rstd) return TF_EINVAL;
  if (ADD && (!res || !sum || ldres < d || ldsum < d)) return TF_EINVAL;
  if (bad_rows(rows, d, ldx) || ldy < d) return TF_EINVAL;
  if (rows == 0) return TF_OK;
  hipStream_t st = (hipStream_t)stream;
  if (param_dtype != dtype && param_dtype != TF_F32) return TF_EDTYPE;
#define LN_FWD_GO(T, TP) \
  return ln_fwd_launch<T, TP, ADD>(st, rows, d, x, ldx, res, ldres, sum, ldsum, gamma, beta, eps, y, ldy, mean, rstd)
  if (dtype == TF_F16) { if (param_dtype == TF_F32) LN_FWD_GO(f16, float); else LN_FWD_GO(f16, f16); }
  if (dtype == TF_BF16) { if (param_dtype == TF_F32) LN_FWD_GO(bf16, float); else LN_FWD_GO(bf16, bf16); }
#undef LN_FWD_GO
  return TF_EDTYPE;
}

extern "C" int tf_layernorm_fwd(void* stream, int dtype, int param_dtype, int64_t rows, int64_t d, const void* x,
                                int64_t ldx, const void* gamma, const void* beta, float eps, void* y, int64_t ldy,
                                float* mean, float* rstd) {
  return ln_fwd_entry<false>(stream, dtype, param_dtype, rows, d, x, ldx, nullptr, 0, nullptr, 0, gamma, beta, eps, y,
                             ldy, mean, rstd);
}

extern "C" int tf_add_layernorm_fwd(void* stream, int dtype, int param_dtype, int64_t rows, int64_t d, const void* x,
                                    int64_t ldx, const void* res, int64_t ldres, void* sum, int64_t ldsum,
                                    const void* gamma, const void* beta, float eps, void* y, int64_t ldy, float* mean,
                                    float* rstd) {
  return ln_fwd_entry<true>(stream, dtype, param_dtype, rows, d, x, ldx, res, ldres, sum, ldsum, gamma, beta, eps, y,
                            ldy, mean, rstd);
}

extern "C" int64_t tf_layernorm_bwd_partial_bytes(int64_t rows, int64_t d) {
  if (rows <= 0 || d <= 0) return 0;
  return (int64_t)ln_bwd_parts(rows) * 2 * d * (int64_t)sizeof(float);
}

template <bool ADD>
static int ln_bwd_entry(void* stream, int dtype, int param_dtype, int64_t rows, int64_t d, const void* dy,
                        int64_t lddy, const void* dsum, int64_t lddsum, const void* x, int64_t ldx,
                        const void* gamma, const float* mean, const float* rstd, void* dx, int64_t lddx,
                        void* dgamma, void* dbeta, float* partial, int64_t partial_bytes) {
  if (!dy || !x || !gamma || !mean || !rstd || !dx || (dgamma == nullptr) != (dbeta == nullptr)) return TF_EINVAL;
  if (ADD && (!dsum || lddsum < d)) return TF_EINVAL;
  if (bad_rows(rows, d, ldx) || lddy < d || lddx < d || rows == 0) return TF_EINVAL;
  if (!partial || partial_bytes < tf_layernorm_bwd_partial_bytes(rows, d)) return TF_EWORKSPACE;
  hipStream_t st = (hipStream_t)stream;
  if (param_dtype != dtype && param_dtype != TF_F32) return TF_EDTYPE;
#define LN_BWD_GO(T, TP)                                                                                          \
  return ln_bwd_launch<T, TP, ADD>(st, rows, d, dy, lddy, dsum, lddsum, x, ldx, gamma, mean, rstd, dx, lddx, dgamma, \
                                   dbeta, partial)
  if (dtype == TF_F16) { if (param_dtype == TF_F32) LN_BWD_GO(f16, float); else LN_BWD_GO(f16, f16); }
  if (dtype == TF_BF16) { if (param_dtype == TF_F32) LN_BWD_GO(bf16, float); else LN_BWD_GO(bf16, bf16); }
#undef LN_BWD_GO
  return TF_EDTYPE;
}

extern "C" int tf_layernorm_bwd(void* stream, int dtype, int param_dtype, int64_t rows, int64_t d, const void* dy,
                                int64_t lddy, const void* x, int64_t ldx, const void* gamma, const float* mean,
                                const float* rstd, void* dx, int64_t lddx, void* dgamma, void* dbeta,
                                float* partial, int64_t partial_bytes) {
  return ln_bwd_entry<false>(stream, dtype, param_dtype, rows, d, dy, lddy, nullptr, 0, x, ldx, gamma, mean, rstd, dx,
                             lddx, dgamma, dbeta, partial, partial_bytes);
}

extern "C" int tf_add_layernorm_bwd(void* stream, int dtype, int param_dtype, int64_t rows, int64_t d, const void* dy,
                                    int64_t lddy, const void* dsum, int64_t lddsum, const void* x, int64_t ldx,
                                    const void* gamma, const float* mean, const float* rstd, void* dx, int64_t lddx,
                                    void* dgamma, void* dbeta, float* partial, int64_t partial_bytes) {
  return ln_bwd_entry<true>(stream, dtype, param_dtype, rows, d, dy, lddy, dsum, lddsum, x, ldx, gamma, mean, rstd, dx,
                            lddx, dgamma, dbeta, partial, partial_bytes);
}

extern "C" int64_t tf_layernorm_bwd_parts(int64_t rows) { return rows > 0 ? ln_bwd_parts(rows) : 0; }

extern "C" int tf_layernorm_param_grads(void* stream, int param_dtype, int64_t d, int count,
                                        const tf_ln_param_grads* items) {
  if (count < 0 || d <= 0 || d > 0x3fffffff || (count > 0 && !items)) return TF_EINVAL;
  if (param_dtype != TF_F16 && param_dtype != TF_BF16 && param_dtype != TF_F32) return TF_EDTYPE;
  for (int i = 0; i < count; ++i)
    if (!items[i].partial || !items[i].dgamma || !items[i].dbeta || items[i].parts < 1 || items[i].parts > 512)
      return TF_EINVAL;
  hipStream_t st = (hipStream_t)stream;
  for (int base = 0; base < count; base += kLnReduceBatch) {
    const int n = count - base < kLnReduceBatch ? count - base : kLnReduceBatch;
    LnReduceBatch b = {};
    for (int i = 0; i < n; ++i)
      b.it[i] = {items[base + i].partial, items[base + i].dgamma, items[base + i].dbeta, (int)items[base + i].parts};
    const dim3 grid((unsigned)ceil_div(2 * d, 16), (unsigned)n), block(256);
    if (param_dtype == TF_F32) ln_bwd_reduce_batch<float><<<grid, block, 0, st>>>(b, (int)d);
    else if (param_dtype == TF_F16) ln_bwd_reduce_batch<f16><<<grid, block, 0, st>>>(b, (int)d);
    else ln_bwd_reduce_batch<bf16><<<grid, block, 0, st>>>(b, (int)d);
    TF_CHECK_LAUNCH();
  }
  return TF_OK;
}

extern "C" int tf_softmax_fwd(void* stream, int dtype, int64_t rows, int64_t cols, const void* x, int64_t ldx,
                              void* y, int64_t ldy) {
  if (!x || !y) return TF_EINVAL;
  if (bad_rows(rows, cols, ldx) || ldy < cols) return TF_EINVAL;
  if (rows == 0) return TF_OK;
  hipStream_t st = (hipStream_t)stream;
  switch (dtype) {
    case TF_F16: return softmax_fwd_launch<f16>(st, rows, cols, x, ldx, y, ldy);
    case TF_BF16: return softmax_fwd_launch<bf16>(st, rows, cols, x, ldx, y, ldy);
    case TF_F32: return softmax_fwd_launch<float>(st, rows, cols, x, ldx, y, ldy);
  }
  return TF_EDTYPE;
}

extern "C" int tf_softmax_bwd(void* stream, int dtype, int64_t rows, int64_t cols, const void* dy, int64_t lddy,
                              const void* y, int64_t ldy, void* dx, int64_t lddx) {
  if (!dy || !y || !dx) return TF_EINVAL;
  if (bad_rows(rows, cols, ldy) || lddy < cols || lddx < cols) return TF_EINVAL;
  if (rows == 0) return TF_OK;
  hipStream_t st = (hipStream_t)stream;
  switch (dtype) {
    case TF_F16: return softmax_bwd_launch<f16>(st, rows, cols, dy, lddy, y, ldy, dx, lddx);
    case TF_BF16: return softmax_bwd_launch<bf16>(st, rows, cols, dy, lddy, y, ldy, dx, lddx);
    case TF_F32: return softmax_bwd_launch<float>(st, rows, cols, dy, lddy, y, ldy, dx, lddx);
  }
  return TF_EDTYPE;
}
