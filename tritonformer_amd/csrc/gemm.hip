// Dense contraction C[M,N] = epilogue(sum_k A(m,k) B(n,k)) on gfx950 MFMA.
//
// One workgroup owns a BM x BN tile of C (or one slice of its contraction).  Two
// kernel families share the tiling and the MFMA code:
//  * gemm_dma_kernel / gemm_dma_group_kernel, the ones a training step runs: per
//    BK-wide step the A and B panels go HBM -> LDS directly (global_load_lds_dwordx4,
//    no VGPR round trip) into two LDS stages; the LDS operand reads, the loads of the
//    next step and the MFMAs are interleaved by hand (bare s_barrier, explicit
//    s_waitcnt); the result leaves through a wave-private LDS slab so that every
//    global store covers whole 128-byte lines;
//  * gemm_kernel, for anything those cannot take (ragged extents, unaligned pointers,
//    a contraction that is not a multiple of BK): operands staged through registers
//    with per-element predication, one barrier per step.
// Both use v_mfma_f32_32x32x16_{f16,bf16} with fp32 accumulators.
//
// Either operand may be stored with the contraction dimension contiguous
// ("K-major": read from LDS with ds_read_b128) or strided ("K-minor": read with
// the gfx950 transposing ds_read_b64_tr_b16), so X.W, dY.W^T and X^T.dY all run
// from the tensors as PyTorch holds them, without transposed copies.  LDS
// tiles are XOR-swizzled at 16-byte granularity to keep both access patterns
// free of bank conflicts.
//
// The MFMA is issued as D^T = B_frag x A_frag, so a lane ends up holding four
// consecutive n for one m: bias, ReLU and rounding need no cross-lane traffic.
//
// Workgroup ids are remapped so that each XCD (which receive ids round-robin)
// works on a compact block of neighbouring tiles and shares the A/B panels
// through its own L2.  The number of XCDs and of CUs is read from the device.
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <type_traits>
#include "rowops.h"


namespace tfa {

struct GemmParams {
  const void* A;
  const void* B;
  void* C;
  const void* bias;
  float* partial;
  int M, N, K;
  int64_t lda, ldb, ldc;
  int relu;
  int splits, k_per_split;
  int tiles_m, tiles_n;
  int flags;  // bit 0: skip the XCD remap (set by the diagnostic entry point only)
  int xcds;   // XCDs of the device (workgroup ids are dealt to them round-robin)
  int out_f32;  // C holds fp32 instead of T
  const void* mask;  // optional (M, N) activation of type T: C = mask > 0 ? C : 0
  int64_t ldmask;
  // One bit per element, rows of ldsign bytes, bit n % 8 of byte n / 8 (direct-to-LDS kernels only):
  // sign_out receives C > 0 (with the ReLU epilogue: the gradient mask of the activation, at a
  // sixteenth of its size); sign_in zeroes C where its bit is clear.
  void* sign_out;
  const void* sign_in;
  int64_t ldsign;
  // Output split into column blocks of chunk_n columns, each its own (M, chunk_n) matrix
  // with leading dimension ldc, chunk_skip + chunk_n elements after the previous one.
  // One matrix: chunk_n = N, chunk_skip = 0.
  int chunk_n;
  int64_t chunk_skip;
  // Optional factor on the whole product, one fp32 value in DEVICE memory (null = 1): it is applied
  // to the fp32 sums before bias / rounding.  A pointer, so that a value computed on the GPU (the
  // upstream gradient of a mean loss) needs no host round trip.
  const float* alpha;
};

__device__ __forceinline__ int64_t c_index(const GemmParams& p, int m, int n) {
  return (int64_t)m * p.ldc + n + (int64_t)(n / p.chunk_n) * p.chunk_skip;
}

// ---------------------------------------------------------------------------
// One operand panel: R rows (m or n) by BK of the contraction.
// ---------------------------------------------------------------------------
template <typename T, int R, int BK, bool KMAJOR, int NT, bool VEC>
struct Panel {
  static constexpr int CPR = KMAJOR ? BK / 8 : R / 8;  // 16-byte chunks per LDS row
  static constexpr int LROWS = KMAJOR ? R : BK;        // LDS rows
  static constexpr int NCHUNK = LROWS * CPR;
  static constexpr int PER_THREAD = NCHUNK / NT;
  static constexpr int BYTES = NCHUNK * 16;
  static_assert(NCHUNK % NT == 0, "panel must divide evenly over the workgroup");
  static_assert(KMAJOR ? (CPR == 4 || CPR == 8) : (CPR >= 16), "unsupported panel shape");

  // chunk-index swizzle; an involution on c for a fixed LDS row
  static __device__ __forceinline__ int swz(int lrow, int c) {
    if constexpr (KMAJOR) return c ^ ((lrow / (16 / CPR)) % CPR);
    else return c ^ ((lrow & 3) << 2);
  }

  // Global -> registers.  (row0, rmax) bound the m/n index, (k0, kend) the contraction.
  static __device__ __forceinline__ void fetch(u32x4 (&regs)[PER_THREAD], const T* __restrict__ base, int64_t ld,
                                               int row0, int rmax, int k0, int kend) {
#pragma unroll
    for (int j = 0; j < PER_THREAD; ++j) {
      const int id = threadIdx.x + j * NT;
      const int lrow = id / CPR, c = id % CPR;
      const int gr = KMAJOR ? row0 + lrow : row0 + c * 8;  // m/n index of the chunk's first element
      const int gk = KMAJOR ? k0 + c * 8 : k0 + lrow;      // contraction index of the first element
      const T* ptr = KMAJOR ? base + (int64_t)gr * ld + gk : base + (int64_t)gk * ld + gr;
      if (VEC) {
        u32x4 v = {0u, 0u, 0u, 0u};
        if (gr < rmax && gk < kend) v = ld16(ptr);
        regs[j] = v;
      } else {
        typename Vec<T>::v8 h;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const bool ok = KMAJOR ? (gr < rmax && gk + e < kend) : (gr + e < rmax && gk < kend);
          h[e] = ok ? ptr[e] : (T)0.f;
        }
        regs[j] = __builtin_bit_cast(u32x4, h);
      }
    }
  }

  static __device__ __forceinline__ void commit(char* lds, const u32x4 (&regs)[PER_THREAD]) {
#pragma unroll
    for (int j = 0; j < PER_THREAD; ++j) {
      const int id = threadIdx.x + j * NT;
      const int lrow = id / CPR, c = id % CPR;
      lds_st16(lds, (lrow * CPR + swz(lrow, c)) * 16, regs[j]);
    }
  }

  // MFMA operand for the 32 rows starting at rb, contraction step ks (16 wide):
  // lane l gets elements (row rb + l%32, k = ks*16 + (l/32)*8 + 0..7).
  static __device__ __forceinline__ typename Vec<T>::v8 frag(const char* lds, int rb, int ks, int lane) {
    if (KMAJOR) {
      const int row = rb + (lane & 31);
      const int c = ks * 2 + (lane >> 5);
      return __builtin_bit_cast(typename Vec<T>::v8, lds_ld16(lds, (row * CPR + swz(row, c)) * 16));
    } else {
      const int i = lane & 15;
      const int col = rb + 16 * ((lane >> 4) & 1) + (i & 3) * 4;
      const int kk0 = ks * 16 + 8 * (lane >> 5) + (i >> 2);
      const int kk1 = kk0 + 4;
      const u32x2 lo = lds_ld8_tr(lds, (kk0 * CPR + swz(kk0, col >> 3)) * 16 + (col & 7) * 2);
      const u32x2 hi = lds_ld8_tr(lds, (kk1 * CPR + swz(kk1, col >> 3)) * 16 + (col & 7) * 2);
      u32x4 v = {lo[0], lo[1], hi[0], hi[1]};
      return __builtin_bit_cast(typename Vec<T>::v8, v);
    }
  }
};

// Round-robin XCD dispatch -> compact per-XCD ranges, then grouped raster.
__device__ __forceinline__ int remap_xcd(int pid, int n, int X) {
  const int xcd = pid % X, local = pid / X;
  const int q = n / X, r = n % X;
  return xcd * q + (xcd < r ? xcd : r) + local;
}

// Epilogue shared by both kernels: lane holds C[m][n .. n+3] for m = .. + lane%32.
template <typename T, int TM, int TN, int WTM, int WTN, bool VEC>
__device__ __forceinline__ void gemm_epilogue(const GemmParams& p, f32x16 (&acc)[TM][TN], int m0, int n0, int wm,
                                              int wn, int lane, int split) {
  const T* bias = (const T*)p.bias;
  T* C = (T*)p.C;
  const float alpha = (p.alpha && p.splits <= 1) ? *p.alpha : 1.f;  // a split contraction is scaled by its reduce pass
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = m0 + wm * WTM + i * 32 + (lane & 31);
    if (m >= p.M) continue;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int n = n0 + wn * WTN + j * 32 + g * 8 + (lane >> 5) * 4;
        if (n >= p.N) continue;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = acc[i][j][g * 4 + e] * alpha;
        if (p.splits > 1) {
          float* dst = p.partial + ((int64_t)split * p.M + m) * p.N + n;
          if (VEC) {
            f32x4 o = {v[0], v[1], v[2], v[3]};
            *reinterpret_cast<f32x4*>(dst) = o;
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (n + e < p.N) dst[e] = v[e];
          }
        } else {
          if (p.mask) {
            const T* mk = (const T*)p.mask + (int64_t)m * p.ldmask + n;
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (n + e < p.N && !((float)mk[e] > 0.f)) v[e] = 0.f;  // no bias / ReLU with a mask (host check)
          }
          if (p.out_f32) {
            float* Cf = reinterpret_cast<float*>(p.C) + c_index(p, m, n);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              if (n + e < p.N) {
                const float x = v[e] + (bias ? (float)bias[n + e] : 0.f);
                Cf[e] = p.relu ? fmaxf(x, 0.f) : x;
              }
            }
          } else if (VEC) {
            typename Vec<T>::v4 o;
            if (bias) {
              const typename Vec<T>::v4 bv = *reinterpret_cast<const typename Vec<T>::v4*>(bias + n);
#pragma unroll
              for (int e = 0; e < 4; ++e) v[e] += (float)bv[e];
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = (T)(p.relu ? fmaxf(v[e], 0.f) : v[e]);
            *reinterpret_cast<typename Vec<T>::v4*>(C + c_index(p, m, n)) = o;
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              if (n + e < p.N) {
                float x = v[e] + (bias ? (float)bias[n + e] : 0.f);
                C[c_index(p, m, n) + e] = (T)(p.relu ? fmaxf(x, 0.f) : x);
              }
            }
          }
        }
      }
    }
  }
}

template <typename T, int BM, int BN, int BK, int WM, int WN, bool A_KMAJOR, bool B_KMAJOR, bool VEC>
__global__ __launch_bounds__(WM* WN * 64) void gemm_kernel(GemmParams p) {
  constexpr int NT = WM * WN * 64;
  constexpr int WTM = BM / WM, WTN = BN / WN;  // wave tile
  constexpr int TM = WTM / 32, TN = WTN / 32;  // MFMA tiles per wave
  constexpr int GROUP_M = 8;
  typedef Panel<T, BM, BK, A_KMAJOR, NT, VEC> PA;
  typedef Panel<T, BN, BK, B_KMAJOR, NT, VEC> PB;
  typedef typename Vec<T>::v8 v8;
  extern __shared__ __attribute__((aligned(16))) char smem[];

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wm = wave / WN, wn = wave % WN;

  // ---- which tile / which slice of the contraction -------------------------
  const int tiles = p.tiles_m * p.tiles_n;
  const int pid = (p.flags & 1) ? (int)blockIdx.x : remap_xcd(blockIdx.x, tiles * p.splits, p.xcds);
  const int split = pid / tiles;
  const int t = pid - split * tiles;
  const int per_group = GROUP_M * p.tiles_n;
  const int group = t / per_group;
  const int first_m = group * GROUP_M;
  const int gsz = min(p.tiles_m - first_m, GROUP_M);
  const int tm = first_m + (t % per_group) % gsz;
  const int tn = (t % per_group) / gsz;
  const int m0 = tm * BM, n0 = tn * BN;
  const int kbeg = split * p.k_per_split;
  const int kend = min(p.K, kbeg + p.k_per_split);
  const int nk = (kend - kbeg + BK - 1) / BK;

  const T* A = (const T*)p.A;
  const T* B = (const T*)p.B;

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  u32x4 ra[PA::PER_THREAD], rb[PB::PER_THREAD];
  constexpr int STAGE = PA::BYTES + PB::BYTES;

  if (nk > 0) {
    PA::fetch(ra, A, p.lda, m0, p.M, kbeg, kend);
    PB::fetch(rb, B, p.ldb, n0, p.N, kbeg, kend);
    PA::commit(smem, ra);
    PB::commit(smem + PA::BYTES, rb);
  }
  __syncthreads();

  for (int kt = 0; kt < nk; ++kt) {
    const char* sa = smem + (kt & 1) * STAGE;
    const char* sb = sa + PA::BYTES;
    const bool more = kt + 1 < nk;
    if (more) {
      const int k0 = kbeg + (kt + 1) * BK;
      PA::fetch(ra, A, p.lda, m0, p.M, k0, kend);
      PB::fetch(rb, B, p.ldb, n0, p.N, k0, kend);
    }
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      v8 fa[TM], fb[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) fa[i] = PA::frag(sa, wm * WTM + i * 32, ks, lane);
#pragma unroll
      for (int j = 0; j < TN; ++j) fb[j] = PB::frag(sb, wn * WTN + j * 32, ks, lane);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = mfma32(fb[j], fa[i], acc[i][j]);
    }
    if (more) {
      char* da = smem + ((kt + 1) & 1) * STAGE;
      PA::commit(da, ra);
      PB::commit(da + PA::BYTES, rb);
    }
    __syncthreads();
  }

  gemm_epilogue<T, TM, TN, WTM, WTN, VEC>(p, acc, m0, n0, wm, wn, lane, split);
}


// ---------------------------------------------------------------------------
// Fast path: HBM -> LDS directly (global_load_lds_dwordx4, no VGPR round trip),
// STAGES LDS buffers, loads issued STAGES-1 steps ahead of their use.
// A wave-level load writes 64 x 16 bytes to consecutive LDS addresses, so the
// chunk swizzle is applied on the GLOBAL side: the lane that owns LDS slot
// (row, c') fetches chunk c = c' ^ swz(row).  Rows / columns beyond M / N are
// clamped to valid memory (their products only reach C entries that are never
// stored); the contraction extent must be a multiple of BK.
// ---------------------------------------------------------------------------
typedef __attribute__((address_space(1))) const void gptr_void;

// s_waitcnt lgkmcnt(n): at most n LDS reads (the youngest) may still be in flight.
template <int N> __device__ __forceinline__ void wait_lgkmcnt() {
  __builtin_amdgcn_s_waitcnt(15 | (3 << 14) | (7 << 4) | ((N & 15) << 8));
}

// LDS operand reads issued as volatile asm: the compiler neither reorders them nor
// waits for them, so the kernel decides how far ahead of their MFMAs they run
// (every consumer sits behind an explicit wait_lgkmcnt + scheduling barrier).
template <bool KMAJOR> struct FragRegs;
template <> struct FragRegs<true> {
  u32x4 q;
  template <typename V8> __device__ __forceinline__ V8 get() const { return __builtin_bit_cast(V8, q); }
};
template <> struct FragRegs<false> {
  u32x2 lo, hi;
  template <typename V8> __device__ __forceinline__ V8 get() const {
    const u32x4 v = {lo[0], lo[1], hi[0], hi[1]};
    return __builtin_bit_cast(V8, v);
  }
};



template <typename T, int R, int BK, bool KMAJOR, int NW>
struct DmaPanel {
  static constexpr int CPR = KMAJOR ? BK / 8 : R / 8;
  static constexpr int LROWS = KMAJOR ? R : BK;
  static constexpr int NCHUNK = LROWS * CPR;
  static constexpr int BYTES = NCHUNK * 16;
  static constexpr int WLOADS = NCHUNK / 64;   // wave-level loads per panel
  static constexpr int PER_WAVE = WLOADS / NW;
  static_assert(WLOADS % NW == 0 && PER_WAVE >= 1, "panel must divide evenly over the waves");
  static_assert(KMAJOR ? (CPR == 4 || CPR == 8) : (CPR >= 16), "unsupported panel shape");

  static __device__ __forceinline__ int swz(int lrow, int c) {
    if constexpr (KMAJOR) return c ^ ((lrow / (16 / CPR)) % CPR);
    else return c ^ ((lrow & 3) << 2);
  }

  // Global address of each of this lane's chunks for the step starting at kbeg.
  static __device__ __forceinline__ void init(const T* (&ptrs)[PER_WAVE], const T* base, int64_t ld, int row0,
                                              int rmax, int kbeg, int wave, int lane) {
#pragma unroll
    for (int j = 0; j < PER_WAVE; ++j) {
      const int slot = (wave * PER_WAVE + j) * 64 + lane;
      const int lrow = slot / CPR;
      const int c = swz(lrow, slot % CPR);
      if (KMAJOR) {
        const int gr = min(row0 + lrow, rmax - 1);
        ptrs[j] = base + (int64_t)gr * ld + kbeg + c * 8;
      } else {
        int gr = row0 + c * 8;
        if (gr >= rmax) gr = row0;
        ptrs[j] = base + (int64_t)(kbeg + lrow) * ld + gr;
      }
    }
  }
  static __device__ __forceinline__ void issue(const T* (&ptrs)[PER_WAVE], char* lds, int wave) {
#pragma unroll
    for (int j = 0; j < PER_WAVE; ++j)
      __builtin_amdgcn_global_load_lds((gptr_void*)ptrs[j], (lds_void*)(lds + (wave * PER_WAVE + j) * 1024), 16, 0, 0);
  }
  static __device__ __forceinline__ void issue_one(const T* (&ptrs)[PER_WAVE], char* lds, int wave, int j) {
    __builtin_amdgcn_global_load_lds((gptr_void*)ptrs[j], (lds_void*)(lds + (wave * PER_WAVE + j) * 1024), 16, 0, 0);
  }
  static __device__ __forceinline__ void advance(const T* (&ptrs)[PER_WAVE], int64_t ld) {
#pragma unroll
    for (int j = 0; j < PER_WAVE; ++j) ptrs[j] += KMAJOR ? (int64_t)BK : (int64_t)BK * ld;
  }
  static __device__ __forceinline__ typename Vec<T>::v8 frag(const char* lds, int rb, int ks, int lane) {
    return Panel<T, R, BK, KMAJOR, 64, true>::frag(lds, rb, ks, lane);
  }
  static constexpr int READS_PER_FRAG = KMAJOR ? 1 : 2;
  // Same operand as frag(), read with volatile asm from the panel at LDS byte address `base`.
  static __device__ __forceinline__ void frag_issue(FragRegs<KMAJOR>& f, uint32_t base, int rb, int ks, int lane) {
    if constexpr (KMAJOR) {
      const int row = rb + (lane & 31);
      const int c = ks * 2 + (lane >> 5);
      const uint32_t a = base + (row * CPR + swz(row, c)) * 16;
      asm volatile("ds_read_b128 %0, %1" : "=v"(f.q) : "v"(a));
    } else {
      const int i = lane & 15;
      const int col = rb + 16 * ((lane >> 4) & 1) + (i & 3) * 4;
      const int kk0 = ks * 16 + 8 * (lane >> 5) + (i >> 2);
      const int kk1 = kk0 + 4;
      const uint32_t a0 = base + (kk0 * CPR + swz(kk0, col >> 3)) * 16 + (col & 7) * 2;
      const uint32_t a1 = base + (kk1 * CPR + swz(kk1, col >> 3)) * 16 + (col & 7) * 2;
      asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(f.lo) : "v"(a0));
      asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(f.hi) : "v"(a1));
    }
  }
};

// Epilogue of the direct-to-LDS kernel.  Each wave rounds its accumulators (after
// bias / ReLU), parks one 32-row block at a time in a private LDS region and
// reads it back row-contiguously, so every global store instruction writes whole
// 16-byte chunks of complete row segments (8 rows x 128 B for a 64-wide wave
// tile) instead of 32 scattered 16-byte pieces.
// PLAIN: the caller knows that there is no bias, ReLU, mask or sign-bit work (most launches of a
// training step): the write-out is then straight-line code without the tests for them.
template <typename T, typename TO, int TM, int TN, int WTM, int WTN, bool PLAIN = false, bool FULL = false>
__device__ __forceinline__ void gemm_epilogue_lds(const GemmParams& p, f32x16 (&acc)[TM][TN], char* smem, int m0,
                                                  int n0, int wm, int wn, int wave, int lane,
                                                  const uint8_t (*sign_bytes)[4] = nullptr) {
  constexpr int ES = (int)sizeof(TO);
  constexpr int ROWB = WTN * ES + 16;     // padded row pitch in bytes
  constexpr int CH = WTN * ES / 16;       // 16-byte chunks per row
  constexpr int RPI = 64 / CH;            // rows covered by one wave-wide access
  constexpr int EPC = 16 / ES;            // elements per chunk
  char* mine = smem + wave * (32 * ROWB);
  const T* bias = PLAIN ? nullptr : (const T*)p.bias;
  const bool relu = !PLAIN && p.relu;
  const void* mask = PLAIN ? nullptr : p.mask;
  const void* sign_in = PLAIN ? nullptr : p.sign_in;
  void* sign_out = PLAIN ? nullptr : p.sign_out;
  const float alpha = (!PLAIN && p.alpha) ? *p.alpha : 1.f;
  TO* C = (TO*)p.C;
  const int nbase = n0 + wn * WTN;
  // this lane stores the same 16-byte column chunk of every row it handles: the column part of the
  // address (with its division by the chunk width) is computed once, not per store (-0.2 ms per
  // step of the 410M model: the store loop is where short-contraction launches spend their time)
  const int n_lane = nbase + (lane % CH) * EPC;
  const int64_t col_off = n_lane + (int64_t)(n_lane / p.chunk_n) * p.chunk_skip;
  // ... and so is the row part of its first store; the others lie whole multiples of ldc further on
  TO* const row0 = C + (int64_t)(m0 + wm * WTM + lane / CH) * p.ldc + col_off;
  // this lane's bias values: the same for every 32-row block, requested once ahead of the loop
  typename Vec<T>::v4 bvals[TN][4] = {};
  if (bias) {
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int nl = j * 32 + g * 8 + (lane >> 5) * 4;
        if (nbase + nl < p.N) bvals[j][g] = *reinterpret_cast<const typename Vec<T>::v4*>(bias + nbase + nl);
      }
  }
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int nl = j * 32 + g * 8 + (lane >> 5) * 4;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = acc[i][j][g * 4 + e];
        if (!PLAIN) {
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] *= alpha;
        }
        if (bias) {
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] += (float)bvals[j][g][e];
        }
        if (relu) {
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = fmaxf(v[e], 0.f);
        }
        if (ES == 4) {
          f32x4 o = {v[0], v[1], v[2], v[3]};
          *reinterpret_cast<f32x4*>(mine + (lane & 31) * ROWB + nl * 4) = o;
        } else {
          typename Vec<T>::v4 o;
#pragma unroll
          for (int e = 0; e < 4; ++e) o[e] = (T)v[e];
          *reinterpret_cast<typename Vec<T>::v4*>(mine + (lane & 31) * ROWB + nl * 2) = o;
        }
      }
    }
    // all row segments of the block are requested from the slab before the first store: each store
    // then waits for its own read only (a read followed at once by its store exposes the LDS
    // latency once per store)
    u32x4 vals[32 / RPI];
#pragma unroll
    for (int rr = 0; rr < 32 / RPI; ++rr) vals[rr] = lds_ld16(mine, (rr * RPI + lane / CH) * ROWB + (lane % CH) * 16);
#pragma unroll
    for (int rr = 0; rr < 32 / RPI; ++rr) {
      const int r = rr * RPI + lane / CH, c = lane % CH;
      u32x4 val = vals[rr];
      const int m = m0 + wm * WTM + i * 32 + r, n = nbase + c * EPC;
      if (FULL || (m < p.M && n < p.N)) {
        if (mask) {  // ReLU gradient mask fused into the write-out: zero where the activation is not positive
          const T* mk = (const T*)mask + (int64_t)m * p.ldmask + n;
          if constexpr (ES == 2) {
            const typename Vec<T>::v8 mv = __builtin_bit_cast(typename Vec<T>::v8, ld16(mk));
            typename Vec<T>::v8 cv = __builtin_bit_cast(typename Vec<T>::v8, val);
#pragma unroll
            for (int e = 0; e < 8; ++e)
              if (!((float)mv[e] > 0.f)) cv[e] = (T)0.f;
            val = __builtin_bit_cast(u32x4, cv);
          } else {
            const typename Vec<T>::v4 mv = *reinterpret_cast<const typename Vec<T>::v4*>(mk);
            f32x4 cv = __builtin_bit_cast(f32x4, val);
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (!((float)mv[e] > 0.f)) cv[e] = 0.f;
            val = __builtin_bit_cast(u32x4, cv);
          }
        }
        if (sign_in) {  // the same mask from one bit per element
          unsigned bits;
          if constexpr (ES == 2) bits = sign_bytes[i][rr];  // requested before the main loop
          else bits = ((const uint8_t*)sign_in)[(int64_t)m * p.ldsign + (n >> 3)] >> (n & 7);
          if constexpr (ES == 2) {
            typename Vec<T>::v8 cv = __builtin_bit_cast(typename Vec<T>::v8, val);
#pragma unroll
            for (int e = 0; e < 8; ++e)
              if (!((bits >> e) & 1u)) cv[e] = (T)0.f;
            val = __builtin_bit_cast(u32x4, cv);
          } else {
            f32x4 cv = __builtin_bit_cast(f32x4, val);
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (!((bits >> e) & 1u)) cv[e] = 0.f;
            val = __builtin_bit_cast(u32x4, cv);
          }
        }
        if constexpr (ES == 2) {
          if (sign_out) {  // a chunk is 8 elements: one byte
            const typename Vec<T>::v8 cv = __builtin_bit_cast(typename Vec<T>::v8, val);
            unsigned bits = 0;
#pragma unroll
            for (int e = 0; e < 8; ++e) bits |= ((float)cv[e] > 0.f ? 1u : 0u) << e;
            ((uint8_t*)sign_out)[(int64_t)m * p.ldsign + (n >> 3)] = (uint8_t)bits;
          }
        }
        st16(row0 + (int64_t)(i * 32 + rr * RPI) * p.ldc, val);
      }
    }
  }
}

// One bit per element of a chunk of eight 16-bit values none of which is negative (a ReLU output;
// -0 counts as zero): bit e set where element e is positive.  Word arithmetic on the packed
// halves: h & 0x7fff is 0 or at least 1, so (h & 0x7fff) + 0x7fff carries into bit 15 exactly
// for the positive ones (and never into the neighbouring half).
__device__ __forceinline__ unsigned positive_bits8(u32x4 v) {
  unsigned b = 0;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const unsigned t = ((v[k] & 0x7fff7fffu) + 0x7fff7fffu) >> 15 & 0x00010001u;  // elements 2k (bit 0), 2k+1 (bit 16)
    b |= t << (2 * k);
  }
  return (b | b >> 15) & 0xffu;
}
// ... and the reverse: the chunk with every element whose bit is clear set to zero
__device__ __forceinline__ u32x4 keep_by_bits8(u32x4 v, unsigned bits) {
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const unsigned lo = (unsigned)__builtin_amdgcn_sbfe((int)bits, 2 * k, 1);      // 0 or 0xffffffff
    const unsigned hi = (unsigned)__builtin_amdgcn_sbfe((int)bits, 2 * k + 1, 1);
    v[k] &= __builtin_amdgcn_perm(hi, lo, 0x05040100u);  // bytes: lo.0 lo.1 hi.0 hi.1
  }
  return v;
}

// Write-out of a full tile with the ReLU sign bits, 16-bit result, no tests in the store loop.
//  BITS_OUT: C = relu(acc + bias), bits = (C > 0).  A lane's bit bytes go to an LDS image of the
//            tile's bits (BM rows of BN / 8 bytes) and leave it as whole 16-byte pieces after a
//            barrier: stored from the loop they would be 64 single bytes per store instruction,
//            eight to a row, a partial write of eight lines each.
//  !BITS_OUT: C = bit ? acc : 0, the bytes requested before the main loop (sign_bytes).
template <typename T, int BM, int BN, int TM, int TN, int WTM, int WTN, bool BITS_OUT>
__device__ __forceinline__ void gemm_epilogue_bits(const GemmParams& p, f32x16 (&acc)[TM][TN], char* smem, int m0, int n0,
                                                   int wm, int wn, int wave, int lane, const uint8_t (*sign_bytes)[4]) {
  constexpr int ROWB = WTN * 2 + 16, CH = WTN * 2 / 16, RPI = 64 / CH;
  constexpr int NW = (BM / WTM) * (BN / WTN);
  constexpr int IMG = NW * 32 * ROWB;  // the bit image lies behind the waves' slabs
  static_assert(BN / 8 % 16 == 0, "rows of the bit image are whole 16-byte pieces");
  char* mine = smem + wave * (32 * ROWB);
  const T* bias = (const T*)p.bias;
  T* C = (T*)p.C;
  const int nbase = n0 + wn * WTN;
  const int n_lane = nbase + (lane % CH) * 8;
  T* const row0 = C + (int64_t)(m0 + wm * WTM + lane / CH) * p.ldc + n_lane + (int64_t)(n_lane / p.chunk_n) * p.chunk_skip;
  typename Vec<T>::v4 bvals[TN][4] = {};
  if (BITS_OUT && bias) {
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int g = 0; g < 4; ++g) bvals[j][g] = *reinterpret_cast<const typename Vec<T>::v4*>(bias + nbase + j * 32 + g * 8 + (lane >> 5) * 4);
  }
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        typename Vec<T>::v4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float v = acc[i][j][g * 4 + e];
          if (BITS_OUT) v = fmaxf(v + (float)bvals[j][g][e], 0.f);
          o[e] = (T)v;
        }
        *reinterpret_cast<typename Vec<T>::v4*>(mine + (lane & 31) * ROWB + (j * 32 + g * 8 + (lane >> 5) * 4) * 2) = o;
      }
    u32x4 vals[32 / RPI];
#pragma unroll
    for (int rr = 0; rr < 32 / RPI; ++rr) vals[rr] = lds_ld16(mine, (rr * RPI + lane / CH) * ROWB + (lane % CH) * 16);
#pragma unroll
    for (int rr = 0; rr < 32 / RPI; ++rr) {
      u32x4 val = vals[rr];
      if (BITS_OUT) {
        const int row = wm * WTM + i * 32 + rr * RPI + lane / CH;  // in the tile
        smem[IMG + row * (BN / 8) + wn * (WTN / 8) + lane % CH] = (char)positive_bits8(val);
      } else {
        val = keep_by_bits8(val, sign_bytes[i][rr]);
      }
      st16(row0 + (int64_t)(i * 32 + rr * RPI) * p.ldc, val);
    }
  }
  if (BITS_OUT) {
    __syncthreads();
    constexpr int PIECES = BM * (BN / 8) / 16, PPR = BN / 8 / 16;  // 16-byte pieces of the image, per row
    uint8_t* out = (uint8_t*)p.sign_out + (int64_t)m0 * p.ldsign + n0 / 8;
    for (int q = threadIdx.x; q < PIECES; q += NW * 64)
      *reinterpret_cast<u32x4*>(out + (int64_t)(q / PPR) * p.ldsign + (q % PPR) * 16) = lds_ld16(smem, IMG + q * 16);
  }
}

// NS: pipeline stages in LDS.  2: ping-pong -- the loads of a stage are requested while the stage before it is
// being multiplied, and have one stage's time to arrive.  3: a stage's loads are requested two stages ahead
// and have two stages' time: for tiles whose stage is short (256x128: half the MFMAs of 256x256 per stage)
// one stage's time does not cover the latency of operands that come from HBM rather than from the L2.
template <typename T, int BM, int BN, int BK, int WM, int WN, bool A_KMAJOR, bool B_KMAJOR, int NS = 2>
__device__ __forceinline__ void gemm_dma_body(const GemmParams& p, const int pid) {
  static_assert(NS == 2 || NS == 3, "two or three pipeline stages");
  constexpr int NW = WM * WN;
  constexpr int WTM = BM / WM, WTN = BN / WN;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int GROUP_M = 8;
  constexpr int KSTEPS = BK / 16;
  typedef DmaPanel<T, BM, BK, A_KMAJOR, NW> PA;
  typedef DmaPanel<T, BN, BK, B_KMAJOR, NW> PB;
  typedef typename Vec<T>::v8 v8;
  constexpr int STAGE = PA::BYTES + PB::BYTES;      // two stages, ping-pong
  constexpr int LPS = PA::PER_WAVE + PB::PER_WAVE;  // loads per wave per stage
  constexpr int NEARLY = LPS / 2;  // loads of a stage issued right after the hand-over to the stage before it
  static_assert(KSTEPS >= 3, "the loop deals its loads and pointer updates over the first two steps and the last one");
  static_assert(KSTEPS % 2 == 0, "operand register ping-pong needs an even number of contraction steps");
  extern __shared__ __attribute__((aligned(16))) char smem[];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform: LDS slab addresses stay scalar
  const int wm = wave / WN, wn = wave % WN;

  const int tiles = p.tiles_m * p.tiles_n;
  const int split = pid / tiles;
  const int t = pid - split * tiles;
  const int per_group = GROUP_M * p.tiles_n;
  const int group = t / per_group;
  const int first_m = group * GROUP_M;
  const int gsz = min(p.tiles_m - first_m, GROUP_M);
  const int tm = first_m + (t % per_group) % gsz;
  const int tn = (t % per_group) / gsz;
  const int m0 = tm * BM, n0 = tn * BN;
  const int kbeg = split * p.k_per_split;
  const int kend = min(p.K, kbeg + p.k_per_split);
  const int nk = (kend - kbeg) / BK;

  const T* pa[PA::PER_WAVE];
  const T* pb[PB::PER_WAVE];
  PA::init(pa, (const T*)p.A, p.lda, m0, p.M, kbeg, wave, lane);
  PB::init(pb, (const T*)p.B, p.ldb, n0, p.N, kbeg, wave, lane);

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // Mask bits of a 16-bit result: this lane's bytes (one per 8-element chunk it will store, in the
  // order of the write-out) are requested here, a whole main loop ahead of their use -- loaded in
  // the write-out they would sit between every LDS read and the store that needs both.
  static_assert(64 / (WTN * 2 / 16) * 4 == 32, "four wave-wide stores per 32-row block of a 16-bit result");
  uint8_t sign_bytes[TM][4] = {};
  if (p.sign_in && !p.out_f32) {
    constexpr int CH16 = WTN * 2 / 16, RPI16 = 64 / CH16;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) {
        const int m = m0 + wm * WTM + i * 32 + rr * RPI16 + lane / CH16, n = n0 + wn * WTN + (lane % CH16) * 8;
        if (m < p.M && n < p.N) sign_bytes[i][rr] = ((const uint8_t*)p.sign_in)[(int64_t)m * p.ldsign + (n >> 3)];
      }
  }

  // Bare s_barrier everywhere in the pipeline: __syncthreads() adds a fence that would
  // drain every outstanding direct-to-LDS load.  The waits that matter are explicit.
  auto barrier = [&]() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };
  FragRegs<A_KMAJOR> fa[2][TM];
  FragRegs<B_KMAJOR> fb[2][TN];
  auto read_operands = [&](const char* stage, int ks, int buf) {
    const uint32_t sa_addr = lds_address(stage), sb_addr = sa_addr + PA::BYTES;
#pragma unroll
    for (int i = 0; i < TM; ++i) PA::frag_issue(fa[buf][i], sa_addr, wm * WTM + i * 32, ks, lane);
#pragma unroll
    for (int j = 0; j < TN; ++j) PB::frag_issue(fb[buf][j], sb_addr, wn * WTN + j * 32, ks, lane);
  };

  // ---- prologue: step 0 into stage 0, then its first operands and the head of step 1
  if (nk > 0) {
    PA::issue(pa, smem, wave);
    PB::issue(pb, smem + PA::BYTES, wave);
    PA::advance(pa, p.lda);
    PB::advance(pb, p.ldb);
    // the head of step 1 goes out before step 0 is waited for: the two travel together through
    // the cold start instead of one after the other
    if constexpr (NS == 3) {
      // three buffers: all of step 1 and the head of step 2
      if (nk > 1) {
        PA::issue(pa, smem + STAGE, wave);
        PB::issue(pb, smem + STAGE + PA::BYTES, wave);
        PA::advance(pa, p.lda);
        PB::advance(pb, p.ldb);
        if (nk > 2) {
#pragma unroll
          for (int q = 0; q < NEARLY; ++q) {
            if (q < PA::PER_WAVE) PA::issue_one(pa, smem + 2 * STAGE, wave, q);
            else PB::issue_one(pb, smem + 2 * STAGE + PA::BYTES, wave, q - PA::PER_WAVE);
          }
          wait_vmcnt<LPS + NEARLY>();  // loads complete in order: all but the youngest LPS + NEARLY = step 0
        } else {
          wait_vmcnt<LPS>();
        }
      } else {
        wait_vmcnt<0>();
      }
    } else if (nk > 1) {
#pragma unroll
      for (int q = 0; q < NEARLY; ++q) {
        if (q < PA::PER_WAVE) PA::issue_one(pa, smem + STAGE, wave, q);
        else PB::issue_one(pb, smem + STAGE + PA::BYTES, wave, q - PA::PER_WAVE);
      }
      wait_vmcnt<NEARLY>();  // loads complete in order: all but the NEARLY youngest = step 0
    } else {
      wait_vmcnt<0>();
    }
    barrier();
    read_operands(smem, 0, 0);
  }

  // ---- main loop.  Every LDS read, load and pointer update sits behind an MFMA, pinned there by
  // scheduling barriers: the matrix pipe is busy for 32 cycles per MFMA and the wave is free to
  // issue meanwhile.  Per 16-wide step there are NMFMA slots; the operand reads of the next step
  // go behind the first ones (register ping-pong: the MFMAs of step ks read set ks % 2), the extras
  // of the step behind the rest -- half of the next stage's loads at step 0, the pointer updates
  // at step 1, and in the last step the hand-over (wait for this wave's loads, barrier) followed
  // by the first operand reads of the next stage and the other half of the loads, which go into
  // the buffer everyone has just left.
  constexpr int NMFMA = TM * TN;
  constexpr int NR = TM + TN;                                       // read items (one fragment each)
  constexpr int RPS = (NR + NMFMA - 1) / NMFMA;                     // read items per slot
  constexpr int RSLOTS = (NR + RPS - 1) / RPS;                      // slots that carry reads
  constexpr int HAND = NMFMA - RSLOTS >= 4 ? 2 : 0;                 // MFMAs of the last step ahead of the barrier
  static_assert(HAND + RSLOTS <= NMFMA, "the reads of a step must fit behind its MFMAs");
  static_assert(LPS % 2 == 0, "loads go out in two halves");
  auto read_item = [&](const char* stage, int ks, int buf, int item) {
    const uint32_t sa_addr = lds_address(stage), sb_addr = sa_addr + PA::BYTES;
    if (item < TM) PA::frag_issue(fa[buf][item], sa_addr, wm * WTM + item * 32, ks, lane);
    else PB::frag_issue(fb[buf][item - TM], sb_addr, wn * WTN + (item - TM) * 32, ks, lane);
  };
  auto load_item = [&](char* dst, int q) {
    if (q < PA::PER_WAVE) PA::issue_one(pa, dst, wave, q);
    else PB::issue_one(pb, dst + PA::BYTES, wave, q - PA::PER_WAVE);
  };
  auto advance_item = [&](int q) {
    if (q < PA::PER_WAVE) pa[q] += A_KMAJOR ? (int64_t)BK : (int64_t)BK * p.lda;
    else pb[q - PA::PER_WAVE] += B_KMAJOR ? (int64_t)BK : (int64_t)BK * p.ldb;
  };
  // One 64-wide stage.  MORE: another stage follows (hand over to it); MORE2: and one after that
  // (its first loads go out).  Compile-time, so the steady state of the loop has no branch.
  // With three buffers (NS == 3) everything that is loaded lies one stage further ahead: step 0 sends the
  // rest of the stage after the next one into the third buffer `far`, the last step the head of the stage
  // after that into `cur`; MORE3: that stage exists.  The hand-over then waits for all but the youngest
  // stage's loads.
  auto stage = [&](char* cur, char* nxt, char* far, auto more_c, auto more2_c, auto more3_c) {
    constexpr bool MORE = decltype(more_c)::value, MORE2 = decltype(more2_c)::value, MORE3 = decltype(more3_c)::value;
    constexpr bool LOAD0 = NS == 3 ? MORE2 : MORE;    // step 0 has loads to send (and step 1 pointers to move)
    constexpr bool LOADL = NS == 3 ? MORE3 : MORE2;   // the last step has
    char* const dst0 = NS == 3 ? far : nxt;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      const bool last = ks + 1 == KSTEPS;
      const int first = last ? HAND : 0;                 // first slot that carries work of this step
      const int xfirst = first + RSLOTS < NMFMA ? first + RSLOTS : NMFMA - 1;  // extras: behind the reads
      const int xslots = NMFMA - xfirst;
      const int nx = last ? (LOADL ? NEARLY : 0) : !LOAD0 ? 0 : ks == 0 ? LPS - NEARLY : ks == 1 ? LPS : 0;
      wait_lgkmcnt<0>();  // the operands of this step were requested a whole step ago
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int m = 0; m < NMFMA; ++m) {
        const int i = m / TN, j = m % TN;
        if (last && m == HAND && MORE) {
          // (Measurement switches, never defined by the build: TF_ABL_NO_LOAD_WAIT_TILE / TF_ABL_NO_HANDOVER_BARRIER_TILE
          // = BM * BN of the configuration whose wait / barrier is compiled out.  The results of such a build are
          // wrong; its step time says what the wait costs -- how the need for a third stage was found.)
#ifdef TF_ABL_NO_LOAD_WAIT_TILE
          if (BM * BN != TF_ABL_NO_LOAD_WAIT_TILE)
#endif
          wait_vmcnt<(NS == 3 && MORE2) ? LPS : 0>();  // this wave's loads of the next stage have landed
#ifdef TF_ABL_NO_HANDOVER_BARRIER_TILE
          if (BM * BN != TF_ABL_NO_HANDOVER_BARRIER_TILE)
#endif
          barrier();        // ... and everyone's; everyone has read the last operands of `cur`
          __builtin_amdgcn_sched_barrier(0);
        }
        acc[i][j] = mfma32(fb[ks & 1][j].template get<v8>(), fa[ks & 1][i].template get<v8>(), acc[i][j]);
        __builtin_amdgcn_sched_barrier(0);
        if (m >= first && (!last || MORE)) {
#pragma unroll
          for (int r = (m - first) * RPS; r < (m - first + 1) * RPS && r < NR; ++r) {
            if (last) read_item(nxt, 0, 0, r);
            else read_item(cur, ks + 1, (ks + 1) & 1, r);
          }
        }
        if (m >= xfirst) {
#pragma unroll
          for (int q = (m - xfirst) * nx / xslots; q < (m - xfirst + 1) * nx / xslots; ++q) {
            if (last) load_item(cur, q);                 // first half of the stage after the next one (NS == 3: one further)
            else if (ks == 0) load_item(dst0, NEARLY + q);  // the rest of the next stage (NS == 3: of the one after it)
            else advance_item(q);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  typedef std::integral_constant<bool, true> yes_t;
  typedef std::integral_constant<bool, false> no_t;
  int kt = 0;
  if constexpr (NS == 3) {
    int o0 = 0, o1 = STAGE, o2 = 2 * STAGE;   // buffers of this stage, the next one and the one after it
    auto rotate = [&]() { const int t = o0; o0 = o1; o1 = o2; o2 = t; ++kt; };
    for (; kt + 3 < nk; rotate()) stage(smem + o0, smem + o1, smem + o2, yes_t(), yes_t(), yes_t());
    if (kt + 2 < nk) { stage(smem + o0, smem + o1, smem + o2, yes_t(), yes_t(), no_t()); rotate(); }
    if (kt + 1 < nk) { stage(smem + o0, smem + o1, smem + o2, yes_t(), no_t(), no_t()); rotate(); }
    if (kt < nk) stage(smem + o0, smem + o1, smem + o2, no_t(), no_t(), no_t());
  } else {
    for (; kt + 2 < nk; ++kt)
      stage(smem + (kt & 1) * STAGE, smem + ((kt + 1) & 1) * STAGE, nullptr, yes_t(), yes_t(), no_t());
    if (kt + 1 < nk) {
      stage(smem + (kt & 1) * STAGE, smem + ((kt + 1) & 1) * STAGE, nullptr, yes_t(), no_t(), no_t());
      ++kt;
    }
    if (kt < nk) stage(smem + (kt & 1) * STAGE, smem + ((kt + 1) & 1) * STAGE, nullptr, no_t(), no_t(), no_t());
  }

  static_assert(NW * 32 * (WTN * 4 + 16) <= 2 * STAGE, "epilogue staging must fit in the pipeline LDS");
  static_assert(NW * 32 * (WTN * 2 + 16) + BM * BN / 8 <= 2 * STAGE, "... and so must the image of a tile's sign bits behind it");
  const bool full = m0 + BM <= p.M && n0 + BN <= p.N;  // no row or column of the tile lies outside C: stores need no test
  if (p.splits > 1) {
    // fp32 partial of this contraction slice: a plain (M, N) matrix, written like an fp32 result
    GemmParams q = p;
    q.C = p.partial + (int64_t)split * p.M * p.N;
    q.ldc = p.N;
    q.bias = nullptr;
    q.relu = 0;
    q.mask = nullptr;
    q.sign_out = nullptr;
    q.sign_in = nullptr;
    q.alpha = nullptr;
    q.chunk_n = p.N;
    q.chunk_skip = 0;
    __syncthreads();  // all waves are done reading the last pipeline stage
    if (full) gemm_epilogue_lds<T, float, TM, TN, WTM, WTN, true, true>(q, acc, smem, m0, n0, wm, wn, wave, lane);
    else gemm_epilogue_lds<T, float, TM, TN, WTM, WTN, true>(q, acc, smem, m0, n0, wm, wn, wave, lane);
  } else {
    __syncthreads();  // all waves are done reading the last pipeline stage
    const bool plain = !p.bias && !p.relu && !p.mask && !p.sign_in && !p.sign_out && !p.alpha;
    if (p.out_f32) {
      if (plain && full) gemm_epilogue_lds<T, float, TM, TN, WTM, WTN, true, true>(p, acc, smem, m0, n0, wm, wn, wave, lane);
      else if (plain) gemm_epilogue_lds<T, float, TM, TN, WTM, WTN, true>(p, acc, smem, m0, n0, wm, wn, wave, lane);
      else gemm_epilogue_lds<T, float, TM, TN, WTM, WTN>(p, acc, smem, m0, n0, wm, wn, wave, lane);
    } else {
      // the two sign-bit launches of a fused MLP, on full tiles of a plain (unchunked) result whose bit rows take
      // 16-byte pieces: write-outs of their own, nothing tested per store
      const bool bits_fast = full && !p.mask && !p.alpha && p.chunk_skip == 0 && p.ldsign % 16 == 0 &&
                             ((reinterpret_cast<uintptr_t>(p.sign_out) | reinterpret_cast<uintptr_t>(p.sign_in)) & 15) == 0;
      if (plain && full) gemm_epilogue_lds<T, T, TM, TN, WTM, WTN, true, true>(p, acc, smem, m0, n0, wm, wn, wave, lane);
      else if (plain) gemm_epilogue_lds<T, T, TM, TN, WTM, WTN, true>(p, acc, smem, m0, n0, wm, wn, wave, lane);
      else if (bits_fast && p.sign_out && p.relu) gemm_epilogue_bits<T, BM, BN, TM, TN, WTM, WTN, true>(p, acc, smem, m0, n0, wm, wn, wave, lane, sign_bytes);
      else if (bits_fast && p.sign_in && !p.bias && !p.relu) gemm_epilogue_bits<T, BM, BN, TM, TN, WTM, WTN, false>(p, acc, smem, m0, n0, wm, wn, wave, lane, sign_bytes);
      else gemm_epilogue_lds<T, T, TM, TN, WTM, WTN>(p, acc, smem, m0, n0, wm, wn, wave, lane, sign_bytes);
    }
  }
}

template <typename T, int BM, int BN, int BK, int WM, int WN, int WPE, bool A_KMAJOR, bool B_KMAJOR, int NS = 2>
__global__ __launch_bounds__(WM* WN * 64, WPE) void gemm_dma_kernel(GemmParams p) {
  const int pid = (p.flags & 1) ? (int)blockIdx.x : remap_xcd(blockIdx.x, p.tiles_m * p.tiles_n * p.splits, p.xcds);
  gemm_dma_body<T, BM, BN, BK, WM, WN, A_KMAJOR, B_KMAJOR, NS>(p, pid);
}

// Up to sixteen independent products of one operand layout in ONE launch: workgroup ids
// [first[i], first[i+1]) belong to problem i.  Used for weight gradients, whose output has
// few tiles: side by side they fill the chip with fewer, longer contraction slices.
constexpr int kMaxGroup = 16;
struct GemmGroup {
  GemmParams p[kMaxGroup];
  int first[kMaxGroup + 1];
  int count;
};
static_assert(sizeof(GemmGroup) <= 4000, "the group travels as a kernel argument (4 KB of them at most)");
template <typename T, int BM, int BN, int BK, int WM, int WN, int WPE, bool A_KMAJOR, bool B_KMAJOR>
__global__ __launch_bounds__(WM* WN * 64, WPE) void gemm_dma_group_kernel(GemmGroup g) {
  // (a group with a split tail keeps the ids as dealt, round-robin over the XCDs: whole tiles first, on every
  // XCD alike, then the short slices of the tail -- the remap would hand all of the tail to the last XCDs)
  const int pid = (g.p[0].flags & 1) ? (int)blockIdx.x : remap_xcd(blockIdx.x, g.first[g.count], g.p[0].xcds);
  int i = 0;
#pragma unroll
  for (int k = 1; k < kMaxGroup; ++k)
    if (k < g.count && pid >= g.first[k]) i = k;
  gemm_dma_body<T, BM, BN, BK, WM, WN, A_KMAJOR, B_KMAJOR>(g.p[i], pid - g.first[i]);
}

// Sum the split-contraction partials in a fixed order and apply the epilogue.
// VEC4: N and ldc multiples of 4, 16-byte aligned partials, 8-byte aligned C.
template <typename T, typename TO, bool VEC4>
__global__ __launch_bounds__(256) void gemm_reduce(int M, int N, int splits, const float* __restrict__ partial,
                                                    const T* __restrict__ bias, int relu, TO* __restrict__ C,
                                                    int64_t ldc, int chunk_n, int64_t chunk_skip,
                                                    const float* __restrict__ alpha_ptr) {
  const int64_t total = (int64_t)M * N;
  const float alpha = alpha_ptr ? *alpha_ptr : 1.f;
  if (VEC4) {
    const int64_t quads = total >> 2;
    for (int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x; q < quads; q += (int64_t)gridDim.x * 256) {
      f32x4 s = *reinterpret_cast<const f32x4*>(partial + q * 4);
      for (int k = 1; k < splits; ++k) s += *reinterpret_cast<const f32x4*>(partial + (int64_t)k * total + q * 4);
      const int64_t i = q * 4;
      const int m = (int)(i / N), n = (int)(i - (int64_t)m * N);
      TO o[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float x = s[e] * alpha + (bias ? (float)bias[n + e] : 0.f);
        o[e] = (TO)(relu ? fmaxf(x, 0.f) : x);
      }
      struct alignas(sizeof(TO) * 4) Quad { TO v[4]; };
      Quad qd;
#pragma unroll
      for (int e = 0; e < 4; ++e) qd.v[e] = o[e];
      store_out(C + (int64_t)m * ldc + n + (int64_t)(n / chunk_n) * chunk_skip, qd);
    }
  } else {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
      float s = 0.f;
      for (int k = 0; k < splits; ++k) s += partial[(int64_t)k * total + i];
      const int m = (int)(i / N), n = (int)(i - (int64_t)m * N);
      s *= alpha;
      if (bias) s += (float)bias[n];
      C[(int64_t)m * ldc + n + (int64_t)(n / chunk_n) * chunk_skip] = (TO)(relu ? fmaxf(s, 0.f) : s);
    }
  }
}

// The same second pass for up to kMaxGroup products of one grouped launch at once (blockIdx.y = product;
// no bias, no ReLU): one launch instead of one per product.
struct ReduceItem {
  const float* partial;
  void* C;
  int64_t ldc, chunk_skip;
  int M, N, splits, chunk_n;
};
struct ReduceBatch { ReduceItem it[kMaxGroup]; };
template <typename TO, bool VEC4>
__global__ __launch_bounds__(256) void gemm_reduce_group(ReduceBatch batch) {
  const ReduceItem r = batch.it[blockIdx.y];
  if (r.splits <= 1) return;
  const int64_t total = (int64_t)r.M * r.N;
  TO* C = (TO*)r.C;
  if (VEC4) {
    const int64_t quads = total >> 2;
    for (int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x; q < quads; q += (int64_t)gridDim.x * 256) {
      f32x4 s = *reinterpret_cast<const f32x4*>(r.partial + q * 4);
      for (int k = 1; k < r.splits; ++k) s += *reinterpret_cast<const f32x4*>(r.partial + (int64_t)k * total + q * 4);
      const int64_t i = q * 4;
      const int m = (int)(i / r.N), n = (int)(i - (int64_t)m * r.N);
      struct alignas(sizeof(TO) * 4) Quad { TO v[4]; };
      Quad qd;
#pragma unroll
      for (int e = 0; e < 4; ++e) qd.v[e] = (TO)s[e];
      store_out(C + (int64_t)m * r.ldc + n + (int64_t)(n / r.chunk_n) * r.chunk_skip, qd);
    }
  } else {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
      float s = 0.f;
      for (int k = 0; k < r.splits; ++k) s += r.partial[(int64_t)k * total + i];
      const int m = (int)(i / r.N), n = (int)(i - (int64_t)m * r.N);
      C[(int64_t)m * r.ldc + n + (int64_t)(n / r.chunk_n) * r.chunk_skip] = (TO)s;
    }
  }
}

// ---------------------------------------------------------------------------
// host side: tile choice, contraction split, launch
// ---------------------------------------------------------------------------
struct GemmPlan {
  int cfg;
  int bm, bn, bk;
  int tiles_m, tiles_n, splits, k_per_split;
};

struct TileCfg { int bm, bn, bk, waves, dma; };  // dma: direct-to-LDS kernel
// index = cfg id used by launch_cfg below
static const TileCfg kCfgs[] = {
    {256, 256, 64, 8, 0},  // 0: register-staged, wave tile 128x64, any shape / alignment
    {128, 128, 64, 4, 0},  // 1: register-staged, wave tile 64x64, any shape / alignment
    {256, 256, 64, 8, 1},  // 2: direct-to-LDS, 128 KB LDS, one workgroup per CU, wave tile 128x64
    {128, 128, 64, 4, 1},  // 3: direct-to-LDS, 64 KB LDS, two workgroups per CU, wave tile 64x64
    {256, 128, 64, 8, 1},  // 4: direct-to-LDS, three stages = 144 KB LDS, waves 4x2, wave tile 64x64
    {128, 256, 64, 8, 1},  // 5: direct-to-LDS, three stages = 144 KB LDS, waves 2x4, wave tile 64x64
};
constexpr int kNumCfgs = (int)(sizeof(kCfgs) / sizeof(kCfgs[0]));

// What the diagnostic entry point may impose on ONE call (nothing is kept between calls):
// a tile configuration (index into kCfgs, -1 = chosen by the cost model), a contraction
// split (0 = chosen), and flag bits -- 1: no XCD remap of the workgroup ids; 64: never cut
// a product along N.  Every product entry point passes kNoForce.
struct GemmForce { int cfg, splits, flags; };
constexpr GemmForce kNoForce = {-1, 0, 0};

// Tile shape, contraction split and the rough cost (microseconds) of running
// M x N x K with tile configuration `cfg`.  The cost constants are fits to
// rocprofv3 kernel durations on MI355X: one "round" of workgroups (one per CU)
// costs a fixed part (launch, cold first loads, result write-out) plus a part
// per 64-wide contraction step.
static GemmPlan plan_for(int cfg, int64_t M, int64_t N, int64_t K, double* cost_us, bool allow_split,
                         int force_splits = 0) {
  GemmPlan pl;
  pl.cfg = cfg;
  pl.bm = kCfgs[cfg].bm;
  pl.bn = kCfgs[cfg].bn;
  pl.bk = kCfgs[cfg].bk;
  pl.tiles_m = (int)((M + pl.bm - 1) / pl.bm);
  pl.tiles_n = (int)((N + pl.bn - 1) / pl.bn);
  const int64_t tiles = (int64_t)pl.tiles_m * pl.tiles_n;
  const int64_t ksteps = (K + pl.bk - 1) / pl.bk;
  const int wg_per_cu = pl.bm * pl.bn <= 128 * 128 ? 2 : 1;
  const int64_t slots = (int64_t)device_shape().cus * wg_per_cu;
  // Split the contraction only when the tiles alone leave most CUs idle (weight
  // gradients: few output tiles, long contraction); never beyond one full round of
  // workgroups, and every slice keeps at least 16 steps so that the fp32 partial
  // traffic stays small.
#ifndef TF_STEP_256x128
#define TF_STEP_256x128 1.0
#endif
  const double fixed = pl.bm * pl.bn >= 256 * 256 ? 10.0 : 7.0;
  const double per_step = pl.bm * pl.bn >= 256 * 256 ? 1.65 : (pl.bm * pl.bn >= 256 * 128 ? TF_STEP_256x128 : 1.1);
  auto cost_of = [&](int64_t nsplit, int64_t steps) {
    const int64_t rounds = (tiles * nsplit + slots - 1) / slots;
    double c = (double)rounds * (fixed + per_step * (double)steps);
    if (nsplit > 1) c += 3.0 + (nsplit + 0.5) * (double)M * (double)N * 4.0 / 5.0e6;
    return c;
  };
  int64_t splits = 1;
  if (tiles <= slots / 2) {
    splits = slots / tiles;
    const int64_t max_by_k = ksteps / 16 > 0 ? ksteps / 16 : 1;
    if (splits > max_by_k) splits = max_by_k;
    if (splits > 16) splits = 16;
  }
  // A long contraction whose tiles leave part of a round idle (0.75 of a round: the LM-head input gradient
  // of a narrow model) may be cheaper in more, shorter slices that fill whole rounds: by the cost model,
  // among slice counts that keep 16 steps per slice, and only when it wins by a tenth.
#ifdef TF_NO_SPLIT_SEARCH
  if (false) {
#else
  if (allow_split && force_splits <= 0 && tiles % slots != 0 && ksteps >= 256) {
#endif
    double best = cost_of(splits, (ksteps + splits - 1) / splits) * 0.9;
    for (int64_t sp = 2; sp <= 16 && ksteps / sp >= 16; ++sp) {
      const double c = cost_of(sp, (ksteps + sp - 1) / sp);
      if (c < best) { best = c; splits = sp; }
    }
  }
  if (force_splits > 0) splits = force_splits;
  if (!allow_split) splits = 1;
  if (splits > ksteps) splits = ksteps > 0 ? ksteps : 1;
  const int64_t steps_per = (ksteps + splits - 1) / splits;
  pl.k_per_split = (int)(steps_per * pl.bk);
  pl.splits = (int)((ksteps + steps_per - 1) / steps_per);
  if (pl.splits < 1) pl.splits = 1;
  if (cost_us) *cost_us = cost_of(pl.splits, steps_per);
  return pl;
}

static GemmPlan make_plan(int64_t M, int64_t N, int64_t K, bool vec, bool allow_split = true,
                          double* cost_us = nullptr, const GemmForce& force = kNoForce) {
  const bool dma = vec && K % 64 == 0;
  if (cost_us) *cost_us = -1.0;  // stays negative when the configuration is forced
  if (force.cfg >= 0 && force.cfg < kNumCfgs) {
    int cfg = force.cfg;
    if (kCfgs[cfg].dma && !dma) cfg = kCfgs[cfg].bm * kCfgs[cfg].bn >= 256 * 256 ? 0 : 1;  // register-staged twin
    return plan_for(cfg, M, N, K, nullptr, allow_split, force.splits);
  }
  // candidates: 256x256 and 256x128 / 128x128 tiles, direct-to-LDS kernels when their
  // preconditions hold, the register-staged twins otherwise
  const int cand_dma[3] = {2, 4, 3};
  const int cand_reg[2] = {0, 1};
  const int* cand = dma ? cand_dma : cand_reg;
  const int ncand = dma ? 3 : 2;
  GemmPlan best = plan_for(cand[0], M, N, K, nullptr, allow_split, force.splits);
  double best_cost = 1e30;
  for (int i = 0; i < ncand; ++i) {
    double c;
    const GemmPlan pl = plan_for(cand[i], M, N, K, &c, allow_split, force.splits);
    if (c < best_cost) { best_cost = c; best = pl; }
  }
  if (cost_us) *cost_us = best_cost;
  return best;
}

// Diagnostic: GEMM kernel launches since the library was loaded (reduce passes not counted).
static std::atomic<int64_t> g_gemm_launches{0};

template <typename K>
static void allow_big_lds(K kernel, int bytes) {
  if (bytes > 64 * 1024)
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
}

template <typename T, int BM, int BN, int BK, int WM, int WN, bool AK, bool BKM, bool VEC>
static int launch_one(hipStream_t st, const GemmParams& p) {
  typedef Panel<T, BM, BK, AK, WM * WN * 64, VEC> PA;
  typedef Panel<T, BN, BK, BKM, WM * WN * 64, VEC> PB;
  constexpr int lds = 2 * (PA::BYTES + PB::BYTES);
  auto kernel = gemm_kernel<T, BM, BN, BK, WM, WN, AK, BKM, VEC>;
  static bool once = (allow_big_lds(kernel, lds), true);
  (void)once;
  const unsigned grid = (unsigned)(p.tiles_m * p.tiles_n * p.splits);
  kernel<<<dim3(grid), dim3(WM * WN * 64), lds, st>>>(p);
  TF_CHECK_LAUNCH();
  g_gemm_launches.fetch_add(1, std::memory_order_relaxed);
  return TF_OK;
}

template <typename T, int BM, int BN, int BK, int WM, int WN, int WPE, bool AK, bool BKM, int NS = 2>
static int launch_dma(hipStream_t st, const GemmParams& p) {
  constexpr int lds = NS * (BM + BN) * BK * 2;
  static_assert(lds <= 160 * 1024, "LDS budget");
  auto kernel = gemm_dma_kernel<T, BM, BN, BK, WM, WN, WPE, AK, BKM, NS>;
  static bool once = (allow_big_lds(kernel, lds), true);
  (void)once;
  const unsigned grid = (unsigned)(p.tiles_m * p.tiles_n * p.splits);
  kernel<<<dim3(grid), dim3(WM * WN * 64), lds, st>>>(p);
  TF_CHECK_LAUNCH();
  g_gemm_launches.fetch_add(1, std::memory_order_relaxed);
  return TF_OK;
}

// The register-staged kernel handles everything (ragged extents, unaligned
// pointers); the direct-to-LDS kernel needs the vector conditions and a
// contraction extent that is a multiple of its BK.
// LDS stages of the 256x128 / 128x256 configurations (a diagnostic build may impose 2)
#ifndef TF_STAGES_NARROW
#define TF_STAGES_NARROW 3
#endif
constexpr int kStagesNarrow = TF_STAGES_NARROW;

template <typename T, bool AK, bool BKM, bool VEC>
static int launch_cfg(hipStream_t st, const GemmPlan& pl, const GemmParams& p) {
  if (kCfgs[pl.cfg].dma && VEC && p.K % pl.bk == 0) {
    switch (pl.cfg) {
      case 2: return launch_dma<T, 256, 256, 64, 2, 4, 2, AK, BKM>(st, p);
      case 3: return launch_dma<T, 128, 128, 64, 2, 2, 2, AK, BKM>(st, p);
      case 4: return launch_dma<T, 256, 128, 64, 4, 2, 2, AK, BKM, kStagesNarrow>(st, p);
      case 5: return launch_dma<T, 128, 256, 64, 2, 4, 2, AK, BKM, kStagesNarrow>(st, p);
    }
  }
  if (pl.bm == 256 && pl.bn == 256) return launch_one<T, 256, 256, 64, 2, 4, AK, BKM, VEC>(st, p);
  if (pl.bm == 128 && pl.bn == 128) return launch_one<T, 128, 128, 64, 2, 2, AK, BKM, VEC>(st, p);
  return TF_EINVAL;
}

// Second pass of a split contraction (no-op when the contraction was not split).
template <typename T>
static int launch_reduce(hipStream_t st, const GemmParams& p) {
  if (p.splits <= 1) return TF_OK;
  const int64_t total = (int64_t)p.M * p.N;
  const bool v4 = p.N % 4 == 0 && p.ldc % 4 == 0 && p.chunk_n % 4 == 0 && p.chunk_skip % 4 == 0 &&
                  (reinterpret_cast<uintptr_t>(p.C) & 15) == 0;
  int64_t blocks = ((v4 ? total / 4 : total) + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  if (blocks < 1) blocks = 1;
  const dim3 g((unsigned)blocks), b(256);
  const T* bias = (const T*)p.bias;
#define REDUCE(TO, V4) \
  gemm_reduce<T, TO, V4><<<g, b, 0, st>>>(p.M, p.N, p.splits, p.partial, bias, p.relu, (TO*)p.C, p.ldc, p.chunk_n, \
                                          p.chunk_skip, p.alpha)
  if (p.out_f32) { if (v4) REDUCE(float, true); else REDUCE(float, false); }
  else { if (v4) REDUCE(T, true); else REDUCE(T, false); }
#undef REDUCE
  TF_CHECK_LAUNCH();
  return TF_OK;
}

template <typename T>
static int gemm_dispatch(hipStream_t st, int la, int lb, bool vec, const GemmPlan& pl, const GemmParams& p) {
  const bool ak = la == TF_OP_KMAJOR, bk = lb == TF_OP_KMAJOR;
  int rc;
#define GO(AK, BKM) rc = vec ? launch_cfg<T, AK, BKM, true>(st, pl, p) : launch_cfg<T, AK, BKM, false>(st, pl, p)
  if (ak && bk) GO(true, true);
  else if (ak && !bk) GO(true, false);
  else if (!ak && bk) GO(false, true);
  else GO(false, false);
#undef GO
  if (rc != TF_OK) return rc;
  return launch_reduce<T>(st, p);
}

// One launch for a group of weight-gradient style products (both operands contraction-strided),
// 256x256 tiles, direct-to-LDS kernel; then one reduce pass per problem.
template <typename T>
static int gemm_group_dispatch(hipStream_t st, const GemmGroup& g) {
  constexpr int lds = 2 * (256 + 256) * 64 * 2;
  auto kernel = gemm_dma_group_kernel<T, 256, 256, 64, 2, 4, 2, false, false>;
  static bool once = (allow_big_lds(kernel, lds), true);
  (void)once;
  kernel<<<dim3((unsigned)g.first[g.count]), dim3(512), lds, st>>>(g);
  TF_CHECK_LAUNCH();
  g_gemm_launches.fetch_add(1, std::memory_order_relaxed);
  // second pass of the split contractions: all products of the group in one launch
  ReduceBatch rb = {};
  bool any = false, v4 = true;
  int64_t most = 0;
  for (int i = 0; i < g.count; ++i) {
    const GemmParams& p = g.p[i];
    rb.it[i] = {p.partial, p.C, p.ldc, p.chunk_skip, p.M, p.N, p.splits, p.chunk_n};
    if (p.splits <= 1) continue;
    any = true;
    v4 = v4 && p.N % 4 == 0 && p.ldc % 4 == 0 && p.chunk_n % 4 == 0 && p.chunk_skip % 4 == 0 &&
         (reinterpret_cast<uintptr_t>(p.C) & 15) == 0;
    const int64_t total = (int64_t)p.M * p.N;
    if (total > most) most = total;
  }
  if (!any) return TF_OK;
  int64_t blocks = ((v4 ? most / 4 : most) + 255) / 256;
  blocks = blocks > 4096 ? 4096 : (blocks < 1 ? 1 : blocks);
  const dim3 grid((unsigned)blocks, (unsigned)g.count), block(256);
  const bool f32 = g.p[0].out_f32 != 0;
  if (f32) { if (v4) gemm_reduce_group<float, true><<<grid, block, 0, st>>>(rb); else gemm_reduce_group<float, false><<<grid, block, 0, st>>>(rb); }
  else { if (v4) gemm_reduce_group<T, true><<<grid, block, 0, st>>>(rb); else gemm_reduce_group<T, false><<<grid, block, 0, st>>>(rb); }
  TF_CHECK_LAUNCH();
  return TF_OK;
}

}  // namespace tfa

using namespace tfa;

extern "C" int64_t tf_diag_gemm_launch_count(void) { return g_gemm_launches.load(std::memory_order_relaxed); }

// Tile columns (of 256x256 tiles) per whole number of rounds of workgroups, one per CU.
static int64_t round_unit(int64_t tiles_m, int64_t cus) {
  int64_t a = tiles_m, b = cus;
  while (b) { const int64_t t = a % b; a = b; b = t; }
  return cus / a;
}

// A product whose 256x256 tiles fill a whole number of rounds of workgroups plus a small
// remainder is cut in two along N: the columns that make whole rounds, and a narrow tail
// that runs as a split contraction on the otherwise idle CUs instead of a nearly empty last
// round (LM-head weight gradient: 4 x 197 tiles = 3 rounds + 20 tiles).  Returns the number
// of tail columns, 0 for no cut.
static int64_t tail_columns(int64_t M, int64_t N, int64_t K, bool vec, bool allow_split, const GemmForce& force) {
  if (!allow_split || force.cfg >= 0 || force.splits > 0 || K < 32 * 64 || (force.flags & 64)) return 0;
  const int64_t cus = device_shape().cus;
  double uncut;
  const GemmPlan pl = make_plan(M, N, K, vec, allow_split, &uncut);
  const int64_t tiles_m = (M + 255) / 256, tiles_n = (N + 255) / 256;
  const int64_t unit = round_unit(tiles_m, cus);
  const int64_t tn1 = (tiles_n / unit) * unit;
  if (tn1 <= 0 || tn1 * 256 >= N) return 0;
  if (pl.cfg == 2 && pl.splits == 1) {
    const int64_t tiles = tiles_m * tiles_n;
    const int64_t rem = tiles % cus;
    if (tiles > cus && rem != 0 && rem <= cus / 4) return N - tn1 * 256;
  }
  return 0;
}

// The same cut for a short contraction, by the cost model: whole rounds of 256x256 tiles, then
// the remaining columns as a product of their own with whatever tiling suits them, when the two
// together are cheaper than the best single launch (q/k/v projection 8192 x 3072 x 1024: one
// round of 256x256 tiles + 1024 columns of 128x128 tiles, 0.2 ms per training step less than
// three rounds of 128x128 tiles).
static int64_t round_cut_columns(int64_t M, int64_t N, int64_t K, bool vec, bool allow_split, const GemmForce& force,
                                 bool allow_cut) {
  if (!allow_cut || force.cfg >= 0 || force.splits > 0 || !(vec && K % 64 == 0) || (force.flags & 64)) return 0;
  const int64_t cus = device_shape().cus;
  double uncut, whole, rest;
  (void)make_plan(M, N, K, vec, allow_split, &uncut);
  if (uncut < 0) return 0;
  const int64_t tiles_m = (M + 255) / 256, tiles_n = (N + 255) / 256;
  if (tiles_m * tiles_n <= cus) return 0;
  const int64_t unit = round_unit(tiles_m, cus);
  const int64_t tn1 = (tiles_n / unit) * unit;
  if (tn1 <= 0 || tn1 * 256 >= N) return 0;
  (void)plan_for(2, M, tn1 * 256, K, &whole, false);
  (void)make_plan(M, N - tn1 * 256, K, vec, allow_split, &rest);
  if (rest < 0) return 0;
  return whole + rest + 3.0 < uncut ? N - tn1 * 256 : 0;
}

static int64_t single_need(int64_t M, int64_t N, int64_t K, bool vec) {
  const GemmPlan pl = make_plan(M, N, K, vec);
  return pl.splits > 1 ? (int64_t)pl.splits * M * N * (int64_t)sizeof(float) : 0;
}

extern "C" int64_t tf_gemm_workspace_bytes(int layout_a, int layout_b, int64_t M, int64_t N, int64_t K) {
  (void)layout_a;
  (void)layout_b;
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  // the caller's alignment is unknown here: cover both kernel families
  int64_t need = 0;
  for (int vec = 0; vec < 2; ++vec) {
    int64_t n = single_need(M, N, K, vec != 0);
    int64_t tail = tail_columns(M, N, K, vec != 0, true, kNoForce);
    if (tail == 0) tail = round_cut_columns(M, N, K, vec != 0, true, kNoForce, true);
    if (tail > 0) {
      const int64_t n1 = single_need(M, N - tail, K, vec != 0), n2 = single_need(M, tail, K, vec != 0);
      if (n1 > n) n = n1;
      if (n2 > n) n = n2;
    }
    if (n > need) need = n;
  }
  return need;
}

extern "C" int tf_gemm(void* stream, int dtype, int layout_a, int layout_b, int64_t M, int64_t N, int64_t K,
                       const void* A, int64_t lda, const void* B, int64_t ldb, void* C, int64_t ldc,
                       const void* bias, int relu, void* workspace, int64_t workspace_bytes) {
  return tf_gemm_out(stream, dtype, dtype, layout_a, layout_b, M, N, K, A, lda, B, ldb, C, ldc, bias, relu, nullptr, 0,
                     workspace, workspace_bytes);
}

extern "C" int tf_gemm_out(void* stream, int dtype, int out_dtype, int layout_a, int layout_b, int64_t M, int64_t N,
                           int64_t K, const void* A, int64_t lda, const void* B, int64_t ldb, void* C, int64_t ldc,
                           const void* bias, int relu, const void* mask_act, int64_t ld_mask, void* workspace,
                           int64_t workspace_bytes) {
  return tf_gemm_out_chunked(stream, dtype, out_dtype, layout_a, layout_b, M, N, K, A, lda, B, ldb, C, ldc, 0, 0, bias,
                             relu, mask_act, ld_mask, workspace, workspace_bytes);
}

static int gemm_entry(void* stream, int dtype, int out_dtype, int layout_a, int layout_b, int64_t M, int64_t N,
                      int64_t K, const void* A, int64_t lda, const void* B, int64_t ldb, void* C, int64_t ldc,
                      int64_t chunk_n, int64_t chunk_stride, const void* bias, int relu, const void* mask_act,
                      int64_t ld_mask, void* workspace, int64_t workspace_bytes, void* sign_out, const void* sign_in,
                      int64_t ld_sign, const GemmForce& force = kNoForce, const float* alpha = nullptr) {
  if (!A || !B || !C) return TF_EINVAL;
  if (alpha && (reinterpret_cast<uintptr_t>(alpha) & 3)) return TF_EALIGN;
  const bool signs = sign_out || sign_in;
  if (signs) {
    if ((sign_out && sign_in) || mask_act || N % 8 != 0 || ld_sign < N / 8 || (chunk_n != 0 && chunk_n < N)) return TF_EINVAL;
    if (sign_out && (!relu || out_dtype != dtype)) return TF_EINVAL;
    if (sign_in && (bias || relu)) return TF_EINVAL;
  }
  if (chunk_n < 0 || chunk_stride < 0) return TF_EINVAL;
  if (mask_act && (bias || relu || ld_mask < N)) return TF_EINVAL;
  if (out_dtype != dtype && out_dtype != TF_F32) return TF_EDTYPE;
  if (M <= 0 || N <= 0 || K <= 0 || M > 0x7fffff00 || N > 0x7fffff00 || K > 0x7fffff00) return TF_EINVAL;
  if (chunk_n == 0 || chunk_n >= N) { chunk_n = N; chunk_stride = N; }
  else if (N % chunk_n != 0 || chunk_n % 8 != 0 || chunk_stride % 8 != 0 ||
           chunk_stride < (M - 1) * ldc + chunk_n) return TF_ESHAPE;
  if ((layout_a != TF_OP_KMAJOR && layout_a != TF_OP_KMINOR) || (layout_b != TF_OP_KMAJOR && layout_b != TF_OP_KMINOR))
    return TF_EINVAL;
  if (dtype != TF_F16 && dtype != TF_BF16) return TF_EDTYPE;
  const int64_t a_contig = layout_a == TF_OP_KMAJOR ? K : M;
  const int64_t b_contig = layout_b == TF_OP_KMAJOR ? K : N;
  if (lda < a_contig || ldb < b_contig || ldc < chunk_n) return TF_ESHAPE;
  if ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B) | reinterpret_cast<uintptr_t>(C) |
       reinterpret_cast<uintptr_t>(bias)) & 1)
    return TF_EALIGN;

  const bool vec = aligned16(A) && aligned16(B) && aligned16(C) && (!bias || aligned16(bias)) && a_contig % 8 == 0 &&
                   b_contig % 8 == 0 && lda % 8 == 0 && ldb % 8 == 0 && N % 8 == 0 && ldc % 8 == 0 &&
                   (!mask_act || (aligned16(mask_act) && ld_mask % 8 == 0));
  if (chunk_n == N) {
    // (a launch with sign bits takes no split contraction: its cut is the one into unsplit products, and only
    // where the bits of both parts are served -- a cut at a multiple of 256 columns keeps whole bytes and the
    // 16-byte pieces of the bit rows)
    const bool may_split = mask_act == nullptr && !signs;
    int64_t tail = signs ? 0 : tail_columns(M, N, K, vec, may_split, force);
    if (tail == 0) tail = round_cut_columns(M, N, K, vec, may_split, force, mask_act == nullptr);
    if (tail > 0 && signs) {
      const GemmPlan p1 = make_plan(M, N - tail, K, vec, false, nullptr, force), p2 = make_plan(M, tail, K, vec, false, nullptr, force);
      if (!(kCfgs[p1.cfg].dma && kCfgs[p2.cfg].dma && K % p1.bk == 0 && K % p2.bk == 0)) tail = 0;
    }
    if (tail > 0) {  // whole rounds first, then the narrow remainder as a split contraction
      const int64_t n1 = N - tail;
      const int64_t osz = out_dtype == TF_F32 ? 4 : 2;
      const char* b2 = (const char*)B + (layout_b == TF_OP_KMAJOR ? n1 * ldb : n1) * 2;
      const void* bias2 = bias ? (const char*)bias + n1 * 2 : nullptr;
      const void* mask2 = mask_act ? (const char*)mask_act + n1 * 2 : nullptr;
      void* so2 = sign_out ? (char*)sign_out + n1 / 8 : nullptr;
      const void* si2 = sign_in ? (const char*)sign_in + n1 / 8 : nullptr;
      const int rc = gemm_entry(stream, dtype, out_dtype, layout_a, layout_b, M, n1, K, A, lda, B, ldb, C, ldc, 0, 0, bias,
                                relu, mask_act, ld_mask, workspace, workspace_bytes, sign_out, sign_in, ld_sign, force, alpha);
      if (rc != TF_OK) return rc;
      return gemm_entry(stream, dtype, out_dtype, layout_a, layout_b, M, tail, K, A, lda, b2, ldb, (char*)C + n1 * osz,
                        ldc, 0, 0, bias2, relu, mask2, ld_mask, workspace, workspace_bytes, so2, si2, ld_sign, force,
                        alpha);
    }
  }
  const GemmPlan pl = make_plan(M, N, K, vec, mask_act == nullptr && !signs, nullptr, force);
  // the sign bits exist in the write-out of the direct-to-LDS kernels only
  // (TF_ESHAPE, so that a caller can tell "this product is not served, use the activation as mask"
  // from a malformed call)
  if (signs && !(kCfgs[pl.cfg].dma && vec && K % pl.bk == 0 && pl.splits == 1)) return TF_ESHAPE;
  const int64_t need = pl.splits > 1 ? (int64_t)pl.splits * M * N * (int64_t)sizeof(float) : 0;
  if (need > 0 && (!workspace || workspace_bytes < need)) return TF_EWORKSPACE;
  if (need > 0 && !aligned16(workspace)) return TF_EALIGN;
  if ((int64_t)pl.tiles_m * pl.tiles_n * pl.splits > 0x7fffffff) return TF_EINVAL;

  GemmParams p;
  p.A = A; p.B = B; p.C = C; p.bias = bias; p.partial = (float*)workspace;
  p.M = (int)M; p.N = (int)N; p.K = (int)K;
  p.lda = lda; p.ldb = ldb; p.ldc = ldc;
  p.relu = relu ? 1 : 0;
  p.splits = pl.splits; p.k_per_split = pl.k_per_split;
  p.tiles_m = pl.tiles_m; p.tiles_n = pl.tiles_n;
  p.flags = force.flags;
  p.xcds = device_shape().xcds;
  p.out_f32 = out_dtype == TF_F32 ? 1 : 0;
  p.mask = mask_act;
  p.ldmask = ld_mask;
  p.sign_out = sign_out;
  p.sign_in = sign_in;
  p.ldsign = ld_sign;
  p.chunk_n = (int)chunk_n;
  p.chunk_skip = chunk_stride - chunk_n;
  p.alpha = alpha;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == TF_F16) return gemm_dispatch<f16>(st, layout_a, layout_b, vec, pl, p);
  return gemm_dispatch<bf16>(st, layout_a, layout_b, vec, pl, p);
}

extern "C" int tf_gemm_out_chunked(void* stream, int dtype, int out_dtype, int layout_a, int layout_b, int64_t M,
                                   int64_t N, int64_t K, const void* A, int64_t lda, const void* B, int64_t ldb,
                                   void* C, int64_t ldc, int64_t chunk_n, int64_t chunk_stride, const void* bias,
                                   int relu, const void* mask_act, int64_t ld_mask, void* workspace,
                                   int64_t workspace_bytes) {
  return gemm_entry(stream, dtype, out_dtype, layout_a, layout_b, M, N, K, A, lda, B, ldb, C, ldc, chunk_n,
                    chunk_stride, bias, relu, mask_act, ld_mask, workspace, workspace_bytes, nullptr, nullptr, 0);
}

extern "C" int tf_gemm_relu_bits(void* stream, int dtype, int out_dtype, int layout_a, int layout_b, int64_t M,
                                 int64_t N, int64_t K, const void* A, int64_t lda, const void* B, int64_t ldb,
                                 void* C, int64_t ldc, const void* bias, void* bits_out, const void* bits_in,
                                 int64_t ld_bits) {
  if (!bits_out && !bits_in) return TF_EINVAL;
  return gemm_entry(stream, dtype, out_dtype, layout_a, layout_b, M, N, K, A, lda, B, ldb, C, ldc, 0, 0, bias,
                    bits_out ? 1 : 0, nullptr, 0, nullptr, 0, bits_out, bits_in, ld_bits);
}

extern "C" int tf_gemm_scaled(void* stream, int dtype, int out_dtype, int layout_a, int layout_b, int64_t M, int64_t N,
                              int64_t K, const void* A, int64_t lda, const void* B, int64_t ldb, void* C, int64_t ldc,
                              const float* alpha, void* workspace, int64_t workspace_bytes) {
  if (!alpha) return TF_EINVAL;
  return gemm_entry(stream, dtype, out_dtype, layout_a, layout_b, M, N, K, A, lda, B, ldb, C, ldc, 0, 0, nullptr, 0,
                    nullptr, 0, workspace, workspace_bytes, nullptr, nullptr, 0, kNoForce, alpha);
}

// Diagnostic twin of tf_gemm_out_chunked: the same call with a tile configuration, a contraction
// split and flag bits imposed on THIS call only (no state is kept).
extern "C" int tf_diag_gemm(void* stream, int cfg, int splits, int flags, int dtype, int out_dtype, int layout_a,
                            int layout_b, int64_t M, int64_t N, int64_t K, const void* A, int64_t lda, const void* B,
                            int64_t ldb, void* C, int64_t ldc, const void* bias, int relu, void* workspace,
                            int64_t workspace_bytes) {
  if (cfg >= kNumCfgs || splits < 0 || (flags & ~(1 | 64))) return TF_EINVAL;
  const GemmForce force = {cfg < 0 ? -1 : cfg, splits, flags};
  return gemm_entry(stream, dtype, out_dtype, layout_a, layout_b, M, N, K, A, lda, B, ldb, C, ldc, 0, 0, bias, relu,
                    nullptr, 0, workspace, workspace_bytes, nullptr, nullptr, 0, force);
}
extern "C" int64_t tf_diag_gemm_workspace_bytes(int cfg, int splits, int64_t M, int64_t N, int64_t K) {
  if (M <= 0 || N <= 0 || K <= 0 || cfg >= kNumCfgs) return 0;
  if (cfg < 0 && splits <= 0) return tf_gemm_workspace_bytes(0, 0, M, N, K);
  const GemmForce force = {cfg < 0 ? -1 : cfg, splits, 0};
  int64_t need = 0;
  for (int vec = 0; vec < 2; ++vec) {
    const GemmPlan pl = make_plan(M, N, K, vec != 0, true, nullptr, force);
    const int64_t n = pl.splits > 1 ? (int64_t)pl.splits * M * N * (int64_t)sizeof(float) : 0;
    if (n > need) need = n;
  }
  return need;
}

// ---- grouped products -------------------------------------------------------
namespace {

struct GroupPlan {
  bool grouped;   // one launch for all problems (otherwise: one tf_gemm_out_chunked call each)
  int splits;
  int64_t need;   // workspace bytes
  // Tiles that make whole rounds of workgroups plus a remainder: the last `cut_cols` tile columns of problem
  // `cut_problem` (-1: none) become a member of the group of their own whose contraction is cut into
  // `tail_splits` slices, so that the remainder fills one short round of all CUs instead of a whole round of
  // a few (what the N-cut of a single product does for the LM-head weight gradient).
  int cut_problem;
  int cut_cols;
  int tail_splits;
};

bool group_problem_ok(const tf_gemm_problem& q) {
  return q.A && q.B && q.C && q.M > 0 && q.N > 0 && q.K > 0 && q.M <= 0x7fffff00 && q.N <= 0x7fffff00 &&
         q.K <= 0x7fffff00;
}

// Fast-path preconditions of the direct-to-LDS kernel for a (K-minor, K-minor) problem.
bool group_problem_fast(const tf_gemm_problem& q) {
  const int64_t cn = (q.chunk_n <= 0 || q.chunk_n >= q.N) ? q.N : q.chunk_n;
  return aligned16(q.A) && aligned16(q.B) && aligned16(q.C) && q.M % 8 == 0 && q.N % 8 == 0 && q.lda % 8 == 0 &&
         q.ldb % 8 == 0 && q.ldc % 8 == 0 && q.K % 64 == 0 && q.lda >= q.M && q.ldb >= q.N && q.ldc >= cn &&
         q.N % cn == 0 && cn % 8 == 0 && (cn == q.N || (q.chunk_stride % 8 == 0 && q.chunk_stride >= (q.M - 1) * q.ldc + cn));
}

GroupPlan plan_group(int la, int lb, int count, const tf_gemm_problem* pr) {
  GroupPlan gp = {false, 1, 0, -1, 0, 1};
  bool fast = count >= 2 && count <= kMaxGroup && la == TF_OP_KMINOR && lb == TF_OP_KMINOR;
  const int64_t cus = device_shape().cus;
  int64_t tiles = 0, min_ksteps = INT64_MAX;
  for (int i = 0; i < count && fast; ++i) {
    fast = group_problem_ok(pr[i]) && group_problem_fast(pr[i]);
    if (!fast) break;
    tiles += ((pr[i].M + 255) / 256) * ((pr[i].N + 255) / 256);
    const int64_t ks = pr[i].K / 64;
    if (ks < min_ksteps) min_ksteps = ks;
  }
  if (fast && tiles < 0x7fffff) {
    // same rule as for a single product: split only when the tiles alone leave most CUs idle,
    // never beyond one round of workgroups, slices of at least 16 steps
    int64_t splits = 1;
    if (tiles <= cus / 2) {
      splits = cus / tiles;
      const int64_t max_by_k = min_ksteps / 16 > 0 ? min_ksteps / 16 : 1;
      if (splits > max_by_k) splits = max_by_k;
      if (splits > 16) splits = 16;
    }
    gp.grouped = true;
    gp.splits = (int)splits;
    if (splits > 1)
      for (int i = 0; i < count; ++i) gp.need += splits * pr[i].M * pr[i].N * (int64_t)sizeof(float);
    // More tiles than CUs and a remainder: look for a cut.  Costs in 64-wide contraction steps of a round of
    // workgroups; the split tail pays its fp32 partials and the reduce pass (about six steps' worth).
    bool same_k = true;
    for (int i = 1; i < count; ++i) same_k = same_k && pr[i].K == pr[0].K;
#ifdef TF_NO_GROUP_CUT
    same_k = false;
#endif
    if (splits == 1 && tiles > cus && tiles % cus != 0 && same_k && count < kMaxGroup) {
      const int64_t ksteps = pr[0].K / 64;
      const int64_t rounds_whole = tiles / cus;
      int64_t best = ((tiles + cus - 1) / cus) * ksteps * 9 / 10;  // a cut must win by a tenth
      for (int i = 0; i < count; ++i) {
        const bool unchunked = pr[i].chunk_n <= 0 || pr[i].chunk_n >= pr[i].N;
        if (!unchunked || pr[i].M % 256 || pr[i].N % 256) continue;
        const int64_t tm = pr[i].M / 256, tn = pr[i].N / 256;
        for (int64_t c = 1; c < tn; ++c) {
          const int64_t tail = c * tm;
          if (tiles - tail > rounds_whole * cus) continue;  // the whole tiles must fit the whole rounds
          int64_t s = cus / tail;
          if (s > ksteps / 8) s = ksteps / 8;               // slices of at least 8 steps
          if (s > 16) s = 16;
          if (s < 2) break;
          const int64_t per = (ksteps + s - 1) / s;
          const int64_t cost = rounds_whole * ksteps + per + 6;
          if (cost < best) {
            best = cost;
            gp.cut_problem = i;
            gp.cut_cols = (int)c;
            gp.tail_splits = (int)((ksteps + per - 1) / per);
          }
        }
      }
      if (gp.cut_problem >= 0)
        gp.need = (int64_t)gp.tail_splits * pr[gp.cut_problem].M * gp.cut_cols * 256 * (int64_t)sizeof(float);
    }
    return gp;
  }
  for (int i = 0; i < count; ++i) {
    if (!group_problem_ok(pr[i])) continue;
    const int64_t n = tf_gemm_workspace_bytes(la, lb, pr[i].M, pr[i].N, pr[i].K);
    if (n > gp.need) gp.need = n;
  }
  return gp;
}

}  // namespace

extern "C" int64_t tf_gemm_group_workspace_bytes(int layout_a, int layout_b, int count, const tf_gemm_problem* problems) {
  if (!problems || count < 1 || count > kMaxGroup) return 0;
  return plan_group(layout_a, layout_b, count, problems).need;
}

extern "C" int tf_gemm_group(void* stream, int dtype, int out_dtype, int layout_a, int layout_b, int count,
                             const tf_gemm_problem* problems, void* workspace, int64_t workspace_bytes) {
  if (!problems || count < 1 || count > kMaxGroup) return TF_EINVAL;
  if (dtype != TF_F16 && dtype != TF_BF16) return TF_EDTYPE;
  if (out_dtype != dtype && out_dtype != TF_F32) return TF_EDTYPE;
  const GroupPlan gp = plan_group(layout_a, layout_b, count, problems);
  if (gp.need > 0 && (!workspace || workspace_bytes < gp.need)) return TF_EWORKSPACE;
  if (!gp.grouped) {
    for (int i = 0; i < count; ++i) {
      const tf_gemm_problem& q = problems[i];
      const int rc = tf_gemm_out_chunked(stream, dtype, out_dtype, layout_a, layout_b, q.M, q.N, q.K, q.A, q.lda, q.B,
                                         q.ldb, q.C, q.ldc, q.chunk_n, q.chunk_stride, nullptr, 0, nullptr, 0,
                                         workspace, workspace_bytes);
      if (rc != TF_OK) return rc;
    }
    return TF_OK;
  }
  if (gp.need > 0 && !aligned16(workspace)) return TF_EALIGN;
  // members of the launch: the problems as given, except that a cut problem keeps its leading columns and a
  // further member takes its last tile columns with a split contraction
  tf_gemm_problem mem[kMaxGroup];
  int mem_splits[kMaxGroup];
  int members = 0;
  for (int i = 0; i < count; ++i) {
    mem[members] = problems[i];
    mem_splits[members] = gp.splits;
    if (i == gp.cut_problem) mem[members].N -= (int64_t)gp.cut_cols * 256;
    ++members;
  }
  if (gp.cut_problem >= 0) {
    const tf_gemm_problem& q = problems[gp.cut_problem];
    const int64_t n1 = q.N - (int64_t)gp.cut_cols * 256;
    const int64_t osz = out_dtype == TF_F32 ? 4 : 2;
    tf_gemm_problem t = q;
    t.N = q.N - n1;
    t.B = (const char*)q.B + n1 * 2;  // (K, N) row-major: the columns from n1 on
    t.C = (char*)q.C + n1 * osz;
    t.chunk_n = 0;
    t.chunk_stride = 0;
    mem[gp.cut_problem].chunk_n = 0;  // (only unchunked problems are cut)
    mem[gp.cut_problem].chunk_stride = 0;
    mem[members] = t;
    mem_splits[members] = gp.tail_splits;
    ++members;
  }
  GemmGroup g;
  g.count = members;
  g.first[0] = 0;
  char* ws = (char*)workspace;
  for (int i = 0; i < kMaxGroup; ++i) {
    const tf_gemm_problem& q = mem[i < members ? i : 0];
    const int want = mem_splits[i < members ? i : 0];
    GemmParams& p = g.p[i];
    const int64_t cn = (q.chunk_n <= 0 || q.chunk_n >= q.N) ? q.N : q.chunk_n;
    p.A = q.A; p.B = q.B; p.C = q.C; p.bias = nullptr; p.partial = (float*)ws;
    p.M = (int)q.M; p.N = (int)q.N; p.K = (int)q.K;
    p.lda = q.lda; p.ldb = q.ldb; p.ldc = q.ldc;
    p.relu = 0;
    p.tiles_m = (int)((q.M + 255) / 256); p.tiles_n = (int)((q.N + 255) / 256);
    const int64_t ksteps = q.K / 64;
    const int64_t steps_per = (ksteps + want - 1) / want;
    p.k_per_split = (int)(steps_per * 64);
    p.splits = (int)((ksteps + steps_per - 1) / steps_per);
    p.flags = gp.cut_problem >= 0 ? 1 : 0;
    p.xcds = device_shape().xcds;
    p.out_f32 = out_dtype == TF_F32 ? 1 : 0;
    p.mask = nullptr; p.ldmask = 0;
    p.sign_out = nullptr; p.sign_in = nullptr; p.ldsign = 0;
    p.chunk_n = (int)cn;
    p.chunk_skip = (cn == q.N ? q.N : q.chunk_stride) - cn;
    p.alpha = nullptr;
    if (i < members) {
      g.first[i + 1] = g.first[i] + p.tiles_m * p.tiles_n * p.splits;
      if (p.splits > 1) ws += (int64_t)want * q.M * q.N * (int64_t)sizeof(float);
    }
  }
  hipStream_t st = (hipStream_t)stream;
  if (dtype == TF_F16) return gemm_group_dispatch<f16>(st, g);
  return gemm_group_dispatch<bf16>(st, g);
}
