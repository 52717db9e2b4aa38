// Dense contraction C[M,N] = epilogue(sum_k A(m,k) B(n,k)) on gfx950 MFMA.
//
// One workgroup owns a BM x BN tile of C.  Per BK-wide step of the contraction
// the A and B panels are brought HBM -> registers -> LDS with 16-byte accesses
// (the next step's loads are in flight while the current step computes, LDS is
// double buffered, one barrier per step) and consumed by
// v_mfma_f32_32x32x16_{f16,bf16} with fp32 accumulators.
//
// Either operand may be stored with the contraction dimension contiguous
// ("K-major": read from LDS with ds_read_b128) or strided ("K-minor": read with
// the gfx950 transposing ds_read_b64_tr_b16), so X.W, dY.W^T and X^T.dY all run
// from the tensors as PyTorch holds them, without transposed copies.  LDS
// tiles are XOR-swizzled at 16-byte granularity to keep both access patterns
// free of bank conflicts.
//
// The MFMA is issued as D^T = B_frag x A_frag, so a lane ends up holding four
// consecutive n for one m: the epilogue (bias, ReLU, rounding) stores 8 bytes
// per lane and needs no cross-lane traffic.
//
// Workgroup ids are remapped so that each of the 8 XCDs (which receive ids
// round-robin) works on a compact block of neighbouring tiles and shares the
// A/B panels through its own L2.
#include <cstdlib>
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
};

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
    if (KMAJOR) return c ^ ((lrow / (16 / CPR)) % CPR);
    return c ^ ((lrow & 3) << 2);
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
__device__ __forceinline__ int remap_xcd(int pid, int n) {
  constexpr int X = 8;
  const int xcd = pid % X, local = pid / X;
  const int q = n / X, r = n % X;
  return xcd * q + (xcd < r ? xcd : r) + local;
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
  const int pid = remap_xcd(blockIdx.x, tiles * p.splits);
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

  // ---- epilogue: lane holds C[m][n .. n+3] for m = .. + lane%32 ------------
  const T* bias = (const T*)p.bias;
  T* C = (T*)p.C;
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
        for (int e = 0; e < 4; ++e) v[e] = acc[i][j][g * 4 + e];
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
          if (VEC) {
            typename Vec<T>::v4 o;
            if (bias) {
              const typename Vec<T>::v4 bv = *reinterpret_cast<const typename Vec<T>::v4*>(bias + n);
#pragma unroll
              for (int e = 0; e < 4; ++e) v[e] += (float)bv[e];
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = (T)(p.relu ? fmaxf(v[e], 0.f) : v[e]);
            *reinterpret_cast<typename Vec<T>::v4*>(C + (int64_t)m * p.ldc + n) = o;
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              if (n + e < p.N) {
                float x = v[e] + (bias ? (float)bias[n + e] : 0.f);
                C[(int64_t)m * p.ldc + n + e] = (T)(p.relu ? fmaxf(x, 0.f) : x);
              }
            }
          }
        }
      }
    }
  }
}

// Sum the split-contraction partials in a fixed order and apply the epilogue.
template <typename T>
__global__ __launch_bounds__(256) void gemm_reduce(int M, int N, int splits, const float* __restrict__ partial,
                                                    const T* __restrict__ bias, int relu, T* __restrict__ C,
                                                    int64_t ldc) {
  const int64_t total = (int64_t)M * N;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    float s = 0.f;
    for (int k = 0; k < splits; ++k) s += partial[(int64_t)k * total + i];
    const int m = (int)(i / N), n = (int)(i - (int64_t)m * N);
    if (bias) s += (float)bias[n];
    C[(int64_t)m * ldc + n] = (T)(relu ? fmaxf(s, 0.f) : s);
  }
}

// ---------------------------------------------------------------------------
// host side: tile choice, contraction split, launch
// ---------------------------------------------------------------------------
struct GemmPlan {
  int cfg;  // 0: 256x256x64 / 8 waves, 1: 128x128x64 / 4 waves
  int bm, bn, bk;
  int tiles_m, tiles_n, splits, k_per_split;
};

static int env_int(const char* name, int dflt) {
  const char* s = getenv(name);
  return s ? atoi(s) : dflt;
}

static GemmPlan make_plan(int64_t M, int64_t N, int64_t K) {
  static const int force_cfg = env_int("TF_GEMM_CFG", -1);
  static const int force_splits = env_int("TF_GEMM_SPLITS", 0);
  GemmPlan pl;
  const int64_t big_tiles = ((M + 255) / 256) * ((N + 255) / 256);
  pl.cfg = big_tiles >= 192 ? 0 : 1;
  if (force_cfg >= 0 && force_cfg <= 1) pl.cfg = force_cfg;
  pl.bm = pl.bn = pl.cfg == 0 ? 256 : 128;
  pl.bk = 64;
  pl.tiles_m = (int)((M + pl.bm - 1) / pl.bm);
  pl.tiles_n = (int)((N + pl.bn - 1) / pl.bn);
  const int64_t tiles = (int64_t)pl.tiles_m * pl.tiles_n;
  const int64_t ksteps = (K + pl.bk - 1) / pl.bk;
  // Split the contraction only when the tile count alone cannot fill 256 CUs
  // and each slice still keeps at least 8 steps of work.
  int64_t splits = 1;
  const int64_t target = pl.cfg == 0 ? 256 : 512;
  if (tiles < target) {
    splits = (target + tiles - 1) / tiles;
    const int64_t max_by_k = ksteps / 8 > 0 ? ksteps / 8 : 1;
    if (splits > max_by_k) splits = max_by_k;
    if (splits > 32) splits = 32;
  }
  if (force_splits > 0) splits = force_splits;
  if (splits > ksteps) splits = ksteps > 0 ? ksteps : 1;
  const int64_t steps_per = (ksteps + splits - 1) / splits;
  pl.k_per_split = (int)(steps_per * pl.bk);
  pl.splits = (int)((ksteps + steps_per - 1) / steps_per);
  if (pl.splits < 1) pl.splits = 1;
  return pl;
}

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
  return TF_OK;
}

template <typename T, bool AK, bool BKM, bool VEC>
static int launch_cfg(hipStream_t st, const GemmPlan& pl, const GemmParams& p) {
  if (pl.cfg == 0) return launch_one<T, 256, 256, 64, 2, 4, AK, BKM, VEC>(st, p);
  return launch_one<T, 128, 128, 64, 2, 2, AK, BKM, VEC>(st, p);
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
  if (p.splits > 1) {
    const int64_t total = (int64_t)p.M * p.N;
    int64_t blocks = (total + 255) / 256;
    if (blocks > 8192) blocks = 8192;
    gemm_reduce<T><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(p.M, p.N, p.splits, p.partial, (const T*)p.bias,
                                                                 p.relu, (T*)p.C, p.ldc);
    TF_CHECK_LAUNCH();
  }
  return TF_OK;
}

}  // namespace tfa

using namespace tfa;

extern "C" int64_t tf_gemm_workspace_bytes(int layout_a, int layout_b, int64_t M, int64_t N, int64_t K) {
  (void)layout_a;
  (void)layout_b;
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  const GemmPlan pl = make_plan(M, N, K);
  return pl.splits > 1 ? (int64_t)pl.splits * M * N * (int64_t)sizeof(float) : 0;
}

extern "C" int tf_gemm(void* stream, int dtype, int layout_a, int layout_b, int64_t M, int64_t N, int64_t K,
                       const void* A, int64_t lda, const void* B, int64_t ldb, void* C, int64_t ldc,
                       const void* bias, int relu, void* workspace, int64_t workspace_bytes) {
  if (!A || !B || !C) return TF_EINVAL;
  if (M <= 0 || N <= 0 || K <= 0 || M > 0x7fffff00 || N > 0x7fffff00 || K > 0x7fffff00) return TF_EINVAL;
  if ((layout_a != TF_OP_KMAJOR && layout_a != TF_OP_KMINOR) || (layout_b != TF_OP_KMAJOR && layout_b != TF_OP_KMINOR))
    return TF_EINVAL;
  if (dtype != TF_F16 && dtype != TF_BF16) return TF_EDTYPE;
  const int64_t a_contig = layout_a == TF_OP_KMAJOR ? K : M;
  const int64_t b_contig = layout_b == TF_OP_KMAJOR ? K : N;
  if (lda < a_contig || ldb < b_contig || ldc < N) return TF_ESHAPE;
  if ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B) | reinterpret_cast<uintptr_t>(C) |
       reinterpret_cast<uintptr_t>(bias)) & 1)
    return TF_EALIGN;

  const GemmPlan pl = make_plan(M, N, K);
  const int64_t need = pl.splits > 1 ? (int64_t)pl.splits * M * N * (int64_t)sizeof(float) : 0;
  if (need > 0 && (!workspace || workspace_bytes < need)) return TF_EWORKSPACE;
  if (need > 0 && !aligned16(workspace)) return TF_EALIGN;
  if ((int64_t)pl.tiles_m * pl.tiles_n * pl.splits > 0x7fffffff) return TF_EINVAL;

  const bool vec = aligned16(A) && aligned16(B) && aligned16(C) && (!bias || aligned16(bias)) && a_contig % 8 == 0 &&
                   b_contig % 8 == 0 && lda % 8 == 0 && ldb % 8 == 0 && N % 8 == 0 && ldc % 8 == 0;

  GemmParams p;
  p.A = A; p.B = B; p.C = C; p.bias = bias; p.partial = (float*)workspace;
  p.M = (int)M; p.N = (int)N; p.K = (int)K;
  p.lda = lda; p.ldb = ldb; p.ldc = ldc;
  p.relu = relu ? 1 : 0;
  p.splits = pl.splits; p.k_per_split = pl.k_per_split;
  p.tiles_m = pl.tiles_m; p.tiles_n = pl.tiles_n;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == TF_F16) return gemm_dispatch<f16>(st, layout_a, layout_b, vec, pl, p);
  return gemm_dispatch<bf16>(st, layout_a, layout_b, vec, pl, p);
}
