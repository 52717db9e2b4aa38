// Causal flash attention forward / backward on gfx950 MFMA, optional additive
// bias (ALiBi).  FlashAttention-2 schedule: the forward and the dQ pass are
// partitioned over query blocks with a loop over key/value blocks up to the
// diagonal; the dK/dV pass is partitioned over key/value blocks with a loop
// over the query blocks at or below the diagonal.  No atomics: results are
// bitwise reproducible.
//
// Layout trick used by all three kernels: score tiles are produced
// TRANSPOSED with respect to the operand that stays in registers, i.e. the
// 32x32 MFMA output has the register-resident index (query in the forward and
// dQ passes, key in the dK/dV pass) along lanes.  Then
//   * per-row softmax statistics are per-lane scalars (one cross-lane op to
//     merge the two half-waves),
//   * the fp32 tile, rounded to 16 bit, already IS the k-contiguous MFMA
//     operand of the second contraction: no LDS round trip for P / dS,
//   * the other operand of the second contraction (V, dO, Q or K, stored
//     row-major [seq][hd] in LDS) is fetched with the transposing
//     ds_read_b64_tr_b16.
// The 16 contraction slots of lane-half h in step t map to sequence offsets
// 16t + 8(s/4) + 4h + s%4 (s = 0..7), on both operands alike.
#include <type_traits>
#include "rowops.h"

namespace tfa {

typedef __attribute__((address_space(1))) const void gptr_void;

struct AttnParams {
  const void *q, *k, *v, *o, *d_o;
  void *out, *dq, *dk, *dv;
  float* lse;    // written by fwd, read by bwd
  float* delta;  // -rowsum(dO * O): written by the dQ pass, read by the dK/dV pass
  const void* bias;
  const void* slopes;         // ALiBi in closed form: nh fp16 slopes instead of a dense bias
  int64_t sb, sh, ss;         // element strides of q, k, v and of dq, dk, dv
  int64_t osb, osh, oss;      // element strides of o and dO
  int64_t bias_sh, bias_sr;   // element strides of bias (head, query row)
  int B, nh, S;
  float scale_log2;           // scale * log2(e)
  float scale;
};

// ---------------------------------------------------------------------------
// LDS tile [ROWS][HD] of 16-bit elements, hd contiguous, chunk-swizzled so that
// both the row-wise 16-byte reads and the transposing 8-byte reads are free of
// bank conflicts.
// ---------------------------------------------------------------------------
template <typename T, int ROWS, int HD>
struct SeqTile {
  static constexpr int CPR = HD / 8;
  static constexpr int BYTES = ROWS * HD * 2;
  static constexpr int PER_THREAD = (ROWS * CPR + 255) / 256;
  typedef typename Vec<T>::v8 v8;

  static __device__ __forceinline__ int swz(int row) {
    if (CPR == 4) return (row >> 2) & 3;
    if (CPR == 8) { const int u = (row >> 1) & 7; return ((u & 1) << 2) | (u >> 1); }
    return ((row & 3) << 2) | ((row >> 2) & 3);
  }
  static __device__ __forceinline__ int addr(int row, int chunk) { return (row * CPR + (chunk ^ swz(row))) * 16; }

  // Direct-to-LDS loads: thread t's j-th 16-byte load lands in LDS slot t + 256 j of the tile,
  // so the chunk swizzle is applied to the global address.  ptr[j] = address of that chunk in
  // the tile whose first row is row0 of a (seq, hd) matrix with row stride ss.
  static __device__ __forceinline__ void stream_init(const T* (&ptr)[PER_THREAD], const T* base, int64_t ss, int row0) {
#pragma unroll
    for (int j = 0; j < PER_THREAD; ++j) {
      const int id = threadIdx.x + j * 256;
      const int row = id / CPR, c = (id % CPR) ^ swz(row);
      ptr[j] = base + (int64_t)(row0 + row) * ss + c * 8;
    }
  }
  // A sequence may end half way through a 64-row block (S = 32 mod 64).  Before the loads of that last
  // block, the pointers of its rows 32 .. 63 -- which lie beyond the sequence, possibly beyond the
  // allocation -- are moved 32 rows back: the tile then holds rows 0 .. 31 twice.  No valid query ever
  // sees the copies (keys beyond the sequence lie above every diagonal; queries beyond it are skipped),
  // they only have to be readable and finite.
  static __device__ __forceinline__ void stream_tail(const T* (&ptr)[PER_THREAD], int64_t ss) {
#pragma unroll
    for (int j = 0; j < PER_THREAD; ++j)
      if ((int)threadIdx.x + j * 256 >= 32 * CPR) ptr[j] -= 32 * ss;
  }
  // LDS destination of a wave's j-th load into the tile at `tile`
  static __device__ __forceinline__ char* stream_slot(char* tile, int wave, int j) {
    return tile + (j * 256 + wave * 64) * 16;
  }
  // Lane-dependent parts of the LDS operand addresses of the tile at LDS address `tile`; block,
  // sub-tile and stage offsets are compile-time constants that go into the offset fields.
  static __device__ __forceinline__ void operand_addrs(uint32_t (&rows)[HD / 16], uint32_t (&hd)[HD / 32][2],
                                                       uint32_t tile, int lane) {
#pragma unroll
    for (int ks = 0; ks < HD / 16; ++ks) rows[ks] = tile + addr(lane & 31, ks * 2 + (lane >> 5));
#pragma unroll
    for (int d = 0; d < HD / 32; ++d) {
      const int i = lane & 15;
      const int col = d * 32 + 16 * ((lane >> 4) & 1) + (i & 3) * 4;
      const int r0 = 4 * (lane >> 5) + (i >> 2);
      hd[d][0] = tile + addr(r0, col >> 3) + (col & 7) * 2;
      hd[d][1] = tile + addr(r0 + 8, col >> 3) + (col & 7) * 2;
    }
  }

  // Operands read from a tile (the kernels issue the reads themselves, see below):
  //  * rows as the MFMA row/col index: lane l reads 16 bytes at addr(rb + l%32, ks*2 + l/32),
  //    i.e. (row rb + l%32, hd = ks*16 + (l/32)*8 + 0..7);
  //  * hd as the MFMA row/col index, rows as the contraction: two transposing 8-byte reads at
  //    addr(r0, col/8) + (col%8)*2 and the same 8 rows further down, with
  //    col = dt*32 + 16*((l/16)%2) + (l%4)*4 and r0 = rb16 + 4*(l/32) + (l%16)/4; lane l ends up
  //    with (hd = dt*32 + l%32, rows rb16 + 8*(s/4) + 4*(l/32) + s%4), s = 0..7.
};

template <typename T> __device__ __forceinline__ typename Vec<T>::v8 round8(const f32x16& x, int t) {
  typename Vec<T>::v8 r;
#pragma unroll
  for (int s = 0; s < 8; ++s) r[s] = (T)x[t * 8 + s];
  return r;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// max(x, x of lane l ^ 32) through the VALU (v_permlane32_swap) rather than the LDS crossbar:
// swapping the upper half of one copy of x with the lower half of another leaves, in every
// lane, its own value in one register and its partner's in the other.
__device__ __forceinline__ float max_with_other_half(float x) {
  const unsigned u = __builtin_bit_cast(unsigned, x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  const unsigned r0 = r[0], r1 = r[1];
  return fmaxf(__builtin_bit_cast(float, r0), __builtin_bit_cast(float, r1));
}

// Bias modes of the kernels: none, a dense (nh, S', S') matrix, ALiBi in closed form.
constexpr int kNoBias = 0, kDenseBias = 1, kAlibi = 2;

// ALiBi biases of four consecutive (query, key) distances d0, d0 + step, ..., bit for bit what the dense
// path reads from the matrix the reference builds (transformer.py:55-75): the distance key - query
// (<= 0) and the slope are fp16 values, their product is rounded to fp16 once, a bf16 kernel sees that
// value rounded to bf16 (the 16-bit matrix cast to the compute type).  Two distances are rounded to fp16
// by one conversion and multiplied by one packed fp16 instruction.  Returned as floats, NOT yet
// multiplied by log2(e): that product rides in the fma that adds the bias to the scaled score.
template <typename T> __device__ __forceinline__ void alibi4(float d0, float step, _Float16 slope, float (&b)[4]) {
  typedef _Float16 h2 __attribute__((ext_vector_type(2)));
  typedef float f2 __attribute__((ext_vector_type(2)));
  const f2 da = {d0, d0 + step}, db = {d0 + 2.f * step, d0 + 3.f * step};
  const h2 s2 = {slope, slope};
  const h2 pa = __builtin_convertvector(da, h2) * s2, pb = __builtin_convertvector(db, h2) * s2;
  b[0] = (float)pa[0]; b[1] = (float)pa[1]; b[2] = (float)pb[0]; b[3] = (float)pb[1];
  if (std::is_same<T, bf16>::value) {
#pragma unroll
    for (int e = 0; e < 4; ++e) b[e] = (float)(T)b[e];
  }
}

// Additive-bias tile of a 128-query block and a 64-key block, 16 KB, staged through LDS with
// coalesced direct-to-LDS loads: row r (128 bytes) keeps its 16-byte chunk c in slot
// c ^ ((r >> 1) & 7), which spreads the 8-byte per-lane reads (one row per lane) over the banks.
struct BiasTile {
  static constexpr int BYTES = 128 * 64 * 2;
  template <typename T>
  static __device__ __forceinline__ void init(const T* (&bp)[4], const T* bias_head, int64_t row_stride, int q0, int S) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int id = threadIdx.x + j * 256;
      const int row = id >> 3, c = (id & 7) ^ ((row >> 1) & 7);
      const int qrow = min(q0 + row, S - 1);  // rows past the sequence are never read back
      bp[j] = bias_head + (int64_t)qrow * row_stride + c * 8;
    }
  }
  // last block of a sequence that ends half way through it: chunks of key columns 32 .. 63 read 32 columns back
  template <typename T> static __device__ __forceinline__ void tail(const T* (&bp)[4]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int id = threadIdx.x + j * 256;
      const int row = id >> 3, c = (id & 7) ^ ((row >> 1) & 7);
      if (c >= 4) bp[j] -= 32;
    }
  }
  // next 64 keys into the tile at `dst`; advances the pointers
  template <typename T> static __device__ __forceinline__ void load(const T* (&bp)[4], char* dst, int wave) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      __builtin_amdgcn_global_load_lds((gptr_void*)bp[j], (lds_void*)(dst + (j * 256 + wave * 64) * 16), 16, 0, 0);
      bp[j] += 64;
    }
  }
  // LDS address (relative to the tile) of keys chunk*8 + 4*half .. +3 of query row r
  static __device__ __forceinline__ uint32_t addr(int r, int chunk, int half) {
    return (uint32_t)(r * 128 + ((chunk ^ ((r >> 1) & 7)) << 4) + half * 8);
  }
};

// (Register r of a 32x32 MFMA result covers row (r/4)*8 + 4*(lane/32) + r%4.)

// Write-out of a wave's 32 x HD result held as 32x32 MFMA accumulators (register g*4+e of slice d,
// lane l = row l%32, column d*32 + g*8 + 4*(l/32) + e): scaled, rounded, parked in a wave-private
// LDS slab and read back row-contiguously, so that every global store instruction covers whole
// 128-byte lines of complete rows (8 bytes per lane straight from the accumulators would fill each
// line piecewise over eight instructions).  LDS accesses of one wave execute in order: no barrier.
template <typename T, int HD>
__device__ __forceinline__ void store_rows32(char* slab, T* dst, int64_t row_stride, const f32x16 (&acc)[HD / 32],
                                             float scale, int lane) {
  typedef typename Vec<T>::v4 v4;
  constexpr int ROWB = HD * 2 + 16;  // padded row pitch in bytes
  constexpr int CH = HD * 2 / 16;    // 16-byte chunks per row
  constexpr int RPI = 64 / CH;       // rows covered by one wave-wide access
#pragma unroll
  for (int d = 0; d < HD / 32; ++d)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      v4 o;
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = (T)(acc[d][g * 4 + e] * scale);
      *reinterpret_cast<v4*>(slab + (lane & 31) * ROWB + (d * 32 + g * 8 + 4 * (lane >> 5)) * 2) = o;
    }
#pragma unroll
  for (int rr = 0; rr < 32 / RPI; ++rr) {
    const int r = rr * RPI + lane / CH, c = lane % CH;
    const u32x4 v = lds_ld16(slab, r * ROWB + c * 16);
    if constexpr (HD >= 64) st16(dst + (int64_t)r * row_stride + c * 8, v);  // whole lines: written through
    else *reinterpret_cast<u32x4*>(dst + (int64_t)r * row_stride + c * 8) = v;
  }
}


// ===========================================================================
// Forward.  Workgroup: 4 waves x 32 queries; key/value blocks of 64.
//
// The softmax arithmetic runs on the VALU and is what bounds this kernel, so it
// is kept to ~6 operations per score: one fma folds scale (and bias) into the
// exp2 argument, the running maximum is only raised (and the accumulators
// rescaled) when a row's maximum grew by more than 2^8 -- probabilities then
// stay below 256, exact in 16 bit -- the causal mask is only evaluated on
// blocks that touch the diagonal, and the row sums are produced by the matrix
// core (an all-ones operand against P) instead of 32 VALU adds per row.
// Occupancy: three waves per SIMD (168 VGPRs) for hd <= 64 without bias -- measured
// 13 % faster than two, the third wave fills VALU/MFMA gaps of the other two.
// K/V (and bias) tiles are loaded one block ahead straight into LDS; within a block all
// K operands are requested before the first MFMA and all V operands before the
// exponentials, as volatile-asm LDS reads with explicit waits (see common.h).
// ===========================================================================
constexpr float kRescaleThreshold = 8.0f;  // log2 domain

template <typename T, int HD, int BMODE, bool TAIL>
__global__ __launch_bounds__(256, HD > 64 ? 1 : (BMODE == kDenseBias ? 2 : 3)) void attn_fwd_kernel(AttnParams p) {
  constexpr bool HAS_BIAS = BMODE == kDenseBias, ALIBI = BMODE == kAlibi;
  typedef SeqTile<T, 64, HD> KT;
  typedef typename Vec<T>::v8 v8;
  typedef typename Vec<T>::v4 v4;
  constexpr int KS = HD / 16, DT = HD / 32;
  constexpr int STAGE = 2 * KT::BYTES + (HAS_BIAS ? BiasTile::BYTES : 0);
  static_assert(4 * 32 * (HD * 2 + 16) <= 2 * STAGE, "the result slabs of the four waves reuse the pipeline stages");
  constexpr int PT = KT::PER_THREAD;  // 16-byte chunks per thread per 64-row tile
  extern __shared__ __attribute__((aligned(16))) char smem[];

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);  // the same number as a scalar: LDS slot addresses of the tile loads stay scalar arithmetic
  const int nbh = p.B * p.nh;
  const int nqb = (p.S + 127) / 128;
  const int qblk = nqb - 1 - (int)(blockIdx.x / nbh);  // heaviest query blocks first
  const int bh = blockIdx.x % nbh;
  const int b = bh / p.nh, h = bh % p.nh;
  const _Float16 slope = ALIBI ? ((const _Float16*)p.slopes)[h] : (_Float16)0.f;
  const int64_t base = (int64_t)b * p.sb + (int64_t)h * p.sh;
  const T* Q = (const T*)p.q + base;
  const T* K = (const T*)p.k + base;
  const T* V = (const T*)p.v + base;
  T* O = (T*)p.out + (int64_t)b * p.osb + (int64_t)h * p.osh;

  const int q0 = qblk * 128;
  const int q0w = q0 + wave * 32;
  const bool active = q0w < p.S;
  const int myq = q0w + (lane & 31);
  const int kv_end = min(p.S, q0 + 128);
  const int nkv = (kv_end + 63) / 64;  // the last block may be half beyond the sequence (S = 32 mod 64)

  v8 qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    u32x4 raw = {0u, 0u, 0u, 0u};
    if (active) raw = ld16(Q + (int64_t)myq * p.ss + ks * 16 + (lane >> 5) * 8);
    qf[ks] = __builtin_bit_cast(v8, raw);
  }
  v8 ones;
#pragma unroll
  for (int e = 0; e < 8; ++e) ones[e] = (T)1.0f;

  f32x16 oacc[DT], lacc;
#pragma unroll
  for (int r = 0; r < 16; ++r) lacc[r] = 0.f;
#pragma unroll
  for (int d = 0; d < DT; ++d)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[d][r] = 0.f;
  float m_ref = -INFINITY;  // reference maximum (log2 domain) the accumulators are scaled to

  // K and V (and bias) tiles go from global memory straight into LDS, no register staging
  const T* kp[PT];
  KT::stream_init(kp, K, p.ss, 0);
  const int64_t v_minus_k = V - K;
  const T* bp[4];
  if (HAS_BIAS) BiasTile::init(bp, (const T*)p.bias + (int64_t)h * p.bias_sh, p.bias_sr, q0, p.S);
  auto load_tile = [&](int stage_off) {  // next 64 keys / values (/ bias columns) into the stage at byte offset stage_off
#pragma unroll
    for (int j = 0; j < PT; ++j) {
      __builtin_amdgcn_global_load_lds((gptr_void*)kp[j], (lds_void*)KT::stream_slot(smem + stage_off, wave_u, j), 16, 0, 0);
      __builtin_amdgcn_global_load_lds((gptr_void*)(kp[j] + v_minus_k),
                                       (lds_void*)KT::stream_slot(smem + stage_off + KT::BYTES, wave_u, j), 16, 0, 0);
      kp[j] += (int64_t)64 * p.ss;
    }
    if (HAS_BIAS) BiasTile::load(bp, smem + stage_off + 2 * KT::BYTES, wave_u);
  };
  // the loads of key block jb: if the sequence ends inside it (TAIL: S = 32 mod 64, an instantiation of its
  // own, so that whole-block sequences pay nothing), rows / bias columns 32 .. 63 are taken 32 earlier
  auto load_block_of = [&](int jb, int stage_off) {
    if (TAIL && (jb + 1) * 64 > p.S) {
      KT::stream_tail(kp, p.ss);
      if (HAS_BIAS) BiasTile::tail(bp);
    }
    load_tile(stage_off);
  };
  uint32_t ka[KS], va[DT][2];
  const uint32_t lds0 = lds_address(smem);
  KT::operand_addrs(ka, va, lds0, lane);

  load_block_of(0, 0);
  __syncthreads();

  // One 64-key block out of the stage at byte offset SOFF.
  auto step = [&](auto stage_tag, int j) {
    constexpr int SOFF = decltype(stage_tag)::value * STAGE;
    constexpr int VOFF = SOFF + KT::BYTES;
    if (j + 1 < nkv) load_block_of(j + 1, STAGE - SOFF);
    const int kb = j * 64;
    if (active && kb <= q0w + 31) {
      auto block = [&](auto diag_tag) {
        constexpr bool DIAG = decltype(diag_tag)::value;
        // on a diagonal block the second 32-key half may lie entirely above the diagonal
        const bool live1 = !DIAG || kb + 32 <= q0w + 31;
        // all K operands of the block are requested before the first MFMA
        u32x4 kf[2][KS];
        static_for<2 * KS>([&](auto it) {
          constexpr int jt = decltype(it)::value % 2, ks = decltype(it)::value / 2;  // the two halves alternate
          lds_read128_at<SOFF + jt * 32 * HD * 2>(kf[jt][ks], ka[ks]);
        });
        // ... and so are this lane's bias values: keys jt*32 + g*8 + 4*(lane/32) .. +3 of its query row
        constexpr int NB = HAS_BIAS ? 8 : 0;
        u32x2 braw[HAS_BIAS ? 8 : 1];
        if constexpr (HAS_BIAS) {
          const int r = wave * 32 + (lane & 31);
          static_for<8>([&](auto it) {
            constexpr int c = decltype(it)::value;  // 16-byte chunk = jt*4 + g
            lds_read64_at<0>(braw[c], lds0 + (SOFF + 2 * KT::BYTES) + BiasTile::addr(r, c, lane >> 5));
          });
        }
        f32x16 st[2];
#pragma unroll
        for (int jt = 0; jt < 2; ++jt)
#pragma unroll
          for (int r = 0; r < 16; ++r) st[jt][r] = 0.f;
        static_for<2 * KS>([&](auto it) {
          constexpr int idx = decltype(it)::value, jt = idx % 2, ks = idx / 2;  // two independent accumulation chains
          constexpr int later = 2 * KS - 1 - idx + NB;
          lds_wait<(later < 15 ? later : 15)>(kf[jt][ks]);
          st[jt] = mfma32(__builtin_bit_cast(v8, kf[jt][ks]), qf[ks], st[jt]);
        });
        // block maximum; without bias it is taken over the raw scores and scaled once
        float mx = -INFINITY;
        static_for<8>([&](auto it) {
          constexpr int jt = decltype(it)::value / 4, g = decltype(it)::value % 4;
          {
            const int key0 = kb + jt * 32 + g * 8 + 4 * (lane >> 5);
            float bv[4] = {0.f, 0.f, 0.f, 0.f};
            if constexpr (HAS_BIAS) {
              lds_wait<7 - decltype(it)::value>(braw[jt * 4 + g]);
              const v4 raw = __builtin_bit_cast(v4, braw[jt * 4 + g]);
#pragma unroll
              for (int e = 0; e < 4; ++e) bv[e] = (float)raw[e];
            }
            if constexpr (ALIBI) alibi4<T>((float)(key0 - myq), 1.f, slope, bv);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              float x = st[jt][g * 4 + e];
              // score * scale * log2e + bias * log2e: the 16-bit bias goes into the fma as it is
              if (HAS_BIAS || ALIBI) x = __builtin_fmaf(bv[e], kLog2e, x * p.scale_log2);
              if (DIAG && (key0 + e > myq || (jt == 1 && !live1))) x = -INFINITY;
              st[jt][g * 4 + e] = x;
              mx = fmaxf(mx, x);
            }
          }
        });
        // the V operands are requested now and arrive while the exponentials are computed
        constexpr int NVF = 4 * DT;  // operands of the block: (32-key half, 16-key step, 32-wide hd slice)
        u32x2 vlo[NVF], vhi[NVF];
        static_for<NVF>([&](auto it) {
          constexpr int idx = decltype(it)::value, jt = idx / (2 * DT), t = (idx / DT) % 2, d = idx % DT;
          constexpr int off = VOFF + (jt * 32 + t * 16) * HD * 2;
          lds_read64_tr_at<off>(vlo[idx], va[d][0]);
          lds_read64_tr_at<off>(vhi[idx], va[d][1]);
        });
        mx = max_with_other_half(mx);
        if (!HAS_BIAS && !ALIBI) mx *= p.scale_log2;  // scale > 0: max(s) * scale = max(s * scale)
        // raise the reference maximum only when some row outgrew it by 2^8
        const bool grow = mx > m_ref + kRescaleThreshold;
        if (__any(grow)) {
          const float m_new = grow ? mx : m_ref;
          const float alpha = grow ? fast_exp2(m_ref - m_new) : 1.0f;  // exp2(-inf) = 0 on the first block
          m_ref = m_new;
#pragma unroll
          for (int r = 0; r < 16; ++r) lacc[r] *= alpha;
#pragma unroll
          for (int d = 0; d < DT; ++d)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[d][r] *= alpha;
        }
        const float m_use = m_ref == -INFINITY ? 0.f : m_ref;  // row with nothing but -inf so far
#pragma unroll
        for (int jt = 0; jt < 2; ++jt)
#pragma unroll
          for (int r = 0; r < 16; ++r)
            st[jt][r] = fast_exp2((HAS_BIAS || ALIBI) ? st[jt][r] - m_use : fmaf(st[jt][r], p.scale_log2, -m_use));
        // every requested operand is consumed (a half above the diagonal contributes P = 0)
        static_for<4>([&](auto it) {
          constexpr int jt = decltype(it)::value / 2, t = decltype(it)::value % 2;
          const v8 pb = round8<T>(st[jt], t);
          lacc = mfma32(ones, pb, lacc);  // every row of lacc = sum over keys of P
          static_for<DT>([&](auto dd) {
            constexpr int d = decltype(dd)::value, idx = (jt * 2 + t) * DT + d;
            constexpr int later = 2 * (NVF - 1 - idx);  // LDS reads requested after this operand
            lds_wait<(later < 15 ? later : 15)>(vhi[idx]);
            lds_tie(vlo[idx]);
            const u32x4 v = {vlo[idx][0], vlo[idx][1], vhi[idx][0], vhi[idx][1]};
            oacc[d] = mfma32(__builtin_bit_cast(v8, v), pb, oacc[d]);
          });
        });
      };
      if (kb + 63 > q0w) block(std::true_type{});
      else block(std::false_type{});
    }
    __syncthreads();  // waits for this thread's tile loads, then for everyone's; all reads of this stage are done
  };

  for (int j = 0; j < nkv; j += 2) {
    step(std::integral_constant<int, 0>{}, j);
    if (j + 1 < nkv) step(std::integral_constant<int, 1>{}, j + 1);
  }

  if (active) {
    const float l_tot = lacc[0];
    const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
    if (lane < 32) p.lse[(int64_t)bh * p.S + myq] = m_ref + log2f(l_tot);
    // the pipeline stages are free: every wave is past the last barrier of the loop
    store_rows32<T, HD>(smem + wave * (32 * (HD * 2 + 16)), O + (int64_t)q0w * p.oss, p.oss, oacc, inv, lane);
  }
}

// ===========================================================================
// dK/dV pass.  Workgroup: 4 waves x 32 keys; query blocks of 64 from the
// diagonal downwards.  Q and dO tiles (+ their lse / delta) go through LDS.
// ===========================================================================
template <typename T, int HD, int BMODE, bool TAIL>
__global__ __launch_bounds__(256, HD <= 64 ? 2 : 1) void attn_dkdv_kernel(AttnParams p) {
  constexpr bool HAS_BIAS = BMODE == kDenseBias, ALIBI = BMODE == kAlibi;
  typedef SeqTile<T, 64, HD> QT;
  typedef typename Vec<T>::v8 v8;
  typedef typename Vec<T>::v4 v4;
  constexpr int KS = HD / 16, DT = HD / 32;
  constexpr int PT = QT::PER_THREAD;
  // one stage: Q tile, dO tile, lse[64] and -delta[64] (fp32), bias tile [64 queries][128 keys]
  constexpr int STAT = 2 * QT::BYTES, BIAS = STAT + 2 * 64 * 4;
  constexpr int BIAS_BYTES = 64 * 128 * 2;
  constexpr int STAGE = BIAS + (HAS_BIAS ? BIAS_BYTES : 0);
  static_assert(4 * 32 * (HD * 2 + 16) <= 2 * STAGE, "the result slabs of the four waves reuse the pipeline stages");
  extern __shared__ __attribute__((aligned(16))) char smem[];

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);  // the same number as a scalar: LDS slot addresses of the tile loads stay scalar arithmetic
  const int nbh = p.B * p.nh;
  const int kblk = (int)(blockIdx.x / nbh);  // lowest key blocks (longest loops) first
  const int bh = blockIdx.x % nbh;
  const int b = bh / p.nh, h = bh % p.nh;
  const _Float16 slope = ALIBI ? ((const _Float16*)p.slopes)[h] : (_Float16)0.f;
  const int64_t base = (int64_t)b * p.sb + (int64_t)h * p.sh;
  const T* Q = (const T*)p.q + base;
  const T* K = (const T*)p.k + base;
  const T* V = (const T*)p.v + base;
  const T* dO = (const T*)p.d_o + (int64_t)b * p.osb + (int64_t)h * p.osh;

  const int k0 = kblk * 128;
  const int kw0 = k0 + wave * 32;
  const bool active = kw0 < p.S;
  const int mykey = kw0 + (lane & 31);

  v8 kf[KS], vf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    u32x4 a = {0u, 0u, 0u, 0u}, c = {0u, 0u, 0u, 0u};
    if (active) {
      a = ld16(K + (int64_t)mykey * p.ss + ks * 16 + (lane >> 5) * 8);
      c = ld16(V + (int64_t)mykey * p.ss + ks * 16 + (lane >> 5) * 8);
    }
    kf[ks] = __builtin_bit_cast(v8, a);
    vf[ks] = __builtin_bit_cast(v8, c);
  }
  f32x16 dk[DT], dv[DT];
#pragma unroll
  for (int d = 0; d < DT; ++d)
#pragma unroll
    for (int r = 0; r < 16; ++r) { dk[d][r] = 0.f; dv[d][r] = 0.f; }

  const int nq = (p.S - k0 + 63) / 64;  // query blocks k0, k0+64, ...; the last one may be half beyond the sequence

  // Everything a query block needs goes from global memory straight into LDS: the Q and dO
  // tiles (chunk swizzle on the global side), the two statistics rows (one float per lane of
  // waves 0 and 1) and, with a bias, its [64][128] tile in plain row-major order.
  const T* qp[PT];
  const T* dop[PT];
  QT::stream_init(qp, Q, p.ss, k0);
  QT::stream_init(dop, dO, p.oss, k0);
  const float* statp = (wave == 0 ? p.lse : p.delta) + (int64_t)bh * p.S + k0 + lane;  // waves 0, 1 only
  const T* bp[4];
  if (HAS_BIAS) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int id = threadIdx.x + j * 256;
      const int row = id >> 4;
      int col = k0 + (id & 15) * 8;
      if (col >= p.S) col = k0;  // keys past the sequence belong to inactive waves: any in-bounds column will do
      bp[j] = (const T*)p.bias + (int64_t)h * p.bias_sh + (int64_t)(k0 + row) * p.bias_sr + col;
    }
  }
  auto load_block = [&](int stage_off) {  // next 64 queries into the stage at byte offset stage_off
#pragma unroll
    for (int j = 0; j < PT; ++j) {
      __builtin_amdgcn_global_load_lds((gptr_void*)qp[j], (lds_void*)QT::stream_slot(smem + stage_off, wave_u, j), 16, 0, 0);
      __builtin_amdgcn_global_load_lds((gptr_void*)dop[j], (lds_void*)QT::stream_slot(smem + stage_off + QT::BYTES, wave_u, j),
                                       16, 0, 0);
      qp[j] += (int64_t)64 * p.ss;
      dop[j] += (int64_t)64 * p.oss;
    }
    if (wave < 2) {
      __builtin_amdgcn_global_load_lds((gptr_void*)statp, (lds_void*)(smem + stage_off + STAT + wave_u * 256), 4, 0, 0);
      statp += 64;
    }
    if (HAS_BIAS) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        __builtin_amdgcn_global_load_lds((gptr_void*)bp[j], (lds_void*)(smem + stage_off + BIAS + (j * 256 + wave_u * 64) * 16),
                                         16, 0, 0);
        bp[j] += (int64_t)64 * p.bias_sr;
      }
    }
  };
  // lane-dependent parts of the LDS addresses
  const uint32_t lds0 = lds_address(smem);
  uint32_t ra[KS], ha[DT][2];
  QT::operand_addrs(ra, ha, lds0, lane);
  const uint32_t sa = lds0 + STAT + 16 * (lane >> 5);  // statistics of queries g*8 + 4*(lane/32) .. +3
  const uint32_t ba = lds0 + BIAS + (4 * (lane >> 5)) * 256 + (wave * 32 + (lane & 31)) * 2;

  // the loads of query block ib: if the sequence ends inside it, its rows 32 .. 63 (tiles, statistics, bias rows)
  // are taken 32 earlier; the sub-tile they fill is never used
  auto load_block_of = [&](int ib, int stage_off) {
    if (TAIL && k0 + (ib + 1) * 64 > p.S) {
      QT::stream_tail(qp, p.ss);
      QT::stream_tail(dop, p.oss);
      if (lane >= 32) statp -= 32;
      if (HAS_BIAS) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (((threadIdx.x + j * 256) >> 4) >= 32) bp[j] -= (int64_t)32 * p.bias_sr;
      }
    }
    load_block(stage_off);
  };
  if (nq > 0) load_block_of(0, 0);
  __syncthreads();

  auto step = [&](auto stage_tag, int it) {
    constexpr int SOFF = decltype(stage_tag)::value * STAGE;
    if (it + 1 < nq) load_block_of(it + 1, STAGE - SOFF);
    const int qb = k0 + it * 64;
    if (active) {
      static_for<2>([&](auto qt_tag) {
        constexpr int qt = decltype(qt_tag)::value;
        const int qs = qb + qt * 32;      // first query of this 32-row sub-tile
        if (qs + 31 < kw0) return;        // entirely above the diagonal for this wave
        if (TAIL && qs >= p.S) return;    // beyond the sequence (the second half of its last block)
        auto tile = [&](auto diag_tag) {
          constexpr bool DIAG = decltype(diag_tag)::value;
          constexpr int ROFF = SOFF + qt * 32 * HD * 2;
          // requests, in the order they are consumed: -delta (dP starts there, so dP - delta costs
          // nothing), lse, then the row-major Q and dO operands
          u32x4 dl[4], ls[4], qr[KS], dor[KS];
          static_for<4>([&](auto g) {
            lds_read128_at<SOFF + 256 + qt * 128 + decltype(g)::value * 32>(dl[decltype(g)::value], sa);
          });
          static_for<4>([&](auto g) {
            lds_read128_at<SOFF + qt * 128 + decltype(g)::value * 32>(ls[decltype(g)::value], sa);
          });
          static_for<KS>([&](auto it2) {
            constexpr int ks = decltype(it2)::value;
            lds_read128_at<ROFF>(qr[ks], ra[ks]);
            lds_read128_at<ROFF + QT::BYTES>(dor[ks], ra[ks]);
          });
          lds_wait<(2 * KS < 15 ? 2 * KS : 15)>(ls[3]);  // statistics have landed; the operands may be in flight
          static_for<4>([&](auto g) { lds_tie(dl[decltype(g)::value]); lds_tie(ls[decltype(g)::value]); });
          f32x16 s, dp;
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const f32x4 d4 = __builtin_bit_cast(f32x4, dl[g]);
#pragma unroll
            for (int e = 0; e < 4; ++e) { s[g * 4 + e] = 0.f; dp[g * 4 + e] = d4[e]; }
          }
          static_for<KS>([&](auto it2) {
            constexpr int ks = decltype(it2)::value;
            constexpr int later_q = 2 * (KS - 1 - ks) + 1;
            lds_wait<(later_q < 15 ? later_q : 15)>(qr[ks]);
            s = mfma32(__builtin_bit_cast(v8, qr[ks]), kf[ks], s);
            lds_wait<(later_q - 1 < 15 ? later_q - 1 : 15)>(dor[ks]);
            dp = mfma32(__builtin_bit_cast(v8, dor[ks]), vf[ks], dp);
          });
          // bias values, then the hd-major operands of the two accumulating products; they arrive
          // during the exponentials
          uint32_t braw[HAS_BIAS ? 16 : 1];
          if constexpr (HAS_BIAS) {
            static_for<16>([&](auto r) {
              constexpr int g = decltype(r)::value / 4, e = decltype(r)::value % 4;
              lds_read_u16_at<SOFF + (qt * 32 + g * 8 + e) * 256>(braw[decltype(r)::value], ba);
            });
          }
          constexpr int NH = 2 * DT;  // (16-query slice, 32-wide hd slice)
          u32x2 dlo[NH], dhi[NH], qlo[NH], qhi[NH];
          static_for<NH>([&](auto it2) {
            constexpr int idx = decltype(it2)::value, t = idx / DT, d = idx % DT;
            constexpr int off = SOFF + (qt * 32 + t * 16) * HD * 2;
            lds_read64_tr_at<off + QT::BYTES>(dlo[idx], ha[d][0]);
            lds_read64_tr_at<off + QT::BYTES>(dhi[idx], ha[d][1]);
            lds_read64_tr_at<off>(qlo[idx], ha[d][0]);
            lds_read64_tr_at<off>(qhi[idx], ha[d][1]);
          });
          if constexpr (HAS_BIAS) {
            lds_wait<(4 * NH < 15 ? 4 * NH : 15)>(braw[15]);  // bias values have landed; operands may be in flight
            static_for<15>([&](auto r) { lds_tie(braw[decltype(r)::value]); });
          }
          static_for<4>([&](auto gt) {
            constexpr int g = decltype(gt)::value;
            const int ql = qt * 32 + g * 8 + 4 * (lane >> 5);  // block-local first query of the group
            const f32x4 l4 = __builtin_bit_cast(f32x4, ls[g]);
            float bv[4] = {0.f, 0.f, 0.f, 0.f};
            if constexpr (ALIBI) alibi4<T>((float)(mykey - (qb + ql)), -1.f, slope, bv);  // queries ascend: distances descend
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const int qi = qb + ql + e;
              float x = fmaf(s[g * 4 + e], p.scale_log2, -l4[e]);  // s*scale*log2e - lse
              if constexpr (HAS_BIAS) bv[e] = (float)__builtin_bit_cast(T, (uint16_t)braw[g * 4 + e]);
              if constexpr (HAS_BIAS || ALIBI) x = __builtin_fmaf(bv[e], kLog2e, x);
              float pr = fast_exp2(x);
              if (DIAG && mykey > qi) pr = 0.f;
              s[g * 4 + e] = pr;
              dp[g * 4 + e] *= pr;
            }
          });
          static_for<NH>([&](auto it2) {
            constexpr int idx = decltype(it2)::value, t = idx / DT, d = idx % DT;
            constexpr int later_d = 4 * (NH - 1 - idx) + 2, later_q = later_d - 2;
            const v8 pa = round8<T>(s, t);
            const v8 dsa = round8<T>(dp, t);
            lds_wait<(later_d < 15 ? later_d : 15)>(dhi[idx]);
            lds_tie(dlo[idx]);
            const u32x4 a = {dlo[idx][0], dlo[idx][1], dhi[idx][0], dhi[idx][1]};
            dv[d] = mfma32(__builtin_bit_cast(v8, a), pa, dv[d]);
            lds_wait<(later_q < 15 ? later_q : 15)>(qhi[idx]);
            lds_tie(qlo[idx]);
            const u32x4 c = {qlo[idx][0], qlo[idx][1], qhi[idx][0], qhi[idx][1]};
            dk[d] = mfma32(__builtin_bit_cast(v8, c), dsa, dk[d]);
          });
        };
        if (qs < kw0 + 31) tile(std::true_type{});
        else tile(std::false_type{});
      });
    }
    __syncthreads();  // this thread's block loads have landed, then everyone's; all reads of this stage are done
  };
  for (int it = 0; it < nq; it += 2) {
    step(std::integral_constant<int, 0>{}, it);
    if (it + 1 < nq) step(std::integral_constant<int, 1>{}, it + 1);
  }

  if (active) {
    T* dK = (T*)p.dk + base;
    T* dV = (T*)p.dv + base;
    // the pipeline stages are free: every wave is past the last barrier of the loop
    char* slab = smem + wave * (32 * (HD * 2 + 16));
    const int64_t row0 = (int64_t)(mykey - (lane & 31)) * p.ss;
    store_rows32<T, HD>(slab, dK + row0, p.ss, dk, p.scale, lane);
    store_rows32<T, HD>(slab, dV + row0, p.ss, dv, 1.0f, lane);
  }
}

// ===========================================================================
// dQ pass.  Workgroup: 4 waves x 32 queries; key/value blocks of 64 up to the
// diagonal, K and V tiles through LDS.
// ===========================================================================
template <typename T, int HD, int BMODE, bool TAIL>
__global__ __launch_bounds__(256, HD > 64 ? 1 : (BMODE != kNoBias ? 2 : 3)) void attn_dq_kernel(AttnParams p) {
  constexpr bool HAS_BIAS = BMODE == kDenseBias, ALIBI = BMODE == kAlibi;
  typedef SeqTile<T, 64, HD> KT;
  typedef typename Vec<T>::v8 v8;
  typedef typename Vec<T>::v4 v4;
  constexpr int KS = HD / 16, DT = HD / 32;
  constexpr int STAGE = 2 * KT::BYTES + (HAS_BIAS ? BiasTile::BYTES : 0);
  static_assert(4 * 32 * (HD * 2 + 16) <= 2 * STAGE, "the result slabs of the four waves reuse the pipeline stages");
  extern __shared__ __attribute__((aligned(16))) char smem[];

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);  // the same number as a scalar: LDS slot addresses of the tile loads stay scalar arithmetic
  const int nbh = p.B * p.nh;
  const int nqb = (p.S + 127) / 128;
  const int qblk = nqb - 1 - (int)(blockIdx.x / nbh);
  const int bh = blockIdx.x % nbh;
  const int b = bh / p.nh, h = bh % p.nh;
  const _Float16 slope = ALIBI ? ((const _Float16*)p.slopes)[h] : (_Float16)0.f;
  const int64_t base = (int64_t)b * p.sb + (int64_t)h * p.sh;
  const T* Q = (const T*)p.q + base;
  const T* K = (const T*)p.k + base;
  const T* V = (const T*)p.v + base;
  const T* dO = (const T*)p.d_o + (int64_t)b * p.osb + (int64_t)h * p.osh;

  const int q0 = qblk * 128;
  const int q0w = q0 + wave * 32;
  const bool active = q0w < p.S;
  const int myq = q0w + (lane & 31);
  const int kv_end = min(p.S, q0 + 128);
  const int nkv = (kv_end + 63) / 64;  // the last block may be half beyond the sequence (S = 32 mod 64)

  v8 qf[KS], dof[KS];
  float neg_lse = 0.f, neg_delta = 0.f;
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    u32x4 a = {0u, 0u, 0u, 0u}, c = {0u, 0u, 0u, 0u};
    if (active) {
      a = ld16(Q + (int64_t)myq * p.ss + ks * 16 + (lane >> 5) * 8);
      c = ld16(dO + (int64_t)myq * p.oss + ks * 16 + (lane >> 5) * 8);
    }
    qf[ks] = __builtin_bit_cast(v8, a);
    dof[ks] = __builtin_bit_cast(v8, c);
  }
  if (active) {
    neg_lse = -p.lse[(int64_t)bh * p.S + myq];
    // -delta = -rowsum(dO * O) of this lane's query row: each of the two lanes that share a row has half
    // of it.  Stored for the dK/dV pass, which runs after this one.
    const T* Orow = (const T*)p.o + (int64_t)b * p.osb + (int64_t)h * p.osh + (int64_t)myq * p.oss + (lane >> 5) * 8;
    float half_sum = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const v8 o = __builtin_bit_cast(v8, ld16(Orow + ks * 16));
#pragma unroll
      for (int e = 0; e < 8; ++e) half_sum = fmaf((float)o[e], (float)dof[ks][e], half_sum);
    }
    const unsigned u = __builtin_bit_cast(unsigned, half_sum);
    const auto both = __builtin_amdgcn_permlane32_swap(u, u, false, false);  // own half and the partner's
    const unsigned u0 = both[0], u1 = both[1];
    neg_delta = -(__builtin_bit_cast(float, u0) + __builtin_bit_cast(float, u1));
    if (lane < 32) p.delta[(int64_t)bh * p.S + myq] = neg_delta;
  }
  f32x16 dq[DT];
#pragma unroll
  for (int d = 0; d < DT; ++d)
#pragma unroll
    for (int r = 0; r < 16; ++r) dq[d][r] = 0.f;

  // K and V (and bias) tiles go from global memory straight into LDS
  constexpr int PT = KT::PER_THREAD;
  const T* kp[PT];
  KT::stream_init(kp, K, p.ss, 0);
  const int64_t v_minus_k = V - K;
  const T* bp[4];
  if (HAS_BIAS) BiasTile::init(bp, (const T*)p.bias + (int64_t)h * p.bias_sh, p.bias_sr, q0, p.S);
  auto load_tile = [&](int stage_off) {
#pragma unroll
    for (int j = 0; j < PT; ++j) {
      __builtin_amdgcn_global_load_lds((gptr_void*)kp[j], (lds_void*)KT::stream_slot(smem + stage_off, wave_u, j), 16, 0, 0);
      __builtin_amdgcn_global_load_lds((gptr_void*)(kp[j] + v_minus_k),
                                       (lds_void*)KT::stream_slot(smem + stage_off + KT::BYTES, wave_u, j), 16, 0, 0);
      kp[j] += (int64_t)64 * p.ss;
    }
    if (HAS_BIAS) BiasTile::load(bp, smem + stage_off + 2 * KT::BYTES, wave_u);
  };
  // the loads of key block jb: if the sequence ends inside it (TAIL: S = 32 mod 64, an instantiation of its
  // own, so that whole-block sequences pay nothing), rows / bias columns 32 .. 63 are taken 32 earlier
  auto load_block_of = [&](int jb, int stage_off) {
    if (TAIL && (jb + 1) * 64 > p.S) {
      KT::stream_tail(kp, p.ss);
      if (HAS_BIAS) BiasTile::tail(bp);
    }
    load_tile(stage_off);
  };
  // row operands of K and V, hd operands of K
  uint32_t ra[KS], ha[DT][2];
  const uint32_t lds0 = lds_address(smem);
  KT::operand_addrs(ra, ha, lds0, lane);

  load_block_of(0, 0);
  __syncthreads();

  auto step = [&](auto stage_tag, int j) {
    constexpr int SOFF = decltype(stage_tag)::value * STAGE;
    if (j + 1 < nkv) load_block_of(j + 1, STAGE - SOFF);
    const int kb = j * 64;
    if (active) {
      static_for<2>([&](auto jt_tag) {
        constexpr int jt = decltype(jt_tag)::value;
        const int ks0 = kb + jt * 32;  // first key of this 32-key sub-tile
        if (ks0 > q0w + 31) return;
        auto tile = [&](auto diag_tag) {
          constexpr bool DIAG = decltype(diag_tag)::value;
          // every operand of the sub-tile is requested before its first MFMA
          constexpr int ROFF = SOFF + jt * 32 * HD * 2;
          u32x4 kr[KS], vr[KS];
          static_for<KS>([&](auto it) {
            constexpr int ks = decltype(it)::value;
            lds_read128_at<ROFF>(kr[ks], ra[ks]);
            lds_read128_at<ROFF + KT::BYTES>(vr[ks], ra[ks]);
          });
          // ... and this lane's bias values: keys jt*32 + g*8 + 4*(lane/32) .. +3 of its query row
          constexpr int NB = HAS_BIAS ? 4 : 0;
          u32x2 braw[HAS_BIAS ? 4 : 1];
          if constexpr (HAS_BIAS) {
            const int r = wave * 32 + (lane & 31);
            static_for<4>([&](auto it) {
              constexpr int g = decltype(it)::value;
              lds_read64_at<0>(braw[g], lds0 + (SOFF + 2 * KT::BYTES) + BiasTile::addr(r, jt * 4 + g, lane >> 5));
            });
          }
          f32x16 s, dp;
#pragma unroll
          for (int r = 0; r < 16; ++r) { s[r] = 0.f; dp[r] = neg_delta; }  // dP - delta for free
          static_for<KS>([&](auto it) {
            constexpr int ks = decltype(it)::value;
            constexpr int later_k = 2 * (KS - 1 - ks) + 1 + NB, later_v = later_k - 1;
            lds_wait<(later_k < 15 ? later_k : 15)>(kr[ks]);
            s = mfma32(__builtin_bit_cast(v8, kr[ks]), qf[ks], s);
            lds_wait<(later_v < 15 ? later_v : 15)>(vr[ks]);
            dp = mfma32(__builtin_bit_cast(v8, vr[ks]), dof[ks], dp);
          });
          // the hd-major K operands of dQ += dS K are requested now and arrive during the VALU work
          constexpr int NH = 2 * DT;
          u32x2 hlo[NH], hhi[NH];
          static_for<NH>([&](auto it) {
            constexpr int idx = decltype(it)::value, t = idx / DT, d = idx % DT;
            constexpr int off = SOFF + (jt * 32 + t * 16) * HD * 2;
            lds_read64_tr_at<off>(hlo[idx], ha[d][0]);
            lds_read64_tr_at<off>(hhi[idx], ha[d][1]);
          });
          // (the bias values were requested before the hd-major operands: NH more reads are in flight)
          static_for<4>([&](auto gt) {
            constexpr int g = decltype(gt)::value;
            const int key0 = ks0 + g * 8 + 4 * (lane >> 5);
            float bv[4] = {0.f, 0.f, 0.f, 0.f};
            if constexpr (HAS_BIAS) {
              constexpr int later = 3 - g + 2 * NH;
              lds_wait<(later < 15 ? later : 15)>(braw[g]);
              const v4 raw = __builtin_bit_cast(v4, braw[g]);
#pragma unroll
              for (int e = 0; e < 4; ++e) bv[e] = (float)raw[e];
            }
            if constexpr (ALIBI) alibi4<T>((float)(key0 - myq), 1.f, slope, bv);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              float x = fmaf(s[g * 4 + e], p.scale_log2, neg_lse);
              if (HAS_BIAS || ALIBI) x = __builtin_fmaf(bv[e], kLog2e, x);
              float pr = fast_exp2(x);
              if (DIAG && key0 + e > myq) pr = 0.f;
              dp[g * 4 + e] *= pr;
            }
          });
          static_for<NH>([&](auto it) {
            constexpr int idx = decltype(it)::value, t = idx / DT, d = idx % DT;
            constexpr int later = 2 * (NH - 1 - idx);
            const v8 dsb = round8<T>(dp, t);
            lds_wait<(later < 15 ? later : 15)>(hhi[idx]);
            lds_tie(hlo[idx]);
            const u32x4 v = {hlo[idx][0], hlo[idx][1], hhi[idx][0], hhi[idx][1]};
            dq[d] = mfma32(__builtin_bit_cast(v8, v), dsb, dq[d]);
          });
        };
        if (ks0 + 31 > q0w) tile(std::true_type{});
        else tile(std::false_type{});
      });
    }
    __syncthreads();  // this thread's tile loads have landed, then everyone's; all reads of this stage are done
  };
  for (int j = 0; j < nkv; j += 2) {
    step(std::integral_constant<int, 0>{}, j);
    if (j + 1 < nkv) step(std::integral_constant<int, 1>{}, j + 1);
  }

  if (active) {
    T* dQ = (T*)p.dq + base;
    // the pipeline stages are free: every wave is past the last barrier of the loop
    store_rows32<T, HD>(smem + wave * (32 * (HD * 2 + 16)), dQ + (int64_t)(myq - (lane & 31)) * p.ss, p.ss, dq, p.scale,
                        lane);
  }
}

// ---------------------------------------------------------------------------
// host dispatch
// ---------------------------------------------------------------------------
template <typename K>
static void allow_lds(K kernel, int bytes) {
  if (bytes > 64 * 1024)
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
}

template <typename T, int HD, int MODE, bool TAIL>
static int fwd_launch(hipStream_t st, const AttnParams& p) {
  constexpr int lds = 2 * (2 * SeqTile<T, 64, HD>::BYTES + (MODE == kDenseBias ? BiasTile::BYTES : 0));
  auto kernel = attn_fwd_kernel<T, HD, MODE, TAIL>;
  static bool once = (allow_lds(kernel, lds), true);
  (void)once;
  const unsigned grid = (unsigned)(((p.S + 127) / 128) * p.B * p.nh);
  kernel<<<dim3(grid), dim3(256), lds, st>>>(p);
  TF_CHECK_LAUNCH();
  return TF_OK;
}

// dQ pass first: it also produces the -delta rows that the dK/dV pass reads.
template <typename T, int HD, int MODE, bool TAIL>
static int bwd_launch(hipStream_t st, const AttnParams& p) {
  const unsigned grid = (unsigned)(((p.S + 127) / 128) * p.B * p.nh);
  {
    constexpr int lds = 2 * (2 * SeqTile<T, 64, HD>::BYTES + (MODE == kDenseBias ? BiasTile::BYTES : 0));
    auto kernel = attn_dq_kernel<T, HD, MODE, TAIL>;
    static bool once = (allow_lds(kernel, lds), true);
    (void)once;
    kernel<<<dim3(grid), dim3(256), lds, st>>>(p);
    TF_CHECK_LAUNCH();
  }
  {
    constexpr int lds = 2 * (2 * SeqTile<T, 64, HD>::BYTES + 2 * 64 * 4 + (MODE == kDenseBias ? 64 * 128 * 2 : 0));
    auto kernel = attn_dkdv_kernel<T, HD, MODE, TAIL>;
    static bool once = (allow_lds(kernel, lds), true);
    (void)once;
    kernel<<<dim3(grid), dim3(256), lds, st>>>(p);
    TF_CHECK_LAUNCH();
  }
  return TF_OK;
}

template <typename T, bool FWD, int MODE, bool TAIL>
static int attn_dispatch_tail(hipStream_t st, int hd, const AttnParams& p) {
  switch (hd) {
    case 32: return FWD ? fwd_launch<T, 32, MODE, TAIL>(st, p) : bwd_launch<T, 32, MODE, TAIL>(st, p);
    case 64: return FWD ? fwd_launch<T, 64, MODE, TAIL>(st, p) : bwd_launch<T, 64, MODE, TAIL>(st, p);
    case 128: return FWD ? fwd_launch<T, 128, MODE, TAIL>(st, p) : bwd_launch<T, 128, MODE, TAIL>(st, p);
  }
  return TF_ESHAPE;
}
template <typename T, bool FWD, int MODE>
static int attn_dispatch_hd(hipStream_t st, int hd, const AttnParams& p) {
  // a sequence that ends half way through its last 64-row block takes kernels of its own
  if (p.S % 64) return attn_dispatch_tail<T, FWD, MODE, true>(st, hd, p);
  return attn_dispatch_tail<T, FWD, MODE, false>(st, hd, p);
}

template <typename T, bool FWD>
static int attn_dispatch(hipStream_t st, int hd, const AttnParams& p) {
  if (p.slopes) return attn_dispatch_hd<T, FWD, kAlibi>(st, hd, p);
  if (p.bias) return attn_dispatch_hd<T, FWD, kDenseBias>(st, hd, p);
  return attn_dispatch_hd<T, FWD, kNoBias>(st, hd, p);
}

static int attn_check(int dtype, int64_t B, int64_t nh, int64_t S, int64_t hd, int64_t sb, int64_t sh, int64_t ss,
                      int64_t osb, int64_t osh, int64_t oss, const void* bias, int64_t bias_sh, int64_t bias_sr) {
  if (dtype != TF_F16 && dtype != TF_BF16) return TF_EDTYPE;
  if (B <= 0 || nh <= 0 || S <= 0) return TF_EINVAL;
  if (hd != 32 && hd != 64 && hd != 128) return TF_ESHAPE;  // as kernels/attention.py:567
  // 64-row blocks for every head_dim, the last one of a sequence half used when S = 32 (mod 64): the
  // reference (kernels/attention.py:177-183) uses 32-row blocks at head_dim 128 and so takes
  // S % 32 == 0 there; here every head_dim does
  if (S % 32 != 0) return TF_ESHAPE;
  if (B * nh * ((S + 127) / 128) > 0x7fffffff || S > (1 << 24)) return TF_EINVAL;
  if (sb % 8 || sh % 8 || ss % 8 || ss < hd) return TF_EALIGN;
  if (osb % 8 || osh % 8 || oss % 8 || oss < hd) return TF_EALIGN;
  if (bias && (bias_sh % 8 || bias_sr % 8 || bias_sr < S)) return TF_EALIGN;
  return TF_OK;
}

}  // namespace tfa

using namespace tfa;

static int attn_fwd_entry(void* stream, int dtype, int64_t B, int64_t nh, int64_t S, int64_t hd, const void* q,
                          const void* k, const void* v, void* o, int64_t sb, int64_t sh, int64_t ss, int64_t osb,
                          int64_t osh, int64_t oss, float* lse, const void* bias, int64_t bias_sh, int64_t bias_sr,
                          const void* slopes, float scale) {
  if (!q || !k || !v || !o || !lse) return TF_EINVAL;
  const int rc = attn_check(dtype, B, nh, S, hd, sb, sh, ss, osb, osh, oss, bias, bias_sh, bias_sr);
  if (rc != TF_OK) return rc;
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o)) return TF_EALIGN;
  if (bias && (reinterpret_cast<uintptr_t>(bias) & 15)) return TF_EALIGN;
  AttnParams p = {};
  p.q = q; p.k = k; p.v = v; p.out = o; p.lse = lse; p.bias = bias; p.slopes = slopes;
  p.sb = sb; p.sh = sh; p.ss = ss; p.osb = osb; p.osh = osh; p.oss = oss;
  p.bias_sh = bias_sh; p.bias_sr = bias_sr;
  p.B = (int)B; p.nh = (int)nh; p.S = (int)S;
  p.scale = scale; p.scale_log2 = scale * kLog2e;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == TF_F16) return attn_dispatch<f16, true>(st, (int)hd, p);
  return attn_dispatch<bf16, true>(st, (int)hd, p);
}

static int attn_bwd_entry(void* stream, int dtype, int64_t B, int64_t nh, int64_t S, int64_t hd, const void* q,
                          const void* k, const void* v, const void* o, const void* d_o, void* dq, void* dk, void* dv,
                          int64_t sb, int64_t sh, int64_t ss, int64_t osb, int64_t osh, int64_t oss, const float* lse,
                          float* delta, const void* bias, int64_t bias_sh, int64_t bias_sr, const void* slopes,
                          float scale) {
  if (!q || !k || !v || !o || !d_o || !dq || !dk || !dv || !lse || !delta) return TF_EINVAL;
  const int rc = attn_check(dtype, B, nh, S, hd, sb, sh, ss, osb, osh, oss, bias, bias_sh, bias_sr);
  if (rc != TF_OK) return rc;
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o) || !aligned16(d_o) || !aligned16(dq) ||
      !aligned16(dk) || !aligned16(dv))
    return TF_EALIGN;
  if (bias && (reinterpret_cast<uintptr_t>(bias) & 15)) return TF_EALIGN;
  AttnParams p = {};
  p.q = q; p.k = k; p.v = v; p.o = o; p.d_o = d_o; p.dq = dq; p.dk = dk; p.dv = dv;
  p.lse = const_cast<float*>(lse); p.delta = delta; p.bias = bias; p.slopes = slopes;
  p.sb = sb; p.sh = sh; p.ss = ss; p.osb = osb; p.osh = osh; p.oss = oss;
  p.bias_sh = bias_sh; p.bias_sr = bias_sr;
  p.B = (int)B; p.nh = (int)nh; p.S = (int)S;
  p.scale = scale; p.scale_log2 = scale * kLog2e;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == TF_F16) return attn_dispatch<f16, false>(st, (int)hd, p);
  return attn_dispatch<bf16, false>(st, (int)hd, p);
}

extern "C" int tf_attn_fwd(void* stream, int dtype, int64_t B, int64_t nh, int64_t S, int64_t hd, const void* q,
                           const void* k, const void* v, void* o, int64_t sb, int64_t sh, int64_t ss, int64_t osb,
                           int64_t osh, int64_t oss, float* lse, const void* bias, int64_t bias_sh, int64_t bias_sr,
                           float scale) {
  return attn_fwd_entry(stream, dtype, B, nh, S, hd, q, k, v, o, sb, sh, ss, osb, osh, oss, lse, bias, bias_sh, bias_sr,
                        nullptr, scale);
}

extern "C" int tf_attn_bwd(void* stream, int dtype, int64_t B, int64_t nh, int64_t S, int64_t hd, const void* q,
                           const void* k, const void* v, const void* o, const void* d_o, void* dq, void* dk, void* dv,
                           int64_t sb, int64_t sh, int64_t ss, int64_t osb, int64_t osh, int64_t oss,
                           const float* lse, float* delta, const void* bias, int64_t bias_sh, int64_t bias_sr,
                           float scale) {
  return attn_bwd_entry(stream, dtype, B, nh, S, hd, q, k, v, o, d_o, dq, dk, dv, sb, sh, ss, osb, osh, oss, lse, delta,
                        bias, bias_sh, bias_sr, nullptr, scale);
}

extern "C" int tf_attn_alibi_fwd(void* stream, int dtype, int64_t B, int64_t nh, int64_t S, int64_t hd, const void* q,
                                 const void* k, const void* v, void* o, int64_t sb, int64_t sh, int64_t ss,
                                 int64_t osb, int64_t osh, int64_t oss, float* lse, const void* slopes, float scale) {
  if (!slopes || (reinterpret_cast<uintptr_t>(slopes) & 1)) return TF_EINVAL;
  return attn_fwd_entry(stream, dtype, B, nh, S, hd, q, k, v, o, sb, sh, ss, osb, osh, oss, lse, nullptr, 0, 0, slopes,
                        scale);
}

extern "C" int tf_attn_alibi_bwd(void* stream, int dtype, int64_t B, int64_t nh, int64_t S, int64_t hd, const void* q,
                                 const void* k, const void* v, const void* o, const void* d_o, void* dq, void* dk,
                                 void* dv, int64_t sb, int64_t sh, int64_t ss, int64_t osb, int64_t osh, int64_t oss,
                                 const float* lse, float* delta, const void* slopes, float scale) {
  if (!slopes || (reinterpret_cast<uintptr_t>(slopes) & 1)) return TF_EINVAL;
  return attn_bwd_entry(stream, dtype, B, nh, S, hd, q, k, v, o, d_o, dq, dk, dv, sb, sh, ss, osb, osh, oss, lse, delta,
                        nullptr, 0, 0, slopes, scale);
}
