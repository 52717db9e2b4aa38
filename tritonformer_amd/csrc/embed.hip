// Token (+ position) embedding for gfx950: forward gather-add with the rounding to the
// compute type folded in, backward as a deterministic scatter-add.  HBM-bound row kernels.
//
// Backward without floating-point atomics and without a sort: positions that hold the same
// token id are linked into chains in increasing order (next[t] = next position with ids[t]),
// and the first position of every chain sums its chain's gradient rows in that order and
// writes the vocabulary row once; every other row of the gradient is zero-filled.  The links
// come from a brute-force scan, T^2 / 2 integer compares: every lane keeps its own id in a
// register and the candidates arrive as wave-uniform (scalar) loads, two VALU instructions
// per candidate and wave; the candidate range is cut into segments that run as separate
// workgroups and meet in an integer atomicMin, whose result does not depend on their order.
#include <climits>
#include "rowops.h"

namespace tfa {


// out[t, :] = tok[ids[t], :] + pos[t % S, :], added in fp32, rounded once.  One row per
// `LPR` lanes; ids outside [0, V) give a row of zeros.
template <typename TP, typename TO, bool VEC>
__global__ __launch_bounds__(256) void embed_fwd(int64_t T, int S, int d, int64_t V, const int64_t* __restrict__ ids,
                                                 const TP* __restrict__ tok, int64_t ld_tok, const TP* __restrict__ pos,
                                                 int64_t ld_pos, TO* __restrict__ out, int64_t ld_out, int lpr) {
  const int rows_per_block = 256 / lpr;
  const int64_t t = (int64_t)blockIdx.x * rows_per_block + threadIdx.x / lpr;
  if (t >= T) return;
  const int l = threadIdx.x % lpr;
  const int64_t id = ids[t];
  const bool ok = id >= 0 && id < V;
  const TP* trow = tok + (ok ? id : 0) * ld_tok;
  const TP* prow = pos ? pos + (t % S) * ld_pos : nullptr;
  TO* orow = out + t * ld_out;
  if constexpr (VEC) {
    for (int c = l * 8; c < d; c += lpr * 8) {
      float a[8], b[8];
      load8<TP>(trow + c, a);
      if (prow) {
        load8<TP>(prow + c, b);
#pragma unroll
        for (int e = 0; e < 8; ++e) a[e] += b[e];
      }
      if (!ok) {
#pragma unroll
        for (int e = 0; e < 8; ++e) a[e] = 0.f;
      }
      if constexpr (sizeof(TO) == 2) {
        Chunk<TO>::store(orow + c, a);
      } else {
        // two 16-byte halves per lane: half lines per instruction, so plain (write-back) stores
        const f32x4 lo = {a[0], a[1], a[2], a[3]}, hi = {a[4], a[5], a[6], a[7]};
        *reinterpret_cast<f32x4*>((float*)orow + c) = lo;
        *reinterpret_cast<f32x4*>((float*)orow + c + 4) = hi;
      }
    }
  } else {
    for (int c = l; c < d; c += lpr) {
      float a = ok ? (float)trow[c] : 0.f;
      if (ok && prow) a += (float)prow[c];
      orow[c] = (TO)a;
    }
  }
}

// Zero fill of the token-gradient matrix (16-byte stores, then its last `tail` (< 16, even) bytes
// two at a time) and initial state of the chain arrays: next = INT_MAX, has_prev = 0.
__global__ __launch_bounds__(256) void embed_init(u32x4* __restrict__ a, int64_t na, int tail, int* __restrict__ next,
                                                  int* __restrict__ has_prev, int T) {
  const u32x4 z = {0u, 0u, 0u, 0u};
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  const int64_t first = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  for (int64_t i = first; i < na; i += stride) a[i] = z;
  if (first < tail / 2) reinterpret_cast<unsigned short*>(a + na)[first] = 0;
  for (int64_t i = first; i < T; i += stride) {
    next[i] = INT_MAX;
    has_prev[i] = 0;
  }
}

// next[t] = min(next[t], smallest c in this workgroup's candidate segment with c > t and
// ids[c] == ids[t]).  grid (T / 256 position blocks, segments).  Positions whose id lies
// outside [0, V) take part in no chain.
__global__ __launch_bounds__(256) void embed_chain(int T, int64_t V, const int64_t* __restrict__ ids, int* __restrict__ next,
                                                   int seg_len) {
  const int t = blockIdx.x * 256 + threadIdx.x;
  int c_begin = blockIdx.y * seg_len, c_end = min(T, c_begin + seg_len);
  c_begin = max(c_begin, (int)blockIdx.x * 256 + 1);
  if (c_begin >= c_end) return;
  int64_t mine = -1;
  if (t < T) {
    const int64_t id = ids[t];
    if (id >= 0 && id < V) mine = id;
  }
  int best = INT_MAX;
#pragma unroll 8
  for (int c = c_begin; c < c_end; ++c) {
    const int64_t cand = ids[c];  // the same address in every lane: a scalar load
    if (cand == mine && c > t) best = min(best, c);
  }
  if (mine >= 0 && best != INT_MAX) atomicMin(&next[t], best);
}

// has_prev[next[t]] = 1: every position has at most one predecessor, so no two threads write
// the same flag.
__global__ __launch_bounds__(256) void embed_mark(int T, const int* __restrict__ next, int* __restrict__ has_prev) {
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (t < T && next[t] < T) has_prev[next[t]] = 1;
}

// Workgroups [0, tok_blocks): the first position of every chain sums the gradient rows of its
// chain (fp32, in increasing position order) into the row of its token.  Workgroups after
// them: d_pos[s, :] = sum over sequences of g[b*S + s, :] for s < S, zero for S <= s < P.
template <typename TG, typename TP, bool VEC>
__global__ __launch_bounds__(256) void embed_bwd(int T, int S, int d, int P, int64_t V, const int64_t* __restrict__ ids,
                                                 const int* __restrict__ next, const int* __restrict__ has_prev,
                                                 const TG* __restrict__ g, int64_t ld_g, TP* __restrict__ d_tok, int64_t ld_dtok,
                                                 TP* __restrict__ d_pos, int64_t ld_dpos, int lpr, int tok_blocks) {
  const int rows_per_block = 256 / lpr;
  const int l = threadIdx.x % lpr;
  const bool token_part = (int)blockIdx.x < tok_blocks;
  const int row = ((int)blockIdx.x - (token_part ? 0 : tok_blocks)) * rows_per_block + threadIdx.x / lpr;
  TP* dst;
  int first, step, count;  // gradient rows first, first + step, ... (position part) or the chain from `first`
  if (token_part) {
    if (row >= T || has_prev[row]) return;
    const int64_t id = ids[row];
    if (id < 0 || id >= V) return;  // no row to write to (the chain scan gave such positions no chain either)
    dst = d_tok + id * ld_dtok;
    first = row; step = 0; count = 0;
  } else {
    if (row >= P) return;
    dst = d_pos + (int64_t)row * ld_dpos;
    first = row; step = S; count = row < S ? T / S : 0;
  }
  constexpr int W = VEC ? 8 : 1;
  for (int c = l * W; c < d; c += lpr * W) {
    float acc[W];
#pragma unroll
    for (int e = 0; e < W; ++e) acc[e] = 0.f;
    auto add_row = [&](int r) {
      if constexpr (VEC) {
        float v[8];
        load8<TG>(g + (int64_t)r * ld_g + c, v);
#pragma unroll
        for (int e = 0; e < W; ++e) acc[e] += v[e];
      } else {
        acc[0] += (float)g[(int64_t)r * ld_g + c];
      }
    };
    if (token_part) {
      for (int r = first; r < T; r = next[r]) add_row(r);
    } else {
      for (int k = 0; k < count; ++k) add_row(first + k * step);
    }
    if constexpr (VEC) {
      if constexpr (sizeof(TP) == 2) {
        Chunk<TP>::store(dst + c, acc);
      } else {
        // two 16-byte halves per lane: half lines per instruction, so plain (write-back) stores
        const f32x4 lo = {acc[0], acc[1], acc[2], acc[3]}, hi = {acc[4], acc[5], acc[6], acc[7]};
        *reinterpret_cast<f32x4*>((float*)dst + c) = lo;
        *reinterpret_cast<f32x4*>((float*)dst + c + 4) = hi;
      }
    } else {
      dst[c] = (TP)acc[0];
    }
  }
}

static int lanes_per_row(int64_t d, bool vec) {
  const int64_t work = vec ? d / 8 : d;
  int lpr = 1;
  while (lpr < 256 && lpr < work) lpr *= 2;
  return lpr;
}

template <typename TP, typename TO>
static int embed_fwd_launch(hipStream_t st, int64_t T, int64_t S, int64_t d, int64_t V, const int64_t* ids, const void* tok,
                            int64_t ld_tok, const void* pos, int64_t ld_pos, void* out, int64_t ld_out) {
  const bool vec = row_vectorizable<TP>(tok, d, ld_tok) && (!pos || row_vectorizable<TP>(pos, d, ld_pos)) &&
                   row_vectorizable<TO>(out, d, ld_out) && d % 8 == 0;
  const int lpr = lanes_per_row(d, vec);
  const int64_t blocks = (T + 256 / lpr - 1) / (256 / lpr);
  if (vec)
    embed_fwd<TP, TO, true><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(T, (int)S, (int)d, V, ids, (const TP*)tok, ld_tok,
                                                                         (const TP*)pos, ld_pos, (TO*)out, ld_out, lpr);
  else
    embed_fwd<TP, TO, false><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(T, (int)S, (int)d, V, ids, (const TP*)tok, ld_tok,
                                                                          (const TP*)pos, ld_pos, (TO*)out, ld_out, lpr);
  TF_CHECK_LAUNCH();
  return TF_OK;
}

template <typename TG, typename TP>
static int embed_bwd_launch(hipStream_t st, int64_t T, int64_t S, int64_t d, int64_t V, int64_t P, const int64_t* ids,
                            const void* g, int64_t ld_g, void* d_tok, int64_t ld_dtok, void* d_pos, int64_t ld_dpos,
                            int* next, int* has_prev) {
  // zero fill of the whole token-gradient matrix (rows are contiguous here, checked by the caller), chain state
  const int64_t tok_bytes = V * d * (int64_t)sizeof(TP);
  embed_init<<<dim3(2048), dim3(256), 0, st>>>((u32x4*)d_tok, tok_bytes / 16, (int)(tok_bytes % 16), next, has_prev, (int)T);
  TF_CHECK_LAUNCH();
  const int pos_blocks256 = (int)((T + 255) / 256);
  const int segments = (int)(T >= 4096 ? 16 : (T + 255) / 256);  // enough workgroups to fill the chip at the sizes that matter
  const int seg_len = (int)((T + segments - 1) / segments);
  embed_chain<<<dim3((unsigned)pos_blocks256, (unsigned)segments), dim3(256), 0, st>>>((int)T, V, ids, next, seg_len);
  TF_CHECK_LAUNCH();
  embed_mark<<<dim3((unsigned)pos_blocks256), dim3(256), 0, st>>>((int)T, next, has_prev);
  TF_CHECK_LAUNCH();
  const bool vec = row_vectorizable<TG>(g, d, ld_g) && row_vectorizable<TP>(d_tok, d, ld_dtok) &&
                   (!d_pos || row_vectorizable<TP>(d_pos, d, ld_dpos)) && d % 8 == 0;
  const int lpr = lanes_per_row(d, vec);
  const int rpb = 256 / lpr;
  const int tok_blocks = (int)((T + rpb - 1) / rpb);
  const int pos_blocks = d_pos ? (int)((P + rpb - 1) / rpb) : 0;
  if (vec)
    embed_bwd<TG, TP, true><<<dim3((unsigned)(tok_blocks + pos_blocks)), dim3(256), 0, st>>>(
        (int)T, (int)S, (int)d, (int)P, V, ids, next, has_prev, (const TG*)g, ld_g, (TP*)d_tok, ld_dtok, (TP*)d_pos, ld_dpos, lpr,
        tok_blocks);
  else
    embed_bwd<TG, TP, false><<<dim3((unsigned)(tok_blocks + pos_blocks)), dim3(256), 0, st>>>(
        (int)T, (int)S, (int)d, (int)P, V, ids, next, has_prev, (const TG*)g, ld_g, (TP*)d_tok, ld_dtok, (TP*)d_pos, ld_dpos, lpr,
        tok_blocks);
  TF_CHECK_LAUNCH();
  return TF_OK;
}

static int embed_check(int64_t T, int64_t S, int64_t d, int64_t V, int64_t P, bool has_pos) {
  if (T <= 0 || S <= 0 || d <= 0 || V <= 0) return TF_EINVAL;
  if (T % S != 0) return TF_ESHAPE;             // whole sequences: position = t mod S
  if (has_pos && P < S) return TF_ESHAPE;       // as nn.Embedding would fail on positions >= P
  if (T > INT_MAX / 2 || V > INT_MAX || d > INT_MAX / 2 || P > INT_MAX / 2) return TF_EINVAL;
  return TF_OK;
}

}  // namespace tfa

using namespace tfa;

extern "C" int tf_embedding_fwd(void* stream, int param_dtype, int out_dtype, int64_t T, int64_t S, int64_t d, int64_t V,
                                int64_t P, const int64_t* ids, const void* tok, int64_t ld_tok, const void* pos,
                                int64_t ld_pos, void* out, int64_t ld_out) {
  if (!ids || !tok || !out) return TF_EINVAL;
  const int rc = embed_check(T, S, d, V, P, pos != nullptr);
  if (rc != TF_OK) return rc;
  if (ld_tok < d || (pos && ld_pos < d) || ld_out < d) return TF_EINVAL;
  hipStream_t st = (hipStream_t)stream;
#define GO(TP, TO) return embed_fwd_launch<TP, TO>(st, T, S, d, V, ids, tok, ld_tok, pos, ld_pos, out, ld_out)
  if (param_dtype == TF_F32) {
    if (out_dtype == TF_F32) GO(float, float);
    if (out_dtype == TF_F16) GO(float, f16);
    if (out_dtype == TF_BF16) GO(float, bf16);
  } else if (param_dtype == TF_F16 && out_dtype == TF_F16) {
    GO(f16, f16);
  } else if (param_dtype == TF_BF16 && out_dtype == TF_BF16) {
    GO(bf16, bf16);
  }
#undef GO
  return TF_EDTYPE;
}

extern "C" int64_t tf_embedding_bwd_workspace_bytes(int64_t T) { return T > 0 ? 2 * ((T * 4 + 15) / 16 * 16) : 0; }

extern "C" int tf_embedding_bwd(void* stream, int grad_dtype, int param_dtype, int64_t T, int64_t S, int64_t d, int64_t V,
                                int64_t P, const int64_t* ids, const void* g, int64_t ld_g, void* d_tok, int64_t ld_dtok,
                                void* d_pos, int64_t ld_dpos, void* workspace, int64_t workspace_bytes) {
  if (!ids || !g || !d_tok) return TF_EINVAL;
  const int rc = embed_check(T, S, d, V, P, d_pos != nullptr);
  if (rc != TF_OK) return rc;
  if (ld_g < d || (d_pos && ld_dpos < d)) return TF_EINVAL;
  if (ld_dtok != d) return TF_EINVAL;  // the zero fill takes the token gradient as one contiguous block
  if (!aligned16(d_tok)) return TF_EALIGN;
  if (!workspace || workspace_bytes < tf_embedding_bwd_workspace_bytes(T) || !aligned16(workspace)) return TF_EWORKSPACE;
  int* next = (int*)workspace;
  int* has_prev = (int*)((char*)workspace + (T * 4 + 15) / 16 * 16);
  hipStream_t st = (hipStream_t)stream;
#define GO(TG, TP) \
  return embed_bwd_launch<TG, TP>(st, T, S, d, V, P, ids, g, ld_g, d_tok, ld_dtok, d_pos, ld_dpos, next, has_prev)
  if (param_dtype == TF_F32) {
    if (grad_dtype == TF_F32) GO(float, float);
    if (grad_dtype == TF_F16) GO(f16, float);
    if (grad_dtype == TF_BF16) GO(bf16, float);
  } else if (param_dtype == TF_F16 && grad_dtype == TF_F16) {
    GO(f16, f16);
  } else if (param_dtype == TF_BF16 && grad_dtype == TF_BF16) {
    GO(bf16, bf16);
  }
#undef GO
  return TF_EDTYPE;
}
