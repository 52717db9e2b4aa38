/*
 * tritonformer_amd.h — C ABI of libtritonformer_amd.so (gfx950 / MI355X).
 *
 * The reference (fattorib/tritonformer) has no FFI: its boundary is a set of
 * Python launcher functions under tritonformer/kernels/ that take torch tensors
 * and start Triton kernels on the current stream.  Each entry point below
 * replaces one (or a fused group) of those launchers and is what a ctypes
 * binding on the reference side would call.
 *
 * Conventions
 *  - every pointer is a DEVICE pointer unless said otherwise; the library
 *    never allocates, frees, retains or synchronises; it reads no environment
 *    variable.  What it keeps between calls: the device's CU / XCD counts (read
 *    from the runtime once per device), the address of the scratch array of
 *    tf_colsum_noalloc (taken once per device), and a counter of GEMM launches
 *    (a relaxed atomic that only tf_diag_gemm_launch_count reads); no result
 *    depends on any of them beyond tile choice.  Work is enqueued on
 *    `stream` (a hipStream_t passed as void*, NULL = the null stream);
 *  - strides and leading dimensions are in ELEMENTS, sizes in elements;
 *  - `dtype`: TF_F16 / TF_BF16 for the 16-bit paths, TF_F32 only where stated;
 *  - return value: TF_OK (0) or a negative TF_E* code; tf_status_string()
 *    gives the text.  Argument checks run on the host before any launch, so a
 *    non-zero status means nothing was enqueued.
 */
#ifndef TRITONFORMER_AMD_H
#define TRITONFORMER_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum tf_dtype { TF_F16 = 0, TF_BF16 = 1, TF_F32 = 2 };

enum tf_status {
  TF_OK = 0,
  TF_EINVAL = -1,    /* bad size / null pointer / unsupported combination   */
  TF_EDTYPE = -2,    /* dtype not supported by this entry point             */
  TF_EALIGN = -3,    /* pointer or stride violates a stated alignment rule  */
  TF_ESHAPE = -4,    /* shape precondition of the reference violated        */
  TF_EWORKSPACE = -5,/* workspace missing or too small                      */
  TF_ELAUNCH = -6    /* the HIP runtime refused the launch                  */
};

/* Operand storage for tf_gemm.  "K" is the contraction dimension.
 *   TF_OP_KMAJOR : element (row, k) at  ptr[row * ld + k]   (k contiguous)
 *   TF_OP_KMINOR : element (row, k) at  ptr[k * ld + row]   (row contiguous)
 * where "row" is m for A and n for B. */
enum tf_op_layout { TF_OP_KMAJOR = 0, TF_OP_KMINOR = 1 };

const char* tf_status_string(int status);
int tf_version(void);
/* Hash of the source files this binary was built from ("" for a build that did not record
 * one); the Python loader refuses a library whose hash differs from the sources beside it. */
const char* tf_source_hash(void);
/* Compute units and XCDs of the current HIP device as the library sees them (read from the
 * runtime once per device; tile choice and the workgroup-id remap of the GEMM kernels use them).
 * The reference has no counterpart: Triton reads the device through its own driver layer. */
int tf_device_info(int* cus, int* xcds);

/* ---- dense contractions (fp16/bf16 MFMA, fp32 accumulate) --------------- */

/* C[M,N] = epilogue( sum_k A(m,k) * B(n,k) ),  epilogue = (+bias[n]) then
 * optional max(.,0), rounded once to `dtype`.
 * Replaces mm / gemm / bmm (+ the torch.sum over the batch that follows bmm):
 *   tritonformer/kernels/gemm.py:361-401 (mm, optional ReLU)
 *   tritonformer/kernels/gemm.py:572-616 (gemm: bias, optional ReLU)
 *   tritonformer/kernels/gemm.py:161-200 (bmm) + tritonformer/linear.py:24-25
 * Forward      Y = X W      : A = X  KMAJOR (M=B*S, K=in),  B = W  KMINOR.
 * Input grad   dX = dY W^T  : A = dY KMAJOR (K=out),        B = W  KMAJOR.
 * Weight grad  dW = X^T dY  : A = X  KMINOR (M=in, K=B*S),  B = dY KMINOR;
 *   the batch dimension is part of the contraction, so no (B,in,out)
 *   temporary exists.
 * `workspace` (fp32, tf_gemm_workspace_bytes() bytes) is needed only when that
 * query returns non-zero (contraction split over several workgroups, summed in
 * a fixed order by a second kernel: results are bitwise reproducible).
 * Fast path needs 16-byte aligned pointers and contiguous-dimension extents
 * and leading dimensions that are multiples of 8; anything else takes a
 * slower element-wise-load path with identical arithmetic. */
int tf_gemm(void* stream, int dtype, int layout_a, int layout_b,
            int64_t M, int64_t N, int64_t K,
            const void* A, int64_t lda, const void* B, int64_t ldb,
            void* C, int64_t ldc, const void* bias, int relu,
            void* workspace, int64_t workspace_bytes);
/* As tf_gemm with two extras.
 * `out_dtype`: C is stored as `dtype` or as TF_F32 (fp32 weight gradients for
 * fp32 master weights, skipping the separate 16->32 bit cast pass autograd would
 * otherwise run; the reference keeps fp16 parameters and has no such case).
 * `mask_act` (NULL, or an (M, N) matrix of `dtype`, leading dimension ld_mask):
 * C[m,n] is zeroed where mask_act[m,n] <= 0 -- the ReLU gradient mask of
 * kernels/activation.py:27-44 applied while the input gradient of the following
 * layer is written, instead of in a pass of its own; excludes bias and relu,
 * and such a call never splits the contraction (no workspace needed). */
int tf_gemm_out(void* stream, int dtype, int out_dtype, int layout_a, int layout_b,
                int64_t M, int64_t N, int64_t K,
                const void* A, int64_t lda, const void* B, int64_t ldb,
                void* C, int64_t ldc, const void* bias, int relu,
                const void* mask_act, int64_t ld_mask,
                void* workspace, int64_t workspace_bytes);
/* As tf_gemm_out, with C split into N / chunk_n column blocks that are separate
 * (M, chunk_n) matrices of leading dimension ldc, `chunk_stride` elements apart:
 * element (m, n) is stored at C[(n / chunk_n) * chunk_stride + m * ldc + n % chunk_n].
 * Used for the weight gradient of the q, k and v projections computed as ONE
 * product x^T . d(qkv) (the three dW products of tritonformer/linear.py:25 for
 * transformer.py:158-160): every projection gets its own contiguous gradient.
 * chunk_n = 0 means one matrix; otherwise chunk_n divides N and chunk_n,
 * chunk_stride are multiples of 8. */
int tf_gemm_out_chunked(void* stream, int dtype, int out_dtype, int layout_a, int layout_b,
                        int64_t M, int64_t N, int64_t K,
                        const void* A, int64_t lda, const void* B, int64_t ldb,
                        void* C, int64_t ldc, int64_t chunk_n, int64_t chunk_stride,
                        const void* bias, int relu, const void* mask_act, int64_t ld_mask,
                        void* workspace, int64_t workspace_bytes);
/* tf_gemm_out with the ReLU mask carried as one bit per element instead of the
 * activation itself.  Exactly one of bits_out / bits_in is given; rows of ld_bits
 * bytes (>= N / 8, N a multiple of 8), element (m, n) is bit n % 8 of byte n / 8.
 *   bits_out: C = relu(A . B + bias) in the operand dtype, bits_out = (C > 0)
 *             (the forward of LinearNoBiasReLU / LinearBiasReLU, tritonformer/linear.py:47-102);
 *   bits_in:  C = bit ? A . B : 0, no bias (mask_grad of kernels/activation.py:27-44
 *             fused into dH = dY . W2^T, reading a sixteenth of what the activation holds).
 * Served by the write-out of the direct-to-LDS kernels only: returns TF_ESHAPE (and
 * launches nothing) when their preconditions (16-byte aligned operands, extents and
 * leading dimensions multiples of 8, K a multiple of 64, a product large enough to run
 * unsplit) do not hold; callers then use tf_gemm_out with the activation as mask_act.
 * Malformed calls get the other codes as everywhere.  Needs no workspace. */
int tf_gemm_relu_bits(void* stream, int dtype, int out_dtype, int layout_a, int layout_b,
                      int64_t M, int64_t N, int64_t K,
                      const void* A, int64_t lda, const void* B, int64_t ldb,
                      void* C, int64_t ldc, const void* bias,
                      void* bits_out, const void* bits_in, int64_t ld_bits);
int64_t tf_gemm_workspace_bytes(int layout_a, int layout_b, int64_t M, int64_t N, int64_t K);
/* C = alpha * (A . B), no bias / ReLU / mask; `alpha`: ONE fp32 value in DEVICE memory, read by
 * the kernel when it writes its result (applied to the fp32 sums before the rounding to
 * out_dtype).  For a factor that is itself computed on the GPU: the upstream gradient of the mean
 * loss divided by the number of rows, which tritonformer/crossentropy.py:24 multiplies into the
 * (N, V) logits gradient in a pass of its own before the two LM-head gradient products
 * (transformer.py:330-343) -- here those products take the unscaled gradient and the factor.
 * Other arguments and the workspace rule as tf_gemm_out. */
int tf_gemm_scaled(void* stream, int dtype, int out_dtype, int layout_a, int layout_b,
                   int64_t M, int64_t N, int64_t K,
                   const void* A, int64_t lda, const void* B, int64_t ldb,
                   void* C, int64_t ldc, const float* alpha,
                   void* workspace, int64_t workspace_bytes);

/* `count` (1..16) independent products of one dtype and one pair of operand layouts,
 * no bias / ReLU / mask, each with the arguments of tf_gemm_out_chunked.  When every
 * problem meets the fast-path preconditions and both operands are TF_OP_KMINOR (the
 * weight-gradient form x^T . dy of tritonformer/linear.py:24-25), all of them run in
 * ONE launch: outputs with few tiles (two MLP weights: 64 tiles each) then fill the
 * GPU side by side, with half as many contraction slices and fp32 partials as two
 * launches would need; products whose tiles together make whole rounds of one workgroup
 * per CU (the weight gradients of several layers, handed over together) run unsplit.
 * Otherwise the problems run one after the other.  The results do not depend on which
 * of the two happens beyond the fp32 summation order. */
typedef struct tf_gemm_problem {
  int64_t M, N, K;
  const void* A; int64_t lda;
  const void* B; int64_t ldb;
  void* C; int64_t ldc;
  int64_t chunk_n, chunk_stride;   /* 0, 0: one output matrix */
} tf_gemm_problem;
int tf_gemm_group(void* stream, int dtype, int out_dtype, int layout_a, int layout_b, int count,
                  const tf_gemm_problem* problems, void* workspace, int64_t workspace_bytes);
int64_t tf_gemm_group_workspace_bytes(int layout_a, int layout_b, int count,
                                      const tf_gemm_problem* problems);
/* Causal flash attention forward.  q, k, v: logical (B, nh, S, hd) sharing the
 * element strides {sb, sh, ss}; o: the same logical shape with its own strides
 * {osb, osh, oss}; unit stride along hd everywhere.  (The reference passes q's
 * strides for all four, kernels/attention.py:202-205; separate output strides
 * also serve q, k, v that are slices of one packed (B, S, 3, nh, hd) buffer.)
 * lse: (B, nh, S) fp32, contiguous, log2-domain log-sum-exp of the scaled
 * (and biased) scores.  bias: NULL, or (nh, Sb, Sb) with Sb >= S, element
 * strides {bias_sh, bias_sr} that are multiples of 8, 16-byte aligned, unit stride
 * along keys, added after scaling
 * (kernels/biased_attention.py:101-106); -inf entries are allowed.
 * Replaces flash_wrapper_fwd (kernels/attention.py:171-217) and
 * flash_wrapper_fwd_attn_bias (kernels/biased_attention.py:188-245).
 * Preconditions: hd in {32,64,128} (as the reference asserts); S % 32 == 0.  The reference
 * asserts S % 64 == 0, except at hd = 128, where its 32-row blocks admit S % 32 == 0
 * (kernels/attention.py:177-183); here every head_dim takes S % 32 == 0 (64-row blocks, the
 * last one of a sequence half used).  Nothing beyond row S - 1 of q, k, v, o, lse or of the
 * bias rows is read or written. */
int tf_attn_fwd(void* stream, int dtype, int64_t B, int64_t nh, int64_t S, int64_t hd,
                const void* q, const void* k, const void* v, void* o,
                int64_t sb, int64_t sh, int64_t ss, int64_t osb, int64_t osh, int64_t oss,
                float* lse, const void* bias, int64_t bias_sh, int64_t bias_sr,
                float scale);

/* Backward of the above: dq, dk, dv have q's strides, o and d_o the output
 * strides.  delta: (B, nh, S) fp32 scratch (negated row sums of dO*O), written then
 * read by this call.
 * Replaces flash_wrapper_bwd (kernels/attention.py:550-607) and
 * flash_wrapper_bwd_attn_bias (kernels/biased_attention.py:598-660).
 * No gradient is produced for the bias (tritonformer/attention.py:60). */
int tf_attn_bwd(void* stream, int dtype, int64_t B, int64_t nh, int64_t S, int64_t hd,
                const void* q, const void* k, const void* v, const void* o, const void* d_o,
                void* dq, void* dk, void* dv,
                int64_t sb, int64_t sh, int64_t ss, int64_t osb, int64_t osh, int64_t oss,
                const float* lse, float* delta,
                const void* bias, int64_t bias_sh, int64_t bias_sr, float scale);

/* tf_attn_fwd / tf_attn_bwd with the ALiBi bias of the reference's model in closed form
 * instead of the dense (nh, S, S) matrix that generate_alibi_mask builds
 * (transformer.py:37-75, 296-302; 805 MB at 24 heads x 4096): `slopes` = nh fp16 values
 * (device memory), bias(h, i, j) = fp16(fp16(j - i) * slopes[h]) for j <= i -- distance,
 * slope and product rounded to fp16 exactly as in that matrix, and the result rounded to
 * bf16 when dtype is TF_BF16 (the matrix cast to the compute type) -- so the results are
 * bit-identical to the dense calls on that matrix.  Other arguments as above. */
int tf_attn_alibi_fwd(void* stream, int dtype, int64_t B, int64_t nh, int64_t S, int64_t hd,
                      const void* q, const void* k, const void* v, void* o,
                      int64_t sb, int64_t sh, int64_t ss, int64_t osb, int64_t osh, int64_t oss,
                      float* lse, const void* slopes, float scale);
int tf_attn_alibi_bwd(void* stream, int dtype, int64_t B, int64_t nh, int64_t S, int64_t hd,
                      const void* q, const void* k, const void* v, const void* o, const void* d_o,
                      void* dq, void* dk, void* dv,
                      int64_t sb, int64_t sh, int64_t ss, int64_t osb, int64_t osh, int64_t oss,
                      const float* lse, float* delta, const void* slopes, float scale);

/* ---- bandwidth-bound kernels -------------------------------------------- */

/* y = gamma * (x - mean) * rstd + beta over the last dimension; biased
 * variance, rstd = 1/sqrt(var + eps), statistics in fp32
 * (kernels/layernorm.py:8-61, launcher :64-87).  mean/rstd: (rows) fp32, saved
 * for the backward pass (the reference recomputes them instead).
 * gamma, beta (and dgamma, dbeta below) have `param_dtype`: `dtype`, or TF_F32
 * for fp32 master parameters used as they are. */
int tf_layernorm_fwd(void* stream, int dtype, int param_dtype, int64_t rows, int64_t d,
                     const void* x, int64_t ldx, const void* gamma, const void* beta,
                     float eps, void* y, int64_t ldy, float* mean, float* rstd);

/* dx, dgamma, dbeta in one pass over (dy, x) plus a small second-stage
 * reduction.  Replaces dx_layernorm (kernels/layernorm.py:140-162) and
 * layernorm_da_db (kernels/layernorm.py:226-259, with its reductions.py
 * second stage).  partial: fp32 scratch of tf_layernorm_bwd_partial_bytes(). */
int tf_layernorm_bwd(void* stream, int dtype, int param_dtype, int64_t rows, int64_t d,
                     const void* dy, int64_t lddy, const void* x, int64_t ldx,
                     const void* gamma, const float* mean, const float* rstd,
                     void* dx, int64_t lddx, void* dgamma, void* dbeta,
                     float* partial, int64_t partial_bytes);
int64_t tf_layernorm_bwd_partial_bytes(int64_t rows, int64_t d);

/* The second stage by itself, for the LayerNorms of a whole backward pass at once.
 * tf_layernorm_bwd / tf_add_layernorm_bwd called with dgamma = dbeta = NULL write dx and
 * leave the column sums of their row blocks in `partial`: tf_layernorm_bwd_parts(rows)
 * rows of 2*d fp32 values (d of dgamma, then d of dbeta).  tf_layernorm_param_grads sums
 * the rows of `count` such buffers (any count; one launch per 64) in the order the
 * one-call form sums them -- the same bits -- into dgamma / dbeta of `param_dtype`.
 * Stands where the reference launches its reductions.py second stage once per LayerNorm
 * (kernels/layernorm.py:226-259). */
typedef struct tf_ln_param_grads {
  const float* partial;
  int64_t parts;
  void* dgamma;
  void* dbeta;
} tf_ln_param_grads;
int64_t tf_layernorm_bwd_parts(int64_t rows);
int tf_layernorm_param_grads(void* stream, int param_dtype, int64_t d, int count,
                             const tf_ln_param_grads* items);

/* Residual addition fused into the LayerNorm that follows it:
 *   sum = x + res (rounded to `dtype`, written out),  y = layernorm(sum).
 * One kernel for the reference model's `hidden_states = residual + hidden_states`
 * followed by the next LayerNorm (transformer.py:245-249, and :250 with the next
 * layer's :243 or the final LayerNorm at :327); the results equal
 * an elementwise addition followed by tf_layernorm_fwd bit for bit.
 * The backward adds dsum, the gradient reaching `sum` along the residual
 * stream, to the LayerNorm's own dx in fp32 before rounding: dx is the gradient
 * of both x and res.  `x` of the backward is the saved `sum`. */
int tf_add_layernorm_fwd(void* stream, int dtype, int param_dtype, int64_t rows, int64_t d,
                         const void* x, int64_t ldx, const void* res, int64_t ldres,
                         void* sum, int64_t ldsum, const void* gamma, const void* beta,
                         float eps, void* y, int64_t ldy, float* mean, float* rstd);
int tf_add_layernorm_bwd(void* stream, int dtype, int param_dtype, int64_t rows, int64_t d,
                         const void* dy, int64_t lddy, const void* dsum, int64_t lddsum,
                         const void* x, int64_t ldx, const void* gamma,
                         const float* mean, const float* rstd,
                         void* dx, int64_t lddx, void* dgamma, void* dbeta,
                         float* partial, int64_t partial_bytes);

/* dst[r, j*cols + c] = (dst_dtype) srcs[j][r*ld_src + c] for j < count (count <= 4):
 * `count` (rows, cols) matrices of src_dtype (TF_F32, or dst_dtype) converted to
 * 16 bits and laid side by side in one (rows, count*cols) matrix, one launch.
 * Builds the 16-bit (d, 3d) operand of the packed q/k/v projection from the three
 * master weights; stands for the three per-parameter casts torch.autocast makes
 * for the reference's three projections (transformer.py:158-160).
 * `srcs`: HOST array of `count` device pointers. */
int tf_cast_pack(void* stream, int src_dtype, int dst_dtype, int count, int64_t rows, int64_t cols,
                 const void* const* srcs, int64_t ld_src, void* dst, int64_t ld_dst);

/* Token (+ position) embedding, the part of the model the reference leaves to
 * nn.Embedding (transformer.py:259-272, 311-323): out[t, :] = tok[ids[t], :] +
 * pos[t mod S, :] for t < T (T = B*S whole sequences; `pos` may be null), added in
 * fp32 and rounded once to out_dtype.  param_dtype TF_F32 with any out_dtype, or a
 * 16-bit param_dtype with the same out_dtype.  tok is (V, d), pos (P, d), P >= S.
 * An id outside [0, V) gives a row of zeros. */
int tf_embedding_fwd(void* stream, int param_dtype, int out_dtype, int64_t T, int64_t S, int64_t d,
                     int64_t V, int64_t P, const int64_t* ids, const void* tok, int64_t ld_tok,
                     const void* pos, int64_t ld_pos, void* out, int64_t ld_out);

/* Its backward: d_tok (V, d; contiguous, ld_dtok == d) = scatter-add of the rows of
 * g (T, d) by token id, every other row zero; d_pos (P, d; may be null) = sum over
 * sequences of g[b*S + s, :] for s < S, zero below.  fp32 accumulation in increasing
 * position order, no atomics: bitwise reproducible.  Outputs are of param_dtype;
 * grad_dtype any with TF_F32 parameters, else equal to param_dtype.  Gradient rows
 * whose id lies outside [0, V) are dropped.  `workspace`: device memory of
 * tf_embedding_bwd_workspace_bytes(T), 16-byte aligned. */
int64_t tf_embedding_bwd_workspace_bytes(int64_t T);
int tf_embedding_bwd(void* stream, int grad_dtype, int param_dtype, int64_t T, int64_t S, int64_t d,
                     int64_t V, int64_t P, const int64_t* ids, const void* g, int64_t ld_g,
                     void* d_tok, int64_t ld_dtok, void* d_pos, int64_t ld_dpos,
                     void* workspace, int64_t workspace_bytes);

/* One AdamW step (decoupled weight decay, no amsgrad; the arithmetic of torch.optim.AdamW
 * operation for operation) over `count` fp32 parameter tensors in as few launches as their
 * descriptors fit into: p, m, v updated in place from the fp32 gradient; when `shadow` is
 * set, the updated parameter is also written there rounded to shadow_dtype -- the 16-bit
 * operand the next forward pass would otherwise produce with a cast kernel.  `step` counts
 * from 1.  No counterpart in the reference, which ships no optimizer; it is what turns the
 * forward + backward step that the reference times (README.md:62-77) into a training
 * step.  `tensors`: HOST array. */
typedef struct tf_adamw_tensor {
  void* param; const void* grad; void* exp_avg; void* exp_avg_sq;   /* fp32, `count` elements each */
  void* shadow;                                                      /* 16-bit, or null */
  int64_t count;
} tf_adamw_tensor;
int tf_adamw_step(void* stream, int shadow_dtype, int count, const tf_adamw_tensor* tensors,
                  float lr, float beta1, float beta2, float eps, float weight_decay, int64_t step);

/* Row softmax / its backward dx = y * (dy - sum(y*dy)); dtype f16/bf16/f32.
 * Replaces softmax_fwd / softmax_bwd (kernels/softmax.py:37-54, 95-111); the
 * backward writes a new buffer instead of overwriting grad_out. */
int tf_softmax_fwd(void* stream, int dtype, int64_t rows, int64_t cols,
                   const void* x, int64_t ldx, void* y, int64_t ldy);
int tf_softmax_bwd(void* stream, int dtype, int64_t rows, int64_t cols,
                   const void* dy, int64_t lddy, const void* y, int64_t ldy,
                   void* dx, int64_t lddx);

/* Per-row loss[r] = logsumexp(logits[r,:]) - logits[r, labels[r]] with an
 * online max/sum single pass; also stores lse[r] (natural log, fp32).
 * labels: int64, each in [0, V).  loss has `dtype`.
 * Row r starts at element (r / inner_rows) * outer_stride + (r % inner_rows) * ld;
 * inner_rows <= 0 means a plain matrix (row r at r * ld).  With inner_rows = S-1,
 * ld = V, outer_stride = S*V the rows are those of a (B, S, V) tensor without the
 * last position of each sequence: the shifted logits of transformer.py:333 read
 * in place, without the .contiguous() copy.
 * Replaces cross_entropy_fwd (kernels/crossentropy.py:47-75). */
int tf_cross_entropy_fwd(void* stream, int dtype, int64_t rows, int64_t V,
                         const void* logits, int64_t ld, int64_t inner_rows, int64_t outer_stride,
                         const int64_t* labels, void* loss, float* lse);

/* tf_cross_entropy_fwd that also writes dlogits[r,v] = (softmax(logits[r,:])[v] - [v == labels[r]])
 * * grad_scale in the same pass: rows of up to 51200 entries are held in registers between the
 * log-sum-exp and the gradient, so the logits are read once and the second pass of
 * tf_cross_entropy_bwd over the (N, V) matrix does not happen (kernels/crossentropy.py:47-75 and
 * :110-127 as one kernel).  The values equal, bit for bit, tf_cross_entropy_bwd with every
 * gout[r] = grad_scale (as a value of `dtype`); rows of dlogits are addressed like those of
 * logits with (ldd, inner_rows, outer_stride_d).  `grad_scale_dev`: one value of `dtype` in device
 * memory holding grad_scale, used only when the one-kernel form does not apply (longer rows,
 * unaligned matrices: forward and backward kernels then run one after the other); may be null
 * otherwise.  grad_scale = 1024 keeps fp16 probabilities of 1e-5 out of the subnormal range. */
int tf_cross_entropy_fwd_grad(void* stream, int dtype, int64_t rows, int64_t V,
                              const void* logits, int64_t ld, int64_t inner_rows, int64_t outer_stride,
                              const int64_t* labels, void* loss, float* lse,
                              void* dlogits, int64_t ldd, int64_t outer_stride_d,
                              float grad_scale, const void* grad_scale_dev);

/* dlogits[r,v] = (exp(logits[r,v] - lse[r]) - [v == labels[r]]) * gout[r], rows of
 * dlogits addressed like those of logits with (ldd, inner_rows, outer_stride_d).
 * Replaces cross_entropy_bwd (kernels/crossentropy.py:110-127) and the
 * broadcast multiply in tritonformer/crossentropy.py:24.  gout has `dtype`;
 * gout_stride 0 broadcasts one value. */
int tf_cross_entropy_bwd(void* stream, int dtype, int64_t rows, int64_t V,
                         const void* logits, int64_t ld, int64_t inner_rows, int64_t outer_stride,
                         const int64_t* labels, const float* lse, const void* gout, int64_t gout_stride,
                         void* dlogits, int64_t ldd, int64_t outer_stride_d);

/* out[c] = sum_r x[r, c] with fp32 accumulation (bias gradient); `out` has out_dtype:
 * `dtype`, or TF_F32 (the gradient of an fp32 master bias, stored unrounded).
 * Replaces unbroadcast_leading (kernels/reductions.py:97-122, two-stage with
 * _unbroadcast :57-63).  partial: fp32 scratch of tf_colsum_partial_bytes(). */
int tf_colsum(void* stream, int dtype, int out_dtype, int64_t rows, int64_t cols,
              const void* x, int64_t ldx, void* out,
              float* partial, int64_t partial_bytes);
int64_t tf_colsum_partial_bytes(int64_t rows, int64_t cols);

/* tf_colsum for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc): same kernels and results, bit for bit, with the
 * first-stage partial sums in a fixed 4 MiB array inside the library instead of a `partial`
 * buffer.  No counterpart in the reference.  The call allocates and frees nothing.
 * Limit: problems whose tf_colsum_partial_bytes(rows, cols) exceeds
 * tf_colsum_noalloc_max_partial_bytes() (4 MiB; the partial sums of a problem take about 2 MiB
 * whatever its shape, more only beyond a million columns) are refused with TF_EWORKSPACE.  Every call on one GPU uses that GPU's one array: calls that overlap in time on
 * one GPU (two streams, two threads) race; calls on one stream are ordered and safe. */
int tf_colsum_noalloc(void* stream, int dtype, int out_dtype, int64_t rows, int64_t cols,
                      const void* x, int64_t ldx, void* out);
int64_t tf_colsum_noalloc_max_partial_bytes(void);

/* out = where(act > 0, grad, 0), out of place.
 * Replaces mask_grad (kernels/activation.py:27-44), which works in place. */
int tf_relu_mask(void* stream, int dtype, int64_t rows, int64_t cols,
                 const void* grad, int64_t ldg, const void* act, int64_t lda,
                 void* out, int64_t ldo);

#ifdef __cplusplus
}
#endif
#endif /* TRITONFORMER_AMD_H */
