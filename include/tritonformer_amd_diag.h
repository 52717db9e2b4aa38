/*
 * tritonformer_amd_diag.h -- diagnostics, NOT part of the drop-in boundary.
 *
 * Nothing here has a counterpart in the reference (its nearest relative is Triton's
 * autotuner, tritonformer/kernels/gemm.py:15-79, which times tile configurations per
 * shape).  No operator of the package calls these; they exist for the benchmark, for
 * tests that want every tile configuration exercised on small shapes, and for kernel
 * work.  All of them are stateless except the launch counter, which is a relaxed atomic.
 *
 * tf_diag_gemm* live in libtritonformer_amd.so (they need the GEMM's internals);
 * tf_diag_mfma_rate* live in libtritonformer_amd_diag.so, a library of its own.
 */
#ifndef TRITONFORMER_AMD_DIAG_H
#define TRITONFORMER_AMD_DIAG_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* tf_gemm_out (include/tritonformer_amd.h) with the tile choice imposed on THIS call:
 *   cfg    -1 = cost model; 0 / 1 = register-staged 256x256 / 128x128;
 *          2..5 = direct-to-LDS 256x256, 128x128, 256x128, 128x256
 *          (a direct-to-LDS cfg falls back to its register-staged twin when the operands
 *          do not meet its preconditions);
 *   splits 0 = chosen by the library, n > 0 = contraction cut into n slices;
 *   flags  bit 0: workgroup ids are not remapped to XCDs; bit 6 (64): the product is never
 *          cut along N into whole rounds + tail.  Other bits are refused.
 * Results are those of tf_gemm_out up to the fp32 summation order of a split contraction.
 * workspace: tf_diag_gemm_workspace_bytes(cfg, splits, M, N, K) bytes. */
int tf_diag_gemm(void* stream, int cfg, int splits, int flags, int dtype, int out_dtype,
                 int layout_a, int layout_b, int64_t M, int64_t N, int64_t K,
                 const void* A, int64_t lda, const void* B, int64_t ldb, void* C, int64_t ldc,
                 const void* bias, int relu, void* workspace, int64_t workspace_bytes);
int64_t tf_diag_gemm_workspace_bytes(int cfg, int splits, int64_t M, int64_t N, int64_t K);

/* GEMM kernels launched by libtritonformer_amd.so since it was loaded (the reduce passes of
 * split contractions are not counted; one tf_gemm* call may launch two kernels when the
 * product is cut along N).  bench.py divides its event times by the difference of two reads. */
int64_t tf_diag_gemm_launch_count(void);

/* The MFMA instruction stream of the 256x256x64 GEMM step alone: `workgroups` workgroups of 8
 * waves, no memory traffic, `iters` steps each, operands taken once from `operands`
 * (8*6*64*8 = 24576 elements of `dtype`, device memory); `sink`: workgroups*512 floats.  Time
 * the call and divide tf_diag_mfma_rate_flops(iters, workgroups) by it: the sustained rate
 * depends on the operand values (the clock drops under the switching activity of random data). */
int tf_diag_mfma_rate(void* stream, int dtype, const void* operands, int iters, int workgroups,
                      float* sink);
int64_t tf_diag_mfma_rate_flops(int iters, int workgroups);

#ifdef __cplusplus
}
#endif
#endif /* TRITONFORMER_AMD_DIAG_H */
