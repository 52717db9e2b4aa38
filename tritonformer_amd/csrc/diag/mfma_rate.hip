// Diagnostic: sustained MFMA rate of the GEMM kernel's instruction stream alone.
// `workgroups` workgroups (one per CU is the intended use), 8 waves, each issuing the 32 v_mfma_f32_32x32x16 of one 256x256x64
// step per loop trip from fixed operand registers -- no memory traffic at all.  The rate
// depends on the operand VALUES (the chip lowers its clock under the switching activity of
// random data), which is why the operands are an argument: it is the practical ceiling a
// GEMM on real data can be compared with.
#include "../rowops.h"
#include "../../../include/tritonformer_amd_diag.h"

namespace tfa {

template <typename T>
__global__ __launch_bounds__(512, 2) void mfma_rate_kernel(const T* __restrict__ operands, int iters, float* __restrict__ sink) {
  typedef typename Vec<T>::v8 v8;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  v8 a[4], b[2];
#pragma unroll
  for (int i = 0; i < 4; ++i) a[i] = __builtin_bit_cast(v8, ld16(operands + ((wave * 6 + i) * 64 + lane) * 8));
#pragma unroll
  for (int i = 0; i < 2; ++i) b[i] = __builtin_bit_cast(v8, ld16(operands + ((wave * 6 + 4 + i) * 64 + lane) * 8));
  f32x16 c[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) c[i][j][r] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) c[i][j] = mfma32(b[j], a[i], c[i][j]);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) s += c[i][j][r];
  sink[blockIdx.x * 512 + threadIdx.x] = s;
}

}  // namespace tfa

using namespace tfa;

extern "C" int64_t tf_diag_mfma_rate_flops(int iters, int workgroups) {
  return iters > 0 && workgroups > 0 ? (int64_t)iters * workgroups * (2ll * 256 * 256 * 64) : 0;
}

extern "C" int tf_diag_mfma_rate(void* stream, int dtype, const void* operands, int iters, int workgroups,
                                 float* sink) {
  if (!operands || !sink || iters <= 0 || workgroups <= 0 || workgroups > 65536) return TF_EINVAL;
  if (!aligned16(operands)) return TF_EALIGN;
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid((unsigned)workgroups);
  if (dtype == TF_F16) mfma_rate_kernel<f16><<<grid, dim3(512), 0, st>>>((const f16*)operands, iters, sink);
  else if (dtype == TF_BF16) mfma_rate_kernel<bf16><<<grid, dim3(512), 0, st>>>((const bf16*)operands, iters, sink);
  else return TF_EDTYPE;
  TF_CHECK_LAUNCH();
  return TF_OK;
}
