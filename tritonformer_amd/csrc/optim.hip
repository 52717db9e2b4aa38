// Fused AdamW step over many parameter tensors in one launch (fp32 master parameters, fp32
// gradients and moments), optionally writing the 16-bit copy of every updated parameter that
// the next forward pass would otherwise make with a cast kernel.  HBM-bound: 16 bytes read and
// 12 (+2) written per parameter.
#include <cmath>
#include "rowops.h"

namespace tfa {

constexpr int kAdamTensors = 24;   // per launch: the descriptors travel as kernel arguments
constexpr int kAdamMaxBlocks = 2048;     // per tensor; a block takes at least 8192 elements

struct AdamTensor {
  float* param;
  const float* grad;
  float* exp_avg;
  float* exp_avg_sq;
  void* shadow;   // 16-bit copy of param after the update, or null
  int64_t count;
  int blocks;     // workgroups that share this tensor (grid.x is the largest of the launch)
};
struct AdamBatch {
  AdamTensor t[kAdamTensors];
};

// The arithmetic of torch.optim.AdamW (decoupled weight decay, no amsgrad), operation for operation:
//   p *= 1 - lr * wd;  m += (g - m) * (1 - b1);  v = v * b2 + (1 - b2) * g * g;
//   p -= (lr / bc1) * m / (sqrt(v) / sqrt(bc2) + eps)
template <typename TS>
__global__ __launch_bounds__(256) void adamw_kernel(AdamBatch batch, float decay, float one_minus_b1, float b2,
                                                    float one_minus_b2, float step_size, float sqrt_bc2, float eps) {
  const AdamTensor t = batch.t[blockIdx.y];
  if ((int)blockIdx.x >= t.blocks) return;
  const int64_t n4 = t.count / 4;
  const int64_t stride = (int64_t)t.blocks * 256;
  auto update = [&](float& p, float g, float& m, float& v) {
    p *= decay;
    m += (g - m) * one_minus_b1;
    v = v * b2 + one_minus_b2 * g * g;
    const float denom = sqrtf(v) / sqrt_bc2 + eps;
    p -= step_size * (m / denom);
  };
  const bool vec = ((reinterpret_cast<uintptr_t>(t.param) | reinterpret_cast<uintptr_t>(t.grad) |
                     reinterpret_cast<uintptr_t>(t.exp_avg) | reinterpret_cast<uintptr_t>(t.exp_avg_sq)) & 15) == 0 &&
                   (reinterpret_cast<uintptr_t>(t.shadow) & 7) == 0;
  int64_t done = 0;
  if (vec) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += stride) {
      f32x4 p = reinterpret_cast<const f32x4*>(t.param)[i];
      const f32x4 g = reinterpret_cast<const f32x4*>(t.grad)[i];
      f32x4 m = reinterpret_cast<const f32x4*>(t.exp_avg)[i];
      f32x4 v = reinterpret_cast<const f32x4*>(t.exp_avg_sq)[i];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float pe = p[e], me = m[e], ve = v[e];
        update(pe, g[e], me, ve);
        p[e] = pe; m[e] = me; v[e] = ve;
      }
      reinterpret_cast<f32x4*>(t.param)[i] = p;
      reinterpret_cast<f32x4*>(t.exp_avg)[i] = m;
      reinterpret_cast<f32x4*>(t.exp_avg_sq)[i] = v;
      if (t.shadow) {
        typename Vec<TS>::v4 s;
#pragma unroll
        for (int e = 0; e < 4; ++e) s[e] = (TS)p[e];
        reinterpret_cast<typename Vec<TS>::v4*>(t.shadow)[i] = s;
      }
    }
    done = n4 * 4;
  }
  for (int64_t i = done + (int64_t)blockIdx.x * 256 + threadIdx.x; i < t.count; i += stride) {
    float p = t.param[i], m = t.exp_avg[i], v = t.exp_avg_sq[i];
    update(p, t.grad[i], m, v);
    t.param[i] = p;
    t.exp_avg[i] = m;
    t.exp_avg_sq[i] = v;
    if (t.shadow) reinterpret_cast<TS*>(t.shadow)[i] = (TS)p;
  }
}

}  // namespace tfa

using namespace tfa;

extern "C" int tf_adamw_step(void* stream, int shadow_dtype, int count, const tf_adamw_tensor* tensors, float lr,
                             float beta1, float beta2, float eps, float weight_decay, int64_t step) {
  if (count < 0 || (count > 0 && !tensors) || step < 1) return TF_EINVAL;
  if (!(beta1 >= 0.f && beta1 < 1.f && beta2 >= 0.f && beta2 < 1.f) || !(eps >= 0.f) || !(lr >= 0.f)) return TF_EINVAL;
  bool any_shadow = false;
  for (int i = 0; i < count; ++i) {
    const tf_adamw_tensor& t = tensors[i];
    if (t.count < 0 || (t.count > 0 && (!t.param || !t.grad || !t.exp_avg || !t.exp_avg_sq))) return TF_EINVAL;
    if (((reinterpret_cast<uintptr_t>(t.param) | reinterpret_cast<uintptr_t>(t.grad) |
          reinterpret_cast<uintptr_t>(t.exp_avg) | reinterpret_cast<uintptr_t>(t.exp_avg_sq)) & 3) ||
        (reinterpret_cast<uintptr_t>(t.shadow) & 1))
      return TF_EALIGN;
    any_shadow = any_shadow || t.shadow != nullptr;
  }
  if (any_shadow && shadow_dtype != TF_F16 && shadow_dtype != TF_BF16) return TF_EDTYPE;
  // bias corrections in double, as the reference implementation computes them on the host
  const double bc1 = 1.0 - pow((double)beta1, (double)step);
  const double bc2 = 1.0 - pow((double)beta2, (double)step);
  const float decay = 1.0f - lr * weight_decay;
  const float step_size = (float)((double)lr / bc1);
  const float sqrt_bc2 = (float)sqrt(bc2);
  hipStream_t st = (hipStream_t)stream;
  for (int first = 0; first < count; first += kAdamTensors) {
    AdamBatch batch = {};
    const int n = count - first < kAdamTensors ? count - first : kAdamTensors;
    int max_blocks = 1;
    for (int i = 0; i < n; ++i) {
      const tf_adamw_tensor& t = tensors[first + i];
      int64_t blocks = (t.count + 8191) / 8192;
      blocks = blocks < 1 ? 1 : (blocks > kAdamMaxBlocks ? kAdamMaxBlocks : blocks);
      batch.t[i] = {(float*)t.param, (const float*)t.grad, (float*)t.exp_avg, (float*)t.exp_avg_sq, t.shadow, t.count,
                    (int)blocks};
      if (blocks > max_blocks) max_blocks = (int)blocks;
    }
    const dim3 grid((unsigned)max_blocks, (unsigned)n);
    if (shadow_dtype == TF_BF16)
      adamw_kernel<bf16><<<grid, dim3(256), 0, st>>>(batch, decay, 1.0f - beta1, beta2, 1.0f - beta2, step_size,
                                                      sqrt_bc2, eps);
    else
      adamw_kernel<f16><<<grid, dim3(256), 0, st>>>(batch, decay, 1.0f - beta1, beta2, 1.0f - beta2, step_size, sqrt_bc2,
                                                     eps);
    TF_CHECK_LAUNCH();
  }
  return TF_OK;
}
