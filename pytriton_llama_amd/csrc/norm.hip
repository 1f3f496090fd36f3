// Fused residual sum + RMSNorm, one workgroup per token row.
// Reference: lite_llama/kernels/skip_rmsnorm.py:94-120 (no residual) and
// :122-156 (with residual): s = x + r in float32, r <- s, var = sum(s*s)/N,
// y = s * rsqrt(var + eps) * w. The sum, the statistics and the product are
// float32; the norm uses the unrounded sum as the reference does (:145-152).
#include "common.h"

template <typename T, int VEC>
__global__ void add_rmsnorm_kernel(T* __restrict__ y, const T* __restrict__ x,
                                   T* __restrict__ residual, const float* __restrict__ w,
                                   int H, float eps, int has_residual) {
  __shared__ float scratch[16];
  extern __shared__ float row[];  // H floats: the summed row
  const size_t base = (size_t)blockIdx.x * H;
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float v = to_float<T>(x[base + i]);
    if (has_residual) {
      v += to_float<T>(residual[base + i]);
      residual[base + i] = from_float<T>(v);
    }
    row[i] = v;
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float rr = 1.0f / sqrtf(ss / (float)H + eps);
  for (int i = threadIdx.x; i < H; i += blockDim.x)
    y[base + i] = from_float<T>(row[i] * rr * w[i]);
}

extern "C" int ptl_add_rmsnorm(void* y, const void* x, void* residual, const float* w,
                               int T_, int H, float eps, int dtype, hipStream_t stream) {
  if (T_ <= 0) return PTL_OK;
  if (H <= 0 || (size_t)H * 4 > 60000) return PTL_ERR_ARG;
  int threads = 64;
  while (threads < 1024 && threads * 4 < H) threads <<= 1;
  const size_t lds = (size_t)H * sizeof(float);
  const int has_res = residual != nullptr;
  if (dtype == PTL_DTYPE_F32)
    add_rmsnorm_kernel<float, 1><<<T_, threads, lds, stream>>>(
        (float*)y, (const float*)x, (float*)residual, w, H, eps, has_res);
  else if (dtype == PTL_DTYPE_BF16)
    add_rmsnorm_kernel<bf16_t, 1><<<T_, threads, lds, stream>>>(
        (bf16_t*)y, (const bf16_t*)x, (bf16_t*)residual, w, H, eps, has_res);
  else
    return PTL_ERR_ARG;
  return ptl_launch_status();
}
