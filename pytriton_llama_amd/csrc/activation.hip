// SiLU-and-multiply on a fused gate|up row: out[t, i] = silu(gu[t, i]) * gu[t, I + i],
// silu(g) = g * sigmoid(g) in float32 (reference: lite_llama/kernels/swiglu.py:44-67).
#include "common.h"

template <typename T>
__global__ void silu_mul_kernel(T* __restrict__ out, const T* __restrict__ gu, int I, size_t total) {
  size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t step = (size_t)gridDim.x * blockDim.x;
  for (; idx < total; idx += step) {
    const size_t t = idx / I;
    const int i = (int)(idx - t * I);
    const float g = to_float<T>(gu[t * 2 * I + i]);
    const float u = to_float<T>(gu[t * 2 * I + I + i]);
    const float s = g / (1.0f + expf(-g));
    out[idx] = from_float<T>(s * u);
  }
}

extern "C" int ptl_silu_mul(void* out, const void* gate_up, int T_, int I, int dtype,
                            hipStream_t stream) {
  if (T_ <= 0) return PTL_OK;
  if (I <= 0) return PTL_ERR_ARG;
  const size_t total = (size_t)T_ * I;
  const int threads = 256;
  size_t blocks = (total + threads - 1) / threads;
  if (blocks > 65536) blocks = 65536;
  if (dtype == PTL_DTYPE_F32)
    silu_mul_kernel<float><<<(int)blocks, threads, 0, stream>>>((float*)out, (const float*)gate_up, I, total);
  else if (dtype == PTL_DTYPE_BF16)
    silu_mul_kernel<bf16_t><<<(int)blocks, threads, 0, stream>>>((bf16_t*)out, (const bf16_t*)gate_up, I, total);
  else
    return PTL_ERR_ARG;
  return ptl_launch_status();
}
