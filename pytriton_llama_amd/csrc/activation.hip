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

// bfloat16 rows with I a multiple of 8: 16-byte loads and stores
__global__ void __launch_bounds__(256)
silu_mul_bf16_vec_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ gu, int I8, size_t total8) {
  size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t step = (size_t)gridDim.x * blockDim.x;
  for (; idx < total8; idx += step) {
    const size_t t = idx / I8;
    const int c = (int)(idx - t * I8);
    union { uint4 u; bf16_t e[8]; } g, u, o;
    g.u = *reinterpret_cast<const uint4*>(gu + (t * 2 * I8 + c) * 8);
    u.u = *reinterpret_cast<const uint4*>(gu + (t * 2 * I8 + I8 + c) * 8);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float gf = bf16_to_float(g.e[j]);
      o.e[j] = float_to_bf16(gf / (1.0f + expf(-gf)) * bf16_to_float(u.e[j]));
    }
    *reinterpret_cast<uint4*>(out + idx * 8) = o.u;
  }
}

extern "C" int ptl_silu_mul(void* out, const void* gate_up, int T_, int I, int dtype,
                            hipStream_t stream) {
  if (T_ <= 0) return PTL_OK;
  if (I <= 0) return PTL_ERR_ARG;
  if (dtype == PTL_DTYPE_BF16 && I % 8 == 0 && ((uintptr_t)out | (uintptr_t)gate_up) % 16 == 0) {
    const size_t total8 = (size_t)T_ * (I / 8);
    size_t vb = (total8 + 255) / 256;
    if (vb > 16384) vb = 16384;
    silu_mul_bf16_vec_kernel<<<(int)vb, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)gate_up, I / 8, total8);
    return ptl_launch_status();
  }
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
