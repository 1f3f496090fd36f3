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

// bfloat16 rows with I a multiple of 8: 16-byte loads and stores. A thread takes the same
// chunk of two rows (blockIdx.y names the pair), so four loads are under way before the
// first exponential; x / (1 + exp(-x)) with the hardware's exp2 and reciprocal (float32,
// a few units in the last place, far below the bfloat16 rounding of the result).
__device__ __forceinline__ float silu_fast(float x) {
  return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * x));
}

__global__ void __launch_bounds__(256)
silu_mul_bf16_vec_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ gu, int I8, int T_) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= I8) return;
  const int t0 = 2 * blockIdx.y;
  const bool two = t0 + 1 < T_;
  const bf16_t* row0 = gu + ((size_t)t0 * 2 * I8 + c) * 8;
  const bf16_t* row1 = two ? row0 + (size_t)2 * I8 * 8 : row0;
  union { uint4 u; bf16_t e[8]; } g[2], u[2], o[2];
  g[0].u = load_once(row0);
  u[0].u = load_once(row0 + (size_t)I8 * 8);
  g[1].u = load_once(row1);
  u[1].u = load_once(row1 + (size_t)I8 * 8);
#pragma unroll
  for (int r = 0; r < 2; ++r)
#pragma unroll
    for (int j = 0; j < 8; ++j)
      o[r].e[j] = float_to_bf16(silu_fast(bf16_to_float(g[r].e[j])) * bf16_to_float(u[r].e[j]));
  bf16_t* dst = out + ((size_t)t0 * I8 + c) * 8;
  *reinterpret_cast<uint4*>(dst) = o[0].u;
  if (two) *reinterpret_cast<uint4*>(dst + (size_t)I8 * 8) = o[1].u;
}

extern "C" int ptl_silu_mul(void* out, const void* gate_up, int T_, int I, int dtype,
                            hipStream_t stream) {
  if (T_ <= 0) return PTL_OK;
  if (I <= 0) return PTL_ERR_ARG;
  if (dtype == PTL_DTYPE_BF16 && I % 8 == 0 && ((uintptr_t)out | (uintptr_t)gate_up) % 16 == 0) {
    const int I8 = I / 8;
    dim3 grid((I8 + 255) / 256, (T_ + 1) / 2);
    if (grid.y > 65535) return PTL_ERR_ARG;
    silu_mul_bf16_vec_kernel<<<grid, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)gate_up, I8, T_);
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
