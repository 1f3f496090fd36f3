// Shared helpers of the gfx950 kernels: storage-type conversion, wave-level
// reductions (64-wide wavefronts) and launch checks. Every exported function
// is extern "C", takes raw device pointers plus a hipStream_t, launches on that
// stream and returns 0 or a negative error code; it allocates nothing (one exception: the
// library product of blaslt.hip allocates the library's workspace at its first call).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define PTL_OK 0
#define PTL_ERR_ARG (-1)
#define PTL_ERR_LAUNCH (-2)

#define PTL_DTYPE_F32 0
#define PTL_DTYPE_BF16 1

typedef uint16_t bf16_t;  // raw bfloat16 bits

__device__ __forceinline__ float bf16_to_float(bf16_t v) {
  return __uint_as_float(((uint32_t)v) << 16);
}

// round to nearest even; NaN stays NaN
__device__ __forceinline__ bf16_t float_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (bf16_t)(u >> 16);
}

// 16 bytes that a kernel reads once (weights, the cache of a decoding request, a product's result
// on its way through an elementwise kernel): a load marked as not to be used again, so that it
// does not displace what later kernels find in the caches.
typedef unsigned int ptl_u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 load_once(const void* p) {
  const ptl_u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const ptl_u32x4_t*>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}

template <typename T> __device__ __forceinline__ float to_float(T v);
template <> __device__ __forceinline__ float to_float<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_float<bf16_t>(bf16_t v) { return bf16_to_float(v); }

template <typename T> __device__ __forceinline__ T from_float(float v);
template <> __device__ __forceinline__ float from_float<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_float<bf16_t>(float v) { return float_to_bf16(v); }

// value as it reads back after a store in T (used where a later kernel reads it)
template <typename T> __device__ __forceinline__ float round_to(float v) {
  return to_float<T>(from_float<T>(v));
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// block-wide sum for blockDim.x a multiple of 64, at most 1024; scratch holds 16 floats
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int nw = blockDim.x >> 6;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float r = 0.f;
  for (int i = 0; i < nw; ++i) r += scratch[i];
  return r;
}
__device__ __forceinline__ float block_max(float v, float* scratch) {
  v = wave_max(v);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int nw = blockDim.x >> 6;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float r = scratch[0];
  for (int i = 1; i < nw; ++i) r = fmaxf(r, scratch[i]);
  return r;
}

static inline int ptl_launch_status() {
  return hipGetLastError() == hipSuccess ? PTL_OK : PTL_ERR_LAUNCH;
}
