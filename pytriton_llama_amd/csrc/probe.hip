// Two probes of what the GPU gives, for the roofline figures of the benchmark:
// ptl_probe_stream_read: a kernel that only reads memory (16-byte loads that are not kept in
//   the caches, eight in flight per thread) and throws it away;
// ptl_probe_mfma: a loop of independent v_mfma_f32_16x16x32_bf16 in every wave.
// Neither is used by the engine.
#include "common.h"
#include "mfma.h"

typedef unsigned int probe_u32x4 __attribute__((ext_vector_type(4)));

__global__ void __launch_bounds__(256)
probe_stream_read_kernel(const probe_u32x4* __restrict__ p, size_t n16, uint32_t* __restrict__ sink) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  uint32_t acc = 0;
  for (; i + 7 * stride < n16; i += 8 * stride) {
    probe_u32x4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load(p + i + u * stride);
#pragma unroll
    for (int u = 0; u < 8; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  for (; i < n16; i += stride) {
    const probe_u32x4 v = __builtin_nontemporal_load(p + i);
    acc ^= v.x ^ v.y ^ v.z ^ v.w;
  }
  sink[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = acc;      // keeps the loads
}

// sink: one 32-bit word per thread of the launch (blocks * 256)
extern "C" int ptl_probe_stream_read(const void* p, size_t bytes, int blocks, void* sink,
                                     hipStream_t stream) {
  if (blocks <= 0 || !p || !sink || ((uintptr_t)p & 15)) return PTL_ERR_ARG;
  probe_stream_read_kernel<<<blocks, 256, 0, stream>>>((const probe_u32x4*)p, bytes / 16,
                                                       (uint32_t*)sink);
  return ptl_launch_status();
}

__global__ void __launch_bounds__(256)
probe_mfma_kernel(float* __restrict__ out, int iters) {
  Frag8 a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a.v[i] = (__bf16)(0.001f * (float)(threadIdx.x & 15) + 0.01f * (float)i);
    b.v[i] = (__bf16)(0.5f - 0.1f * (float)i);
  }
  f32x4_t c[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) c[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  for (int it = 0; it < iters; it += 4) {        // (iters is a multiple of 4)
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int j = 0; j < 8; ++j) c[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, b.v, c[j], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j) s += c[j][0] + c[j][1] + c[j][2] + c[j][3];
  out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = s;
}

// out: one float per thread of the launch (blocks * 256). Every wave issues iters * 8 MFMAs of
// 16 * 16 * 32 * 2 floating-point operations.
extern "C" int ptl_probe_mfma(void* out, int iters, int blocks, hipStream_t stream) {
  if (blocks <= 0 || iters <= 0 || iters % 4 || !out) return PTL_ERR_ARG;
  probe_mfma_kernel<<<blocks, 256, 0, stream>>>((float*)out, iters);
  return ptl_launch_status();
}
