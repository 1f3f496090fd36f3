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

// Rows too wide for the LDS copy above: two passes over memory. The first adds up the squares of
// the sums without storing them, the second makes the sums again (from the same inputs, so they
// are the same numbers), stores them as the new residual and writes the result. Every element is
// read and written by one thread only, so y may be x.
template <typename T>
__global__ void __launch_bounds__(1024)
add_rmsnorm_wide_kernel(T* __restrict__ y, const T* __restrict__ x, T* __restrict__ residual,
                        const float* __restrict__ w, int H, float eps, int has_residual) {
  __shared__ float scratch[16];
  const size_t base = (size_t)blockIdx.x * H;
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float v = to_float<T>(x[base + i]);
    if (has_residual) v += to_float<T>(residual[base + i]);
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float rr = 1.0f / sqrtf(ss / (float)H + eps);
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float v = to_float<T>(x[base + i]);
    if (has_residual) {
      v += to_float<T>(residual[base + i]);
      residual[base + i] = from_float<T>(v);
    }
    y[base + i] = from_float<T>(v * rr * w[i]);
  }
}

// bfloat16 rows whose width is a multiple of 8: 16-byte loads, the summed row stays in
// registers (CH chunks of 8 elements per thread), one pass over memory.
template <int CH>
__global__ void __launch_bounds__(256)
add_rmsnorm_bf16_vec_kernel(bf16_t* __restrict__ y, const bf16_t* __restrict__ x,
                            bf16_t* __restrict__ residual, const float* __restrict__ w, int H,
                            float eps, int has_residual) {
  __shared__ float scratch[16];
  const size_t base = (size_t)blockIdx.x * H;
  const int nchunk = H >> 3;
  float v[CH][8];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int ci = threadIdx.x + c * blockDim.x;
    if (ci < nchunk) {
      union { uint4 u; bf16_t e[8]; } a, r;
      a.u = load_once(x + base + (size_t)ci * 8);
      if (has_residual) r.u = *reinterpret_cast<const uint4*>(residual + base + (size_t)ci * 8);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        float f = bf16_to_float(a.e[j]);
        if (has_residual) {
          f += bf16_to_float(r.e[j]);
          r.e[j] = float_to_bf16(f);
        }
        v[c][j] = f;
        ss += f * f;
      }
      if (has_residual) *reinterpret_cast<uint4*>(residual + base + (size_t)ci * 8) = r.u;
    }
  }
  ss = block_sum(ss, scratch);
  const float rr = 1.0f / sqrtf(ss / (float)H + eps);
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int ci = threadIdx.x + c * blockDim.x;
    if (ci < nchunk) {
      const float4 w0 = *reinterpret_cast<const float4*>(w + (size_t)ci * 8);
      const float4 w1 = *reinterpret_cast<const float4*>(w + (size_t)ci * 8 + 4);
      const float ww[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
      union { uint4 u; bf16_t e[8]; } o;
#pragma unroll
      for (int j = 0; j < 8; ++j) o.e[j] = float_to_bf16(v[c][j] * rr * ww[j]);
      *reinterpret_cast<uint4*>(y + base + (size_t)ci * 8) = o.u;
    }
  }
}

extern "C" int ptl_add_rmsnorm(void* y, const void* x, void* residual, const float* w,
                               int T_, int H, float eps, int dtype, hipStream_t stream) {
  if (T_ <= 0) return PTL_OK;
  if (H <= 0) return PTL_ERR_ARG;
  if (dtype == PTL_DTYPE_BF16 && H % 8 == 0 && H <= 8 * 256 * 4 &&
      ((uintptr_t)x | (uintptr_t)y | (uintptr_t)residual | (uintptr_t)w) % 16 == 0) {
    const int nchunk = H / 8;
    int vt = 64;
    while (vt < 256 && vt < nchunk) vt <<= 1;
    const int ch = (nchunk + vt - 1) / vt;
    const int has = residual != nullptr;
#define GO(C) add_rmsnorm_bf16_vec_kernel<C><<<T_, vt, 0, stream>>>(                              \
      (bf16_t*)y, (const bf16_t*)x, (bf16_t*)residual, w, H, eps, has)
    if (ch <= 1) GO(1); else if (ch == 2) GO(2); else if (ch == 3) GO(3); else GO(4);
#undef GO
    return ptl_launch_status();
  }
  int threads = 64;
  while (threads < 1024 && threads * 4 < H) threads <<= 1;
  const size_t lds = (size_t)H * sizeof(float);
  const int has_res = residual != nullptr;
  if (lds > 60000) {        // the row does not fit the LDS a workgroup may ask for
    if (dtype == PTL_DTYPE_F32)
      add_rmsnorm_wide_kernel<float><<<T_, 1024, 0, stream>>>(
          (float*)y, (const float*)x, (float*)residual, w, H, eps, has_res);
    else if (dtype == PTL_DTYPE_BF16)
      add_rmsnorm_wide_kernel<bf16_t><<<T_, 1024, 0, stream>>>(
          (bf16_t*)y, (const bf16_t*)x, (bf16_t*)residual, w, H, eps, has_res);
    else
      return PTL_ERR_ARG;
    return ptl_launch_status();
  }
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

// y[m, :] = v[m, :] * rsqrt(sum_j partials[m][j] / H + eps): finishes a normalisation whose
// weight is already in v and whose sums of squares lie in ``count`` partial sums a row (written
// by the product that made v, see gemm.hip). For consumers that cannot apply the factor to
// their own results. bfloat16.
__global__ void __launch_bounds__(256)
row_scale_kernel(bf16_t* __restrict__ y, const bf16_t* __restrict__ v,
                 const float* __restrict__ partials, int count, int H, float eps) {
  __shared__ float scratch[16];
  const int m = blockIdx.x;
  float sum = 0.f;
  for (int j = threadIdx.x; j < count; j += blockDim.x) sum += partials[(size_t)m * count + j];
  sum = block_sum(sum, scratch);
  const float f = 1.0f / sqrtf(sum / (float)H + eps);
  for (int i = threadIdx.x; i < H; i += blockDim.x)
    y[(size_t)m * H + i] = float_to_bf16(bf16_to_float(v[(size_t)m * H + i]) * f);
}

extern "C" int ptl_row_scale_bf16(void* y, const void* v, const float* partials, int count, int T_,
                                  int H, float eps, hipStream_t stream) {
  if (T_ <= 0) return PTL_OK;
  if (H <= 0 || count <= 0 || !partials) return PTL_ERR_ARG;
  row_scale_kernel<<<T_, 256, 0, stream>>>((bf16_t*)y, (const bf16_t*)v, partials, count, H, eps);
  return ptl_launch_status();
}
