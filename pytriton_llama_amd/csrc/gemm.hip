// y = x W^T for row-major x [M, K] (row stride ldx) and W [N, K]: every linear
// layer of the model (the reference uses cuBLAS through nn.Linear / F.linear,
// lite_llama/models/llama.py:37-40,61,120,221).
//
// ptl_gemm_nt: a tiled vector-FMA kernel with float32 accumulation for any
// M, N, K and any mix of float32 / bfloat16 inputs and outputs. It is the whole
// matrix path of the true 32-bit mode (no reduced-precision matrix mode can
// hide in it) and the fallback of the bfloat16 mode.
#include "common.h"

#define TM 64
#define TN 64
#define TK 16

template <typename TX, typename TW, typename TY>
__global__ void __launch_bounds__(256)
gemm_nt_kernel(TY* __restrict__ y, const TX* __restrict__ x, const TW* __restrict__ w,
               int M, int N, int K, long ldx, long ldy) {
  __shared__ float As[TK][TM + 4];
  __shared__ float Bs[TK][TN + 4];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;
  const int lr = tid >> 2;         // 0..63: tile row loaded by this thread
  const int lk = (tid & 3) << 2;   // 0,4,8,12: first k of its four
  const int ty = tid >> 4, tx = tid & 15;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += TK) {
    {
      const int m = m0 + lr;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int k = k0 + lk + i;
        As[lk + i][lr] = (m < M && k < K) ? to_float<TX>(x[(size_t)m * ldx + k]) : 0.f;
      }
      const int n = n0 + lr;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int k = k0 + lk + i;
        Bs[lk + i][lr] = (n < N && k < K) ? to_float<TW>(w[(size_t)n * K + k]) : 0.f;
      }
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < TK; ++k) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Bs[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N) y[(size_t)m * ldy + n] = from_float<TY>(acc[i][j]);
    }
  }
}

template <typename TX, typename TW, typename TY>
static int launch_gemm_nt(void* y, const void* x, const void* w, int M, int N, int K,
                          long ldx, long ldy, hipStream_t stream) {
  dim3 grid((N + TN - 1) / TN, (M + TM - 1) / TM);
  gemm_nt_kernel<TX, TW, TY><<<grid, 256, 0, stream>>>((TY*)y, (const TX*)x, (const TW*)w,
                                                       M, N, K, ldx, ldy);
  return ptl_launch_status();
}

// in_dtype: of x and w; out_dtype: of y
extern "C" int ptl_gemm_nt(void* y, const void* x, const void* w, int M, int N, int K,
                           long ldx, long ldy, int in_dtype, int out_dtype, hipStream_t stream) {
  if (M <= 0 || N <= 0) return PTL_OK;
  if (K <= 0 || ldx < K || ldy < N) return PTL_ERR_ARG;
  if ((M + TM - 1) / TM > 65535) return PTL_ERR_ARG;
  if (in_dtype == PTL_DTYPE_F32 && out_dtype == PTL_DTYPE_F32)
    return launch_gemm_nt<float, float, float>(y, x, w, M, N, K, ldx, ldy, stream);
  if (in_dtype == PTL_DTYPE_BF16 && out_dtype == PTL_DTYPE_BF16)
    return launch_gemm_nt<bf16_t, bf16_t, bf16_t>(y, x, w, M, N, K, ldx, ldy, stream);
  if (in_dtype == PTL_DTYPE_BF16 && out_dtype == PTL_DTYPE_F32)
    return launch_gemm_nt<bf16_t, bf16_t, float>(y, x, w, M, N, K, ldx, ldy, stream);
  return PTL_ERR_ARG;
}
