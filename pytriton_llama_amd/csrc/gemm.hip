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

// ===========================================================================
// ptl_gemm_skinny_bf16: y = x W^T for the few rows of a decode step (M <= 64)
// in bfloat16 on the matrix cores. The step is bound by reading W once from
// HBM, so the kernel is built around streaming weight rows: a workgroup owns 16
// rows of W (16 output columns); its waves split K among themselves and every
// wave keeps many 16-byte loads in flight. v_mfma_f32_16x16x32_bf16 takes the
// weight tile as A (row lane%16, 8 consecutive k of group lane/16: one 16-byte
// load straight from global memory) and x^T as B (row m = lane%16 of x, the
// same 8 k), and leaves y^T[n, m] in float32; the waves' partial sums meet in
// LDS. x is small and stays in L2. Output bfloat16 or float32.
// Needs K % 8 == 0 and 16-byte aligned rows of x.
// ===========================================================================
typedef __bf16 gs_bf16x8_t __attribute__((ext_vector_type(8)));
typedef float gs_f32x4_t __attribute__((ext_vector_type(4)));

union GsFrag {
  uint4 u;
  gs_bf16x8_t v;
};

template <int MT, int U, typename TY>
__global__ void __launch_bounds__(1024)
gemm_skinny_kernel(TY* __restrict__ y, const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                   int M, int N, int K, long ldx, long ldy, int k_per_wave) {
  extern __shared__ float red[];                 // [waves][MT][64][4]
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, ln = lane & 15, lg = lane >> 4;
  const int nwaves = blockDim.x >> 6;
  const int n0 = blockIdx.x * 16;
  const bf16_t* wp = w + (size_t)min(n0 + ln, N - 1) * K + 8 * lg;
  const bf16_t* xp[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) xp[t] = x + (size_t)min(16 * t + ln, M - 1) * ldx + 8 * lg;
  gs_f32x4_t acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = gs_f32x4_t{0.f, 0.f, 0.f, 0.f};

  const int kb = wave * k_per_wave;
  const int ke = min(K, kb + k_per_wave);
  for (int k = kb; k < ke; k += 32 * U) {
    GsFrag wf[U], xf[MT][U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kk = k + 32 * u;
      const bool ok = kk + 8 * lg < ke;
      wf[u].u = ok ? *reinterpret_cast<const uint4*>(wp + kk) : make_uint4(0, 0, 0, 0);
#pragma unroll
      for (int t = 0; t < MT; ++t)   // columns past the last row of x are never stored: no load
        xf[t][u].u = (ok && 16 * t + ln < M) ? *reinterpret_cast<const uint4*>(xp[t] + kk)
                                             : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int t = 0; t < MT; ++t)
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[u].v, xf[t][u].v, acc[t], 0, 0, 0);
  }

  if (nwaves > 1) {
#pragma unroll
    for (int t = 0; t < MT; ++t)
      *reinterpret_cast<gs_f32x4_t*>(red + (((size_t)wave * MT + t) * 64 + lane) * 4) = acc[t];
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int t = 0; t < MT; ++t)
      for (int wv = 1; wv < nwaves; ++wv) {
        const gs_f32x4_t o = *reinterpret_cast<const gs_f32x4_t*>(red + (((size_t)wv * MT + t) * 64 + lane) * 4);
        acc[t] += o;
      }
  }
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = 16 * t + ln;
    if (m >= M) continue;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = n0 + 4 * lg + i;
      if (n < N) y[(size_t)m * ldy + n] = from_float<TY>(acc[t][i]);
    }
  }
}

template <int MT, int U>
static int launch_skinny(void* y, const void* x, const void* w, int M, int N, int K, long ldx,
                         long ldy, int out_dtype, hipStream_t stream) {
  const int blocks = (N + 15) / 16;
  // enough waves to keep every SIMD of 256 CUs busy a few times over, each with
  // at least 256 elements of K to stream
  // (measured on MI355X: 4 waves a workgroup are best from N = 2048 to N = 128256 at
  // K = 2048, 8 to 16 at K = 8192)
  int waves = 1;
  while (waves < 16 && (long)blocks * waves < 4096 && K / (waves * 2) >= 256) waves <<= 1;
  if (waves < 4 && K >= 1024) waves = 4;
  int k_per_wave = ((K + waves - 1) / waves + 31) / 32 * 32;
  const size_t lds = waves > 1 ? (size_t)waves * MT * 64 * 4 * sizeof(float) : 0;
  if (out_dtype == PTL_DTYPE_F32)
    gemm_skinny_kernel<MT, U, float><<<blocks, waves * 64, lds, stream>>>(
        (float*)y, (const bf16_t*)x, (const bf16_t*)w, M, N, K, ldx, ldy, k_per_wave);
  else
    gemm_skinny_kernel<MT, U, bf16_t><<<blocks, waves * 64, lds, stream>>>(
        (bf16_t*)y, (const bf16_t*)x, (const bf16_t*)w, M, N, K, ldx, ldy, k_per_wave);
  return ptl_launch_status();
}

extern "C" int ptl_gemm_skinny_bf16(void* y, const void* x, const void* w, int M, int N, int K,
                                    long ldx, long ldy, int out_dtype, hipStream_t stream) {
  if (M <= 0 || N <= 0) return PTL_OK;
  if (M > 64 || K <= 0 || K % 8 || ldx % 8 || ldx < K || ldy < N ||
      (out_dtype != PTL_DTYPE_F32 && out_dtype != PTL_DTYPE_BF16))
    return PTL_ERR_ARG;
  if (M <= 16) return launch_skinny<1, 8>(y, x, w, M, N, K, ldx, ldy, out_dtype, stream);
  if (M <= 32) return launch_skinny<2, 4>(y, x, w, M, N, K, ldx, ldy, out_dtype, stream);
  return launch_skinny<4, 4>(y, x, w, M, N, K, ldx, ldy, out_dtype, stream);
}
