// y = x W^T for row-major x [M, K] (row stride ldx) and W [N, K]: every linear
// layer of the model (the reference uses cuBLAS through nn.Linear / F.linear,
// lite_llama/models/llama.py:37-40,61,120,221).
//
// ptl_gemm_nt: a tiled vector-FMA kernel with float32 accumulation for any
// M, N, K and any mix of float32 / bfloat16 inputs and outputs. It is the whole
// matrix path of the true 32-bit mode (no reduced-precision matrix mode can
// hide in it) and the fallback of the bfloat16 mode.
#include "common.h"
#include <stdlib.h>

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

// x for few rows, with fewer load instructions. The MFMA takes x^T as B: lane (ln, lg) holds
// row ln of x, 8 elements of k-group lg, for one block of 32 k. With M <= XR rows (XR = 4 or 8)
// only the lanes ln < XR of a block matter, so one load instruction fetches 16 / XR blocks at
// once: lane ln asks for row ln % XR of block ln / XR. Block j then reaches the lanes ln < XR by
// a shift of XR * j lanes inside the rows of 16 lanes (DPP row_shl, no memory and no LDS). The
// other lanes of a shifted fragment hold rows of other blocks or zeros: they feed result
// columns m >= XR >= M, which are never stored. Halving the load instructions of x at 8 rows
// took 60 us off a decode step of 1.15 ms: the instructions count, not the bytes.
template <int SH>
__device__ __forceinline__ uint4 gs_from_lane_up(uint4 v) {      // lane i <- lane i + SH of its row
  constexpr int ctrl = 0x100 + SH;                               // row_shl:SH
  uint4 r;
  r.x = __builtin_amdgcn_update_dpp(0, (int)v.x, ctrl, 0xf, 0xf, true);
  r.y = __builtin_amdgcn_update_dpp(0, (int)v.y, ctrl, 0xf, 0xf, true);
  r.z = __builtin_amdgcn_update_dpp(0, (int)v.z, ctrl, 0xf, 0xf, true);
  r.w = __builtin_amdgcn_update_dpp(0, (int)v.w, ctrl, 0xf, 0xf, true);
  return r;
}
__device__ __forceinline__ uint4 gs_from_lane_up_by(uint4 v, int sh) {   // sh: a constant after unrolling
  switch (sh) {
    case 4: return gs_from_lane_up<4>(v);
    case 8: return gs_from_lane_up<8>(v);
    case 12: return gs_from_lane_up<12>(v);
    default: return v;
  }
}
// blocks of 32 k that one load instruction fetches with XR rows a block (at most U of them)
template <int XR, int U> struct GsPack { static constexpr int P = (16 / XR < U) ? 16 / XR : U; };
// (measured: packing finer than four rows a block, for one or two rows, gains nothing more)
static int gs_rows_of(int M) { return M <= 4 ? 4 : M <= 8 ? 8 : 16; }

// Where a lane finds its 8 elements of weight row r from column 8 * lg on. Row-major: the rows of
// a 16-row tile lie K elements apart, and one load instruction of a wave touches 16 pieces of 64
// bytes. BLOCKED: a second copy of W (made once, for the decode kernels only) cut into tiles of
// 16 rows x 32 columns, each tile row-major in 1 KB, the tiles of a row block one after the other
// along K: a load instruction of a wave reads 1 KB in one piece (512 bytes for an 8-row tile), a
// wave's batch of eight 8 KB. Going from columns k to k + 32 is 512 elements there (GS_KSTEP).
template <bool BLOCKED>
__device__ __forceinline__ const bf16_t* gs_row_ptr(const bf16_t* w, int r, int K, int lg) {
  if (BLOCKED) return w + ((size_t)(r >> 4) * (K >> 5) * 512 + (r & 15) * 32 + 8 * lg);
  return w + (size_t)r * K + 8 * lg;
}
#define GS_KSTEP(BLOCKED) ((BLOCKED) ? 16 : 1)

// The follow-up of a product whose result is added to the residual stream and normalised
// (ptl_gemm_skinny_add_norm_bf16). The normalisation needs the whole row, which no workgroup
// has, so the product's kernel does what it can see: s = round_bf16(x W^T) + residual, the
// sum written back as the new residual, y = bf16(s * norm_w) and the sum of s^2 over the
// workgroup's columns into partials[m][workgroup]. The kernel that consumes y multiplies its
// own results by rsqrt(mean(s^2) + eps), which it gets from the partials (RowScaleArgs).
struct AddNormArgs {
  bf16_t* residual;        // [M, N], row stride ldr; updated in place
  const float* norm_w;     // [N]
  float* partials;         // [M, gridDim.x]
  long ldr;
};

// ROWS: weight rows a workgroup owns: 16 fill the MFMA tile; 8 (half the tile idle) give twice
// the workgroups when N is so small that 16-row tiles would leave CUs without work.
// ADD_NORM: the epilogue described at AddNormArgs (MT = 1, bfloat16 output).
// XR: rows of x a packed load takes per block (see gs_from_lane_up); 16: no packing.
template <int MT, int U, int ROWS, typename TY, bool ADD_NORM = false, int XR = 16, bool BLOCKED = false>
__global__ void __launch_bounds__(1024)
gemm_skinny_kernel(TY* __restrict__ y, const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                   int M, int N, int K, long ldx, long ldy, int k_per_wave, AddNormArgs an) {
  extern __shared__ float red[];                 // [waves][MT][64][4]
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, ln = lane & 15, lg = lane >> 4;
  const int nwaves = blockDim.x >> 6;
  const int n0 = blockIdx.x * ROWS;
  const bool wrow = ln < ROWS;
  const bf16_t* wp = gs_row_ptr<BLOCKED>(w, min(n0 + min(ln, ROWS - 1), N - 1), K, lg);
  static_assert(XR == 16 || MT == 1, "packed loads of x are for one tile of rows");
  constexpr int P = GsPack<XR, U>::P;          // blocks a load instruction of x fetches
  const int xrow = ln % XR, xblock = ln / XR;
  const bf16_t* xp[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t)
    xp[t] = x + (size_t)min(16 * t + xrow, M - 1) * ldx + 8 * lg + 32 * (xblock < P ? xblock : 0);
  gs_f32x4_t acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = gs_f32x4_t{0.f, 0.f, 0.f, 0.f};

  const int kb = wave * k_per_wave;
  const int ke = min(K, kb + k_per_wave);
  // Two sets of weight registers: the loads of the next 32 U columns are under way while
  // this set is multiplied, and a wave with at most 64 U columns has asked for all of its
  // weights before it waits for any. x, which lies in L2, is fetched as it is needed.
  GsFrag wa[U], wb[U], xf[MT][U / P];
  auto load_w = [&](GsFrag (&wf)[U], int k) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const bool ok = k + 32 * u + 8 * lg < ke && wrow;
      wf[u].u = ok ? load_once(wp + (k + 32 * u) * GS_KSTEP(BLOCKED)) : make_uint4(0, 0, 0, 0);
    }
  };
  auto multiply = [&](GsFrag (&wf)[U], int k) {
#pragma unroll
    for (int v = 0; v < U / P; ++v) {
      const bool ok = xblock < P && k + 32 * (v * P + xblock) + 8 * lg < ke;
#pragma unroll
      for (int t = 0; t < MT; ++t)   // columns past the last row of x are never stored: no load
        xf[t][v].u = (ok && 16 * t + xrow < M) ? *reinterpret_cast<const uint4*>(xp[t] + k + 32 * v * P)
                                               : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        GsFrag f;
        f.u = gs_from_lane_up_by(xf[t][u / P].u, XR * (u % P));
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[u].v, f.v, acc[t], 0, 0, 0);
      }
  };
  if (kb < ke) load_w(wa, kb);
  // what the epilogue of the first wave adds and multiplies by, asked for behind the first
  // weights: it is there long before the sums of the waves have met
  float res_in[4] = {0.f, 0.f, 0.f, 0.f}, nw_in[4] = {0.f, 0.f, 0.f, 0.f};
  // a lane's four columns as one access each where strides and pointers allow it
  const bool four = (N & 3) == 0 && (ldy & 3) == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0 &&
                    (!ADD_NORM || ((an.ldr & 3) == 0 && (reinterpret_cast<uintptr_t>(an.residual) & 7) == 0 &&
                                   (reinterpret_cast<uintptr_t>(an.norm_w) & 15) == 0));
  if (ADD_NORM && wave == 0 && ln < M && 4 * lg < ROWS && n0 + 4 * lg < N) {
    if (four) {
      union { uint2 u; bf16_t e[4]; } r;
      r.u = *reinterpret_cast<const uint2*>(an.residual + (size_t)ln * an.ldr + n0 + 4 * lg);
      const float4 w4 = *reinterpret_cast<const float4*>(an.norm_w + n0 + 4 * lg);
      nw_in[0] = w4.x; nw_in[1] = w4.y; nw_in[2] = w4.z; nw_in[3] = w4.w;
#pragma unroll
      for (int i = 0; i < 4; ++i) res_in[i] = bf16_to_float(r.e[i]);
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = n0 + 4 * lg + i;
        if (n < N) {
          res_in[i] = bf16_to_float(an.residual[(size_t)ln * an.ldr + n]);
          nw_in[i] = an.norm_w[n];
        }
      }
    }
  }
  for (int k = kb; k < ke; k += 64 * U) {
    const int k1 = k + 32 * U, k2 = k + 64 * U;
    if (k1 < ke) load_w(wb, k1);
    multiply(wa, k);
    if (k1 >= ke) break;
    if (k2 < ke) load_w(wa, k2);
    multiply(wb, k1);
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
  if (ADD_NORM) {
    const int m = ln;
    float ss = 0.f;
    if (four && sizeof(TY) == 2) {
      if (m < M && 4 * lg < ROWS && n0 + 4 * lg < N) {
        union { uint2 u; bf16_t e[4]; } r, o;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          // as the separate kernels do it: the product rounded to bfloat16, the sum in float32
          const float f = round_to<bf16_t>(acc[0][i]) + res_in[i];
          r.e[i] = float_to_bf16(f);
          o.e[i] = float_to_bf16(f * nw_in[i]);
          ss += f * f;
        }
        *reinterpret_cast<uint2*>(an.residual + (size_t)m * an.ldr + n0 + 4 * lg) = r.u;
        *reinterpret_cast<uint2*>(reinterpret_cast<bf16_t*>(y) + (size_t)m * ldy + n0 + 4 * lg) = o.u;
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = n0 + 4 * lg + i;
        if (m < M && 4 * lg + i < ROWS && n < N) {
          const float f = round_to<bf16_t>(acc[0][i]) + res_in[i];
          an.residual[(size_t)m * an.ldr + n] = float_to_bf16(f);
          y[(size_t)m * ldy + n] = from_float<TY>(f * nw_in[i]);
          ss += f * f;
        }
      }
    }
    ss += __shfl_xor(ss, 16, 64);
    ss += __shfl_xor(ss, 32, 64);
    if (lg == 0 && m < M) an.partials[(size_t)m * gridDim.x + blockIdx.x] = ss;
    return;
  }
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = 16 * t + ln;
    if (m >= M) continue;
    if (four) {
      if (4 * lg < ROWS && n0 + 4 * lg < N) {
        TY* at = y + (size_t)m * ldy + n0 + 4 * lg;
        if (sizeof(TY) == 4) {
          *reinterpret_cast<float4*>(at) = make_float4(acc[t][0], acc[t][1], acc[t][2], acc[t][3]);
        } else {
          union { uint2 u; bf16_t e[4]; } o;
#pragma unroll
          for (int i = 0; i < 4; ++i) o.e[i] = float_to_bf16(acc[t][i]);
          *reinterpret_cast<uint2*>(at) = o.u;
        }
      }
      continue;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = n0 + 4 * lg + i;
      if (4 * lg + i < ROWS && n < N) y[(size_t)m * ldy + n] = from_float<TY>(acc[t][i]);
    }
  }
}

// Compute units of the current device (256 on MI355X), asked for once a device: the launch
// rules below were measured there and are stated in compute units, not as numbers of that chip.
static int compute_units() {
  constexpr int MAX_DEVICES = 64;
  static int cached[MAX_DEVICES];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) {
    (void)hipGetLastError();
    return 256;
  }
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
      (void)hipGetLastError();
      n = 256;
    }
    cached[dev] = n;
  }
  return cached[dev];
}

template <int MT, int U, int ROWS>
static int launch_skinny_rows(void* y, const void* x, const void* w, int M, int N, int K, long ldx,
                              long ldy, int out_dtype, hipStream_t stream,
                              const AddNormArgs* an = nullptr, bool blocked = false) {
  if (blocked && K % 32) return PTL_ERR_ARG;
  const int blocks = (N + ROWS - 1) / ROWS;
  // enough waves to keep every SIMD of the chip busy a few times over (16 waves a compute
  // unit), each with at least 256 elements of K to stream
  // (measured on MI355X: 4 waves a workgroup are best from N = 2048 to N = 128256 at
  // K = 2048, 8 to 16 at K = 8192)
  int waves = 1;
  while (waves < 16 && (long)blocks * waves < 16L * compute_units() && K / (waves * 2) >= 256) waves <<= 1;
  if (waves < 4 && K >= 1024) waves = 4;
  int k_per_wave = ((K + waves - 1) / waves + 31) / 32 * 32;
  const size_t lds = waves > 1 ? (size_t)waves * MT * 64 * 4 * sizeof(float) : 0;
  const int xr = MT == 1 ? gs_rows_of(M) : 16;
#define GO1(TY, AN, XR, BL, args)                                                                    \
  gemm_skinny_kernel<(XR == 16 ? MT : 1), U, ROWS, TY, AN, XR, BL><<<blocks, waves * 64, lds, stream>>>( \
      (TY*)y, (const bf16_t*)x, (const bf16_t*)w, M, N, K, ldx, ldy, k_per_wave, args)
#define GO(TY, AN, XR, args)                                                                         \
  if (blocked) GO1(TY, AN, XR, true, args); else GO1(TY, AN, XR, false, args)
#define BY_ROWS(TY, AN, args)                                                                        \
  switch (xr) {                                                                                      \
    case 4: GO(TY, AN, 4, args); break;                                                              \
    case 8: GO(TY, AN, 8, args); break;                                                              \
    default: GO(TY, AN, 16, args); break;                                                            \
  }
  if (an != nullptr) {
    if (MT != 1 || out_dtype != PTL_DTYPE_BF16) return PTL_ERR_ARG;
    BY_ROWS(bf16_t, true, *an)
  } else if (out_dtype == PTL_DTYPE_F32) {
    BY_ROWS(float, false, AddNormArgs{})
  } else {
    BY_ROWS(bf16_t, false, AddNormArgs{})
  }
#undef BY_ROWS
#undef GO
#undef GO1
  return ptl_launch_status();
}

// weight rows a workgroup of the skinny kernel owns: 8 while 16-row tiles would leave more than
// three compute units in eight without one (160 tiles on 256 compute units)
static int few_tiles() { return compute_units() * 5 / 8; }
static int skinny_rows(int N) { return (N + 15) / 16 <= few_tiles() ? 8 : 16; }

template <int MT, int U>
static int launch_skinny(void* y, const void* x, const void* w, int M, int N, int K, long ldx,
                         long ldy, int out_dtype, hipStream_t stream,
                         const AddNormArgs* an = nullptr, bool blocked = false) {
  // measured on MI355X at K = 2048 and 8192: N = 2048 (128 tiles of 16 rows) gains 10 to 20 %
  // from 8-row tiles, N = 3072 (192 tiles) loses
  if (skinny_rows(N) == 8)
    return launch_skinny_rows<MT, U, 8>(y, x, w, M, N, K, ldx, ldy, out_dtype, stream, an, blocked);
  return launch_skinny_rows<MT, U, 16>(y, x, w, M, N, K, ldx, ldy, out_dtype, stream, an, blocked);
}

// w_blocked != 0: ``w`` is the blocked copy of the matrix (see gs_row_ptr; rows padded to a
// multiple of 16, K a multiple of 32).
extern "C" int ptl_gemm_skinny_bf16(void* y, const void* x, const void* w, int w_blocked, int M, int N,
                                    int K, long ldx, long ldy, int out_dtype, hipStream_t stream) {
  if (M <= 0 || N <= 0) return PTL_OK;
  if (M > 64 || K <= 0 || K % 8 || ldx % 8 || ldx < K || ldy < N ||
      (out_dtype != PTL_DTYPE_F32 && out_dtype != PTL_DTYPE_BF16) || (w_blocked && K % 32))
    return PTL_ERR_ARG;
  const bool bl = w_blocked != 0;
  if (M <= 16) return launch_skinny<1, 8>(y, x, w, M, N, K, ldx, ldy, out_dtype, stream, nullptr, bl);
  if (M <= 32) return launch_skinny<2, 4>(y, x, w, M, N, K, ldx, ldy, out_dtype, stream, nullptr, bl);
  return launch_skinny<4, 2>(y, x, w, M, N, K, ldx, ldy, out_dtype, stream, nullptr, bl);
}

// How many partial sums a row gets from ptl_gemm_skinny_add_norm_bf16 with N columns (on the
// current device: the tile height follows its number of compute units).
extern "C" int ptl_gemm_skinny_partials(int N) {
  const int rows = skinny_rows(N);
  return (N + rows - 1) / rows;
}

// y = bf16((x W^T + residual) * norm_w), residual <- x W^T + residual, partials[m][j] = sums of
// squares of the new residual over column blocks (ptl_gemm_skinny_partials(N) of them a row):
// see AddNormArgs. M <= 16.
extern "C" int ptl_gemm_skinny_add_norm_bf16(void* y, const void* x, const void* w, int w_blocked,
                                             void* residual, const float* norm_w, float* partials,
                                             int M, int N, int K, long ldx, long ldy, long ldr,
                                             hipStream_t stream) {
  if (M <= 0 || N <= 0) return PTL_OK;
  if (M > 16 || K <= 0 || K % 8 || ldx % 8 || ldx < K || ldy < N || ldr < N || !residual ||
      !norm_w || !partials || (w_blocked && K % 32))
    return PTL_ERR_ARG;
  const AddNormArgs an = {(bf16_t*)residual, norm_w, partials, ldr};
  return launch_skinny<1, 8>(y, x, w, M, N, K, ldx, ldy, PTL_DTYPE_BF16, stream, &an, w_blocked != 0);
}

// ===========================================================================
// Decode-step products with their follow-up fused in, for at most 16 rows of x:
//
// ptl_gate_up_silu_bf16:  out[m, c] = silu(x . Wg[c]) * (x . Wu[c])   (W = [Wg; Wu], [2I, K])
// ptl_qkv_rope_store_bf16: q, k, v = x . Wqkv^T; q and k rotated by the angles
//     positions[m] * inv_freq[j] on the pairs (j, j + D/2); q written out, the
//     rotated k and v written into the cache pages at slots[m].
//
// Both are the skinny kernel above with two 16-row weight tiles per workgroup,
// chosen so that the two values an output needs meet in one lane of the result
// tile: gate row c with up row I + c; column j of a head with column j + D/2.
// They replace a product, an element-wise kernel and the trip through memory
// between them (lite_llama/models/llama.py:75-90 runs q_proj, kv_proj, the rotary
// kernel and the cache copy one after the other; :120 gate, up, SwiGLU, down).
// The projections are rounded to bfloat16 before the follow-up, as the unfused path
// stores them, so both paths agree to the order of the sums.
// ===========================================================================
#define PAIR_SILU 0
#define PAIR_ROPE 1

struct RopeStoreArgs {
  const int32_t* positions;   // [M]
  const float* inv_freq;      // [D/2] or null: no rotation
  const int32_t* slots;       // [M] or null: no store
  bf16_t* k_cache;            // [pages, Hkv, page_size, D]
  bf16_t* v_cache;
  int Hq, Hkv, D, page_size;
};

// Rows of x that still lack their normalisation factor (see AddNormArgs): the results of row m
// are multiplied by rsqrt(sum_j partials[m][j] * inv_n + eps). partials == null: no factor.
struct RowScaleArgs {
  const float* partials;   // [M, count]
  int count;
  float inv_n, eps;
};

template <int MODE, int U, int ROWS, int XR, bool BLOCKED>
__global__ void __launch_bounds__(1024)
gemm_pair_kernel(bf16_t* __restrict__ y, const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                 int M, int N_out, int K, long ldx, long ldy, int k_per_wave, int pair_offset,
                 int tiles_per_group, int group_rows, RopeStoreArgs rs, RowScaleArgs sc) {
  extern __shared__ float red[];                 // [waves][2][64][4]
  __shared__ float row_factor[16];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, ln = lane & 15, lg = lane >> 4;
  const int nwaves = blockDim.x >> 6;
  // workgroup b takes tile (b % tiles_per_group) of group (b / tiles_per_group): rows
  // r1 .. r1+15 and r1 + pair_offset .. of W. SiLU: one group, tiles over I. Rope: a
  // group is a head (group_rows = D), its tiles cover the first half of the head.
  const int group = blockIdx.x / tiles_per_group;
  const int tile = blockIdx.x - group * tiles_per_group;
  // (ROWS = 8: half of the MFMA tile idle, twice the workgroups, for products with few rows)
  const int r1 = group * group_rows + ROWS * tile;
  const int r2 = r1 + pair_offset;
  const bool wrow = ln < ROWS;
  const bf16_t* wp1 = gs_row_ptr<BLOCKED>(w, r1 + min(ln, ROWS - 1), K, lg);
  const bf16_t* wp2 = gs_row_ptr<BLOCKED>(w, r2 + min(ln, ROWS - 1), K, lg);
  constexpr int P = GsPack<XR, U>::P;          // blocks a load instruction of x fetches
  const int xrow = ln % XR, xblock = ln / XR;
  const bf16_t* xp = x + (size_t)min(xrow, M - 1) * ldx + 8 * lg + 32 * (xblock < P ? xblock : 0);
  gs_f32x4_t acc1 = {0.f, 0.f, 0.f, 0.f}, acc2 = {0.f, 0.f, 0.f, 0.f};

  const int kb = wave * k_per_wave;
  const int ke = min(K, kb + k_per_wave);
  GsFrag w1[U], w2[U], xf[U / P];
  auto load_w = [&](int k) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const bool ok = k + 32 * u + 8 * lg < ke && wrow;
      w1[u].u = ok ? load_once(wp1 + (k + 32 * u) * GS_KSTEP(BLOCKED)) : make_uint4(0, 0, 0, 0);
      w2[u].u = ok ? load_once(wp2 + (k + 32 * u) * GS_KSTEP(BLOCKED)) : make_uint4(0, 0, 0, 0);
    }
  };
  auto load_x = [&](int k) {
#pragma unroll
    for (int v = 0; v < U / P; ++v) {
      const bool ok = xblock < P && k + 32 * (v * P + xblock) + 8 * lg < ke && xrow < M;
      xf[v].u = ok ? *reinterpret_cast<const uint4*>(xp + k + 32 * v * P) : make_uint4(0, 0, 0, 0);
    }
  };
  // The first weights set out before anything else: they come from HBM and are what the
  // kernel's time goes to. The rows' factors (a few dependent reads of L2) are worked out
  // while they fly; x, which lies in L2, follows.
  // The loads are answered in the order they were asked: the partial sums of this wave's row
  // first (a wait for them then leaves the weights under way), then the first weights, which
  // come from HBM and are what the kernel's time goes to; the row's factor is worked out while
  // they fly, and x, which lies in L2, follows.
  const bool my_row = sc.partials != nullptr && wave < M;
  const float* prow = sc.partials + (size_t)(my_row ? wave : 0) * sc.count;
  float part[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) part[u] = (my_row && lane + 64 * u < sc.count) ? prow[lane + 64 * u] : 0.f;
  int k = kb;
  if (k < ke) load_w(k);
  // rotation mode: the position and the cache slot that the epilogue of the first wave needs,
  // asked for behind the first weights
  float pos_in = 0.f;
  int slot_in = -1;
  if (MODE == PAIR_ROPE && wave == 0 && ln < M) {
    pos_in = (float)rs.positions[ln];
    slot_in = rs.slots ? rs.slots[ln] : -1;
  }
  if (sc.partials != nullptr) {
    // the waves share the rows; a row's partial sums are added in a fixed order
    for (int m = wave; m < M; m += nwaves) {
      const float* row = sc.partials + (size_t)m * sc.count;
      float sum = 0.f;
      if (m == wave) {
        sum = (part[0] + part[1]) + (part[2] + part[3]);
        for (int j = lane + 256; j < sc.count; j += 64) sum += row[j];
      } else {
        for (int j = lane; j < sc.count; j += 64) sum += row[j];
      }
      sum = wave_sum(sum);
      if (lane == 0) row_factor[m] = 1.0f / sqrtf(sum * sc.inv_n + sc.eps);
    }
  }
  while (k < ke) {
    load_x(k);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      GsFrag f;
      f.u = gs_from_lane_up_by(xf[u / P].u, XR * (u % P));
      acc1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w1[u].v, f.v, acc1, 0, 0, 0);
      acc2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w2[u].v, f.v, acc2, 0, 0, 0);
    }
    k += 32 * U;
    if (k < ke) load_w(k);
  }
  // sines and cosines while the other waves finish
  float sn_in[4] = {0.f, 0.f, 0.f, 0.f}, cs_in[4] = {1.f, 1.f, 1.f, 1.f};
  if (MODE == PAIR_ROPE && wave == 0 && rs.inv_freq && group < rs.Hq + rs.Hkv) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (4 * lg + i < ROWS) sincosf(pos_in * rs.inv_freq[ROWS * tile + 4 * lg + i], &sn_in[i], &cs_in[i]);
  }
  if (nwaves > 1) {
    *reinterpret_cast<gs_f32x4_t*>(red + (((size_t)wave * 2 + 0) * 64 + lane) * 4) = acc1;
    *reinterpret_cast<gs_f32x4_t*>(red + (((size_t)wave * 2 + 1) * 64 + lane) * 4) = acc2;
    __syncthreads();
    if (wave != 0) return;
    for (int wv = 1; wv < nwaves; ++wv) {
      acc1 += *reinterpret_cast<const gs_f32x4_t*>(red + (((size_t)wv * 2 + 0) * 64 + lane) * 4);
      acc2 += *reinterpret_cast<const gs_f32x4_t*>(red + (((size_t)wv * 2 + 1) * 64 + lane) * 4);
    }
  }
  const int m = ln;                 // the result tiles hold rows 4*lg+i of W, column m of x^T
  if (sc.partials != nullptr) {
    if (nwaves == 1) __syncthreads();            // (more waves: the barrier above was passed)
    const float f = row_factor[min(m, M - 1)];
#pragma unroll
    for (int i = 0; i < 4; ++i) { acc1[i] *= f; acc2[i] *= f; }
  }
  if (m >= M) return;
  if (MODE == PAIR_SILU) {
    union { uint2 u; bf16_t e[4]; } o;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      // the gate and up products are rounded to bfloat16 as the unfused path stores them
      const float g = round_to<bf16_t>(acc1[i]), u = round_to<bf16_t>(acc2[i]);
      o.e[i] = float_to_bf16(g / (1.0f + expf(-g)) * u);
    }
    const int c0 = r1 + 4 * lg;
    if ((N_out & 3) == 0 && (ldy & 3) == 0 && (reinterpret_cast<uintptr_t>(y) & 7) == 0) {
      // a lane's four columns as one 8-byte store
      if (4 * lg < ROWS && c0 < N_out) *reinterpret_cast<uint2*>(y + (size_t)m * ldy + c0) = o.u;
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (4 * lg + i < ROWS && c0 + i < N_out) y[(size_t)m * ldy + c0 + i] = o.e[i];
    }
  } else {
    const int D = rs.D, half = D >> 1;
    const int head = group;                      // 0..Hq-1: q; then Hkv k heads; then Hkv v heads
    const bool is_q = head < rs.Hq, is_k = !is_q && head < rs.Hq + rs.Hkv;
    const int slot = slot_in;
    bf16_t* dst = nullptr;
    if (is_q) {
      dst = y + (size_t)m * ldy + (size_t)head * D;
    } else if (slot >= 0) {
      const int kvh = is_k ? head - rs.Hq : head - rs.Hq - rs.Hkv;
      const int page = slot / rs.page_size, off = slot - page * rs.page_size;
      dst = (is_k ? rs.k_cache : rs.v_cache) + (((size_t)page * rs.Hkv + kvh) * rs.page_size + off) * D;
    }
    if (dst == nullptr) return;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (4 * lg + i >= ROWS) continue;
      const int j = ROWS * tile + 4 * lg + i;    // column in the first half of the head
      // as in the unfused path, the projection is rounded to bfloat16 before the rotation
      float x1 = round_to<bf16_t>(acc1[i]), x2 = round_to<bf16_t>(acc2[i]);
      if ((is_q || is_k) && rs.inv_freq) {
        const float o1 = x1 * cs_in[i] - x2 * sn_in[i], o2 = x2 * cs_in[i] + x1 * sn_in[i];
        x1 = o1; x2 = o2;
      }
      dst[j] = float_to_bf16(x1);
      dst[j + half] = float_to_bf16(x2);
    }
  }
}

static int pair_waves(int blocks, int K) {
  int waves = 1;
  while (waves < 16 && (long)blocks * waves < 16L * compute_units() && K / (waves * 2) >= 256) waves <<= 1;
  if (waves < 4 && K >= 1024) waves = 4;
  return waves;
}

// out [M, I] = silu(x Wg^T) * (x Wu^T) for W = [Wg; Wu] of shape [2I, K]; M <= 16, I % 16 == 0
// partials / n_partials / eps: the normalisation factor of x's rows that is still to be applied
// (RowScaleArgs; K is the size of the normalised rows); partials == null: none.
// w_blocked: as for ptl_gemm_skinny_bf16
extern "C" int ptl_gate_up_silu_bf16(void* out, const void* x, const void* w, int w_blocked, int M, int I,
                                     int K, long ldx, const float* partials, int n_partials, float eps,
                                     hipStream_t stream) {
  if (M <= 0 || I <= 0) return PTL_OK;
  if (M > 16 || I % 16 || K <= 0 || K % 8 || ldx % 8 || ldx < K || (partials && n_partials <= 0) ||
      (w_blocked && K % 32))
    return PTL_ERR_ARG;
  const RowScaleArgs sc = {partials, n_partials, 1.0f / (float)K, eps};
  const int blocks = I / 16;
  const int waves = pair_waves(blocks, K);
  const int k_per_wave = ((K + waves - 1) / waves + 31) / 32 * 32;
  const size_t lds = waves > 1 ? (size_t)waves * 2 * 64 * 4 * sizeof(float) : 0;
  RopeStoreArgs none = {};
#define GO1(XR, BL)                                                                                   \
  gemm_pair_kernel<PAIR_SILU, 8, 16, XR, BL><<<blocks, waves * 64, lds, stream>>>(                    \
      (bf16_t*)out, (const bf16_t*)x, (const bf16_t*)w, M, I, K, ldx, I, k_per_wave, I, blocks, 0, none, sc)
#define GO(XR) if (w_blocked) GO1(XR, true); else GO1(XR, false)
  switch (gs_rows_of(M)) {
    case 4: GO(4); break;
    case 8: GO(8); break;
    default: GO(16); break;
  }
#undef GO
#undef GO1
  return ptl_launch_status();
}

// q_out [M, Hq, D] (row stride ldq); w [(Hq + 2 Hkv) D, K] rows q | k | v; M <= 16, D % 32 == 0
extern "C" int ptl_qkv_rope_store_bf16(void* q_out, long ldq, const void* x, const void* w, int w_blocked,
                                       int M, int K, long ldx, const int32_t* positions,
                                       const float* inv_freq, const int32_t* slots, void* k_cache,
                                       void* v_cache, int Hq, int Hkv, int D, int page_size,
                                       const float* partials, int n_partials, float eps,
                                       hipStream_t stream) {
  if (M <= 0) return PTL_OK;
  if (M > 16 || Hq <= 0 || Hkv <= 0 || D <= 0 || D % 32 || K <= 0 || K % 8 || ldx % 8 || ldx < K ||
      ldq < (long)Hq * D || page_size <= 0 || !positions || (slots && (!k_cache || !v_cache)) ||
      (partials && n_partials <= 0) || (w_blocked && K % 32))
    return PTL_ERR_ARG;
  const RowScaleArgs sc = {partials, n_partials, 1.0f / (float)K, eps};
  // few heads: 8-column tiles, so that twice as many workgroups share the weight stream
  const bool small = (Hq + 2 * Hkv) * (D / 32) <= few_tiles();
  const int tiles = small ? D / 16 : D / 32;      // tiles in half a head
  const int blocks = (Hq + 2 * Hkv) * tiles;
  const int waves = pair_waves(blocks, K);
  const int k_per_wave = ((K + waves - 1) / waves + 31) / 32 * 32;
  const size_t lds = waves > 1 ? (size_t)waves * 2 * 64 * 4 * sizeof(float) : 0;
  RopeStoreArgs rs = {positions, inv_freq, slots, (bf16_t*)k_cache, (bf16_t*)v_cache, Hq, Hkv, D, page_size};
#define GO1(ROWS, XR, BL)                                                                             \
  gemm_pair_kernel<PAIR_ROPE, 8, ROWS, XR, BL><<<blocks, waves * 64, lds, stream>>>(                  \
      (bf16_t*)q_out, (const bf16_t*)x, (const bf16_t*)w, M, Hq * D, K, ldx, ldq, k_per_wave, D / 2,  \
      tiles, D, rs, sc)
#define GO(ROWS, XR) if (w_blocked) GO1(ROWS, XR, true); else GO1(ROWS, XR, false)
#define BY_ROWS(ROWS)                                                                                 \
  switch (gs_rows_of(M)) {                                                                            \
    case 4: GO(ROWS, 4); break;                                                                       \
    case 8: GO(ROWS, 8); break;                                                                       \
    default: GO(ROWS, 16); break;                                                                     \
  }
  if (small) { BY_ROWS(8) } else { BY_ROWS(16) }
#undef BY_ROWS
#undef GO
#undef GO1
  return ptl_launch_status();
}
