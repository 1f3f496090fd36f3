// The matrix products of a decode step with 9 to 128 rows (a batch of that many requests, one
// token each), in bfloat16 on the matrix cores, with what follows a product done in its epilogue
// or in one kernel behind it:
//   ptl_rows_gemm_bf16        y = x W^T (bfloat16 or float32), or its float32 partial sums over
//                             slices of K, one slice a workgroup, for the two kernels below
//   ptl_rows_sum_add_rmsnorm  sum of those partial sums + residual + RMSNorm (whole rows)
//   ptl_rows_sum_rope_store   sum of the partial sums of a q | k | v projection, rotation of q
//                             and k, k and v into the cache pages
//   ptl_rows_gate_up_silu     silu(x Wg^T) * (x Wu^T)
// The reference runs these products through cuBLAS and the rest as kernels of their own
// (lite_llama/models/llama.py:37-40,120, lite_llama/kernels/rope_emb.py, swiglu.py,
// skip_rmsnorm.py).
//
// Such a step is bound by reading every weight once from HBM, like the steps of fewer rows
// (gemm.hip), but its x is up to 8 MFMA tiles tall: a workgroup that owned 16 weight rows and
// fetched its x from L2 would read 4 to 8 times more of x than of W, in half cache lines, and
// the chip's L2 would be the bound (measured: 1.0 to 1.5 TB/s of weights). So here
//   * a workgroup has four waves that multiply, each owning one tile of 16 weight rows and all
//     rows of x (64 weight rows a workgroup), and a fifth wave that does nothing but bring x
//     into LDS, chunk of K by chunk, two chunks ahead, with loads that go from global memory
//     straight to LDS (no register in between). A wave's loads are answered in the order it
//     asked, so a wave that fetched x between its weights could never have more than one
//     chunk of weights under way; with a wave of its own for x the four others keep DEPTH
//     chunks of W in flight, which is what reading HBM at its rate takes;
//   * x lies in LDS row-major without padding, the 16-byte pieces of a row permuted by the row
//     number (piece p of row r at p ^ (r % 16)), which spreads the 16 rows that a fragment
//     read touches over all banks;
//   * W comes from the blocked copy (tiles of 16 rows x 32 columns in 1 KB, see gs_row_ptr in
//     gemm.hip) straight into registers: a load instruction of a wave is one contiguous KB;
//   * a matrix with few rows and a deep K (the output, down and q|k|v projections) is cut along K
//     among workgroups so that every compute unit still gets one; those leave float32 partial
//     sums, which the kernel that follows anyway (the norm, the rotation) adds up;
//   * the waves meet at one barrier a chunk (a bare s_barrier: the usual one would first wait
//     for every load a wave has under way), and no sums cross waves (pairs of tiles that an
//     epilogue combines, gate with up, meet in LDS once at the end).
#include "common.h"
#include "mfma.h"

namespace {

enum { MODE_PLAIN = 0, MODE_SILU = 1 };

constexpr int TILES = 4;                   // tiles of 16 weight rows a workgroup owns: 64 rows
constexpr int NB = 3;                      // chunks of x in LDS: one in use, two on their way
// Columns of a chunk (KC) and chunks of W a wave has under way (DEPTH) for 1, 2, 3, 4 and 8 tiles of
// x, with one tile of W a wave: 8 KB of weights a wave in flight, chunks of x of at most 32 KB.
// Measured at 64 rows and the 1B widths: 128 to 512 columns a chunk and 2 to 12 chunks under
// way differ by a few per cent. With two tiles a wave: 128 columns, 4 chunks (the head of
// vocabulary size: 112 us against 137 with 256 and 2).
constexpr int KC_1 = 256, DEPTH_1 = 2;
constexpr int KC_2 = 256, DEPTH_2 = 2;
constexpr int KC_3 = 256, DEPTH_3 = 2;
constexpr int KC_4 = 256, DEPTH_4 = 2;
constexpr int KC_8 = 128, DEPTH_8 = 4;

// element (row r, column 32 kb + 8 lg) of the blocked copy of a matrix with K columns
__device__ __forceinline__ const bf16_t* blocked_at(const bf16_t* w, int r, int K, int lg) {
  return w + ((size_t)(r >> 4) * (K >> 5) * 512 + (r & 15) * 32 + 8 * lg);
}

// All waves of the workgroup meet; nothing but the meeting (the loads a wave has under way
// stay under way). The clobbers keep the compiler from moving LDS accesses across it.
__device__ __forceinline__ void meet() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// s_waitcnt vmcnt(N) alone (expcnt and lgkmcnt left at their maxima)
template <int N> __device__ __forceinline__ void wait_loads_but() {
  static_assert(N >= 0 && N < 64, "vmcnt has six bits");
  __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
}

// MT: tiles of 16 rows of x. KC: columns a chunk (KC / 32 weight fragments a wave and chunk).
// DEPTH: chunks of W a wave has under way. MODE_PLAIN: wave w owns rows r0 + 16 w, y (or the
// partial sums of this workgroup's slice of K) gets the product. MODE_SILU: waves 0, 1 own gate
// rows r0 .. r0 + 31, waves 2, 3 the up rows r0 + I ..; out = silu(gate) * up.
template <int MT, int KC, int DEPTH, int WT, int MODE, typename TY>
__global__ void __launch_bounds__((4 / WT + 1) * 64)
gemm_rows_kernel(TY* __restrict__ y, const bf16_t* __restrict__ x, const bf16_t* __restrict__ wb,
                 int M, int N_out, int w_rows, int K, long ldx, long ldy, int k_per_split,
                 int pair_offset) {
  constexpr int FRAGS = KC / 32;                 // weight fragments a wave and chunk
  constexpr int PIECES = KC / 8;                 // 16-byte pieces of a row of a chunk of x
  constexpr int XI = MT * 16 * PIECES / 64;      // load instructions that bring a chunk of x
  constexpr int CHUNK = MT * 16 * KC;            // elements of a chunk of x
  static_assert(PIECES >= 16 && (PIECES & (PIECES - 1)) == 0, "rows of at least 16 pieces, a power of two");
  static_assert(NB >= 3 && NB <= 5 && (NB - 2) * XI < 64, "the loader waits by instruction counts of six bits");
  extern __shared__ __align__(16) unsigned char lds[];     // [NB][MT * 16][KC] bfloat16
  bf16_t* xs = reinterpret_cast<bf16_t*>(lds);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63, ln = lane & 15, lg = lane >> 4;
  const int k_lo = blockIdx.y * k_per_split;
  const int k_hi = min(K, k_lo + k_per_split);
  const int nchunks = (k_hi - k_lo + KC - 1) / KC;

  constexpr int WAVES = TILES / WT;              // waves that multiply, WT tiles of W each
  if (wave == WAVES) {
    // ---- the wave that brings x: chunk c into buffer c % NB, two chunks ahead ----
    // instruction i of a chunk fills the 64 pieces 64 i .. 64 i + 63 of the buffer, lane l the
    // l-th: piece s is row s / PIECES, place s % PIECES, and holds the row's piece
    // (s % PIECES) ^ (row % 16). Rows past M repeat the last row (their results are never
    // stored), columns past K the first of the chunk (they meet weights that are zero).
    int src[XI];                                 // element offsets into x, without k
#pragma unroll
    for (int i = 0; i < XI; ++i) {
      const int s_ = 64 * i + lane;
      const int row = s_ / PIECES, place = s_ - row * PIECES;
      src[i] = min(row, M - 1) * (int)ldx + 8 * (place ^ (row & 15));
    }
    auto fetch = [&](int c) {
      const int k = k_lo + c * KC;
      bf16_t* dst = xs + (size_t)(c % NB) * CHUNK;
#pragma unroll
      for (int i = 0; i < XI; ++i) {
        const int piece_col = 8 * (((64 * i + lane) % PIECES) ^ (((64 * i + lane) / PIECES) & 15));
        const int col = k + piece_col < K ? k + piece_col : k;
        __builtin_amdgcn_global_load_lds(
            (const __attribute__((address_space(1))) void*)(x + (size_t)(src[i] - piece_col) + col),
            (__attribute__((address_space(3))) void*)(dst + 512 * i), 16, 0, 0);
      }
    };
#pragma unroll
    for (int c = 0; c < NB - 1; ++c)
      if (c < nchunks) fetch(c);
    for (int c = 0; c < nchunks; ++c) {
      // chunk c has landed when at most the chunks after it are still under way
      switch (min(NB - 2, nchunks - 1 - c)) {
        case 0: wait_loads_but<0>(); break;
        case 1: wait_loads_but<XI>(); break;
        case 2: wait_loads_but<(NB > 3 ? 2 * XI : 0)>(); break;
        default: wait_loads_but<(NB > 4 ? 3 * XI : 0)>(); break;
      }
      meet();                                    // chunk c is there; chunk c - 1 has been used
      if (c + NB - 1 < nchunks) fetch(c + NB - 1);
    }
    if (MODE == MODE_SILU) { meet(); meet(); }
    return;
  }

  const int r0 = blockIdx.x * (TILES * 16) / (MODE == MODE_SILU ? 2 : 1);
  // tile g = WT * wave + j of the workgroup: rows r0 + 16 g, or, with gate and up rows, tiles
  // 0, 1 the gate rows r0 .. r0 + 31 and tiles 2, 3 the up rows r0 + pair_offset ..
  int tile_row[WT];
  const bf16_t* wp[WT];
#pragma unroll
  for (int j = 0; j < WT; ++j) {
    const int g = WT * wave + j;
    tile_row[j] = MODE == MODE_SILU ? r0 + (g >> 1) * pair_offset + 16 * (g & 1) : r0 + 16 * g;
    wp[j] = blocked_at(wb, min(tile_row[j] + ln, w_rows - 1), K, lg) + (size_t)(k_lo >> 5) * 512;
  }

  f32x4_t acc[WT][MT];
#pragma unroll
  for (int j = 0; j < WT; ++j)
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[j][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  Frag8 ring[DEPTH][FRAGS][WT];
  auto load_w = [&](Frag8 (&wf)[FRAGS][WT], int c) {
#pragma unroll
    for (int u = 0; u < FRAGS; ++u)
#pragma unroll
      for (int j = 0; j < WT; ++j)
        wf[u][j].u = (k_lo + c * KC + 32 * u < k_hi) ? load_once(wp[j] + (size_t)(c * FRAGS + u) * 512)
                                                     : make_uint4(0, 0, 0, 0);
  };
  // Every fragment of x that is read from LDS meets the WT tiles of W the wave owns. A chunk is
  // taken in stages of two column blocks: the fragments of the next stage are asked for, then
  // the products of this stage are made, so that LDS and the matrix cores work at the same
  // time (left to itself the compiler reads two fragments, waits, multiplies, reads two more,
  // and the wave, alone on its SIMD, stands through the latency of LDS eight times a chunk).
  constexpr int SK = 2;                          // column blocks a stage
  constexpr int STAGES = FRAGS / SK;             // stages a chunk: even, so that a stage's registers are known
  static_assert(FRAGS % (2 * SK) == 0, "an even number of stages a chunk");
  Frag8 xf[2][SK][MT];
  auto read_x = [&](Frag8 (&f)[SK][MT], int c, int h) {
    const bf16_t* xb = xs + (size_t)(c % NB) * CHUNK + (size_t)ln * KC;
#pragma unroll
    for (int u = 0; u < SK; ++u)
#pragma unroll
      for (int t = 0; t < MT; ++t)
        f[u][t].u = *reinterpret_cast<const uint4*>(xb + (size_t)t * 16 * KC + 8 * ((4 * (h * SK + u) + lg) ^ ln));
  };
  auto multiply = [&](Frag8 (&wf)[FRAGS][WT], Frag8 (&f)[SK][MT], int h) {
#pragma unroll
    for (int u = 0; u < SK; ++u)
#pragma unroll
      for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int j = 0; j < WT; ++j)
          acc[j][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[h * SK + u][j].v, f[u][t].v, acc[j][t], 0, 0, 0);
  };
  // DEPTH chunks of weights set out before anything else: they come from HBM and are what the
  // kernel's time goes to
#pragma unroll
  for (int d = 0; d < DEPTH; ++d)
    if (d < nchunks) load_w(ring[d], d);
  if (nchunks > 0) {
    meet();                                      // x of chunk 0 is in LDS
    read_x(xf[0], 0, 0);
  }
  for (int c0 = 0; c0 < nchunks; c0 += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const int c = c0 + d;
      if (c < nchunks) {
#pragma unroll
        for (int h = 0; h < STAGES; ++h) {
          if (h + 1 < STAGES) {
            read_x(xf[(h + 1) & 1], c, h + 1);
          } else if (c + 1 < nchunks) {
            // every read of chunk c has come back before the wave says that it is done with it
            __builtin_amdgcn_s_waitcnt(0xC07F);
            meet();                              // x of chunk c + 1 is in LDS; chunk c may be overwritten
            read_x(xf[0], c + 1, 0);
          }
          __builtin_amdgcn_sched_barrier(0);
          multiply(ring[d], xf[h & 1], h);
          __builtin_amdgcn_sched_barrier(0);
        }
        if (c + DEPTH < nchunks) load_w(ring[d], c + DEPTH);
      }
    }
  }

  // the lane holds rows 4 lg + i of a tile of W and row m = 16 t + ln of x
  if (MODE == MODE_PLAIN) {
#pragma unroll
    for (int j = 0; j < WT; ++j) {
      const int n0 = tile_row[j] + 4 * lg;
      TY* base = y + (size_t)blockIdx.y * M * ldy + n0;
      const bool four = n0 + 3 < N_out && (ldy & 3) == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0;
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const int m = 16 * t + ln;
        if (m >= M) continue;
        TY* at = base + (size_t)m * ldy;
        if (four) {
          if (sizeof(TY) == 4) {
            *reinterpret_cast<float4*>(at) = make_float4(acc[j][t][0], acc[j][t][1], acc[j][t][2], acc[j][t][3]);
          } else {
            union { uint2 u; bf16_t e[4]; } o;
#pragma unroll
            for (int i = 0; i < 4; ++i) o.e[i] = float_to_bf16(acc[j][t][i]);
            *reinterpret_cast<uint2*>(at) = o.u;
          }
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (n0 + i < N_out) at[i] = from_float<TY>(acc[j][t][i]);
        }
      }
    }
  } else {
    // the up tiles (2, 3) go through LDS (the chunks of x are done with) to the waves that hold
    // the gate tiles (0, 1)
    meet();
    float* ex = reinterpret_cast<float*>(lds);           // [2][MT][64][4]
#pragma unroll
    for (int j = 0; j < WT; ++j) {
      const int g = WT * wave + j;
      if (g >= 2) {
#pragma unroll
        for (int t = 0; t < MT; ++t)
          *reinterpret_cast<f32x4_t*>(ex + (((size_t)(g - 2) * MT + t) * 64 + lane) * 4) = acc[j][t];
      }
    }
    __builtin_amdgcn_s_waitcnt(0xC07F);            // lgkmcnt(0): the stores to LDS are done
    meet();
    bf16_t* out = reinterpret_cast<bf16_t*>(y);
#pragma unroll
    for (int j = 0; j < WT; ++j) {
      const int g = WT * wave + j;
      if (g >= 2) continue;
      const int c0 = r0 + 16 * g + 4 * lg;                // first of the lane's four output columns
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const int m = 16 * t + ln;
        if (m >= M) continue;
        const f32x4_t up = *reinterpret_cast<const f32x4_t*>(ex + (((size_t)g * MT + t) * 64 + lane) * 4);
        union { uint2 u; bf16_t e[4]; } o;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          // the gate and up products are rounded to bfloat16 as the unfused path stores them
          const float gt = round_to<bf16_t>(acc[j][t][i]), u = round_to<bf16_t>(up[i]);
          o.e[i] = float_to_bf16(gt / (1.0f + expf(-gt)) * u);
        }
        bf16_t* at = out + (size_t)m * ldy + c0;
        if ((ldy & 3) == 0 && (reinterpret_cast<uintptr_t>(out) & 7) == 0) {
          *reinterpret_cast<uint2*>(at) = o.u;
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i) at[i] = o.e[i];
        }
      }
    }
  }
}

int compute_units() {
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

template <int MT, int KC, int DEPTH, int WT, int MODE, typename TY>
int launch(void* y, const void* x, const void* wb, int M, int N_out, int w_rows, int K, long ldx, long ldy,
           int blocks, int splits, int pair_offset, hipStream_t stream) {
  const size_t lds = (size_t)NB * MT * 16 * KC * sizeof(bf16_t);
  auto kernel = gemm_rows_kernel<MT, KC, DEPTH, WT, MODE, TY>;
  static bool raised = false;                  // (per instantiation)
  if (!raised) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds) != hipSuccess) {
      (void)hipGetLastError();
      return PTL_ERR_LAUNCH;
    }
    raised = true;
  }
  const int k_per_split = ((K + splits - 1) / splits + 31) / 32 * 32;
  kernel<<<dim3(blocks, splits), (TILES / WT + 1) * 64, lds, stream>>>(
      (TY*)y, (const bf16_t*)x, (const bf16_t*)wb, M, N_out, w_rows, K, ldx, ldy, k_per_split, pair_offset);
  return ptl_launch_status();
}

bool bad_common(int M, int K, long ldx) {
  return M <= 0 || M > 128 || K <= 0 || K % 32 || ldx % 8 || ldx < K;
}

int m_tiles(int M) { return M <= 16 ? 1 : M <= 32 ? 2 : M <= 48 ? 3 : M <= 64 ? 4 : 8; }

// The slices of K that a product should be cut into when the caller can take partial sums:
// doubled while the workgroups are fewer than the compute units and a slice keeps at least 256
// columns. On the current device.
int plain_splits(int N, int K) {
  const int blocks = (N + 63) / 64, cus = compute_units();
  int splits = 1;
  while (blocks * splits < cus && K / (2 * splits) >= 256 && splits < 16) splits *= 2;
  return splits;
}

}  // namespace

extern "C" int ptl_rows_gemm_splits(int M, int N, int K) {
  if (M <= 0 || N <= 0 || K <= 0) return 1;
  return plain_splits(N, K);
}

// y [splits, M, N] = x [M, K] W^T over ``splits`` slices of K (1: the product itself), W given
// as its blocked copy (rows padded to a multiple of 16). out_dtype: bfloat16 (splits = 1 only)
// or float32. 9..128 rows are what it is made for; fewer work too. splits: what
// ptl_rows_gemm_splits says, or 1.
extern "C" int ptl_rows_gemm_bf16(void* y, const void* x, const void* w_blocked, int M, int N, int K,
                                  long ldx, long ldy, int out_dtype, int splits, hipStream_t stream) {
  if (N <= 0 || M == 0) return PTL_OK;
  if (bad_common(M, K, ldx) || ldy < N || splits < 1 || splits > 64 || (splits > 1 && out_dtype != PTL_DTYPE_F32) ||
      (out_dtype != PTL_DTYPE_F32 && out_dtype != PTL_DTYPE_BF16))
    return PTL_ERR_ARG;
  const int blocks = (N + 63) / 64;
  const int w_rows = (N + 15) / 16 * 16;
  // two tiles of W a wave (two waves multiply, every fragment of x read from LDS meets two tiles)
  // where the workgroups are many to a compute unit, as for a head of vocabulary size; one tile
  // a wave (four waves multiply) where there is about one workgroup a compute unit (measured)
  const bool two = (long)blocks * splits >= 4L * compute_units();
#define GO(MT, KC, DEPTH, WT, TY) launch<MT, KC, DEPTH, WT, MODE_PLAIN, TY>(y, x, w_blocked, M, N, w_rows, K, ldx, ldy, \
                                                                           blocks, splits, 0, stream)
#define BY_TYPE(MT, KC, DEPTH, WT) (out_dtype == PTL_DTYPE_F32 ? GO(MT, KC, DEPTH, WT, float) : GO(MT, KC, DEPTH, WT, bf16_t))
#define BY_WT(MT, KC, DEPTH) (two ? BY_TYPE(MT, 128, 4, 2) : BY_TYPE(MT, KC, DEPTH, 1))
  switch (m_tiles(M)) {
    case 1: return BY_WT(1, KC_1, DEPTH_1);
    case 2: return BY_WT(2, KC_2, DEPTH_2);
    case 3: return BY_WT(3, KC_3, DEPTH_3);
    case 4: return BY_WT(4, KC_4, DEPTH_4);
    default: return BY_WT(8, KC_8, DEPTH_8);
  }
#undef BY_WT
#undef BY_TYPE
#undef GO
}

// out [M, I] = silu(x Wg^T) * (x Wu^T) for W = [Wg; Wu] of shape [2 I, K] given as its blocked
// copy; I % 32 == 0.
extern "C" int ptl_rows_gate_up_silu(void* out, const void* x, const void* w_blocked, int M, int I, int K,
                                     long ldx, hipStream_t stream) {
  if (I <= 0 || M == 0) return PTL_OK;
  if (bad_common(M, K, ldx) || I % 32) return PTL_ERR_ARG;
  const int blocks = I / 32;
#define GO(MT, KC, DEPTH) launch<MT, KC, DEPTH, 1, MODE_SILU, bf16_t>(out, x, w_blocked, M, I, 2 * I, K, ldx, I, blocks, 1, I, stream)
  switch (m_tiles(M)) {
    case 1: return GO(1, KC_1, DEPTH_1);
    case 2: return GO(2, KC_2, DEPTH_2);
    case 3: return GO(3, KC_3, DEPTH_3);
    case 4: return GO(4, KC_4, DEPTH_4);
    default: return GO(8, KC_8, DEPTH_8);
  }
#undef GO
}

// y = RMSNorm(round_bf16(sum_s partials[s]) + residual) * w, residual <- the sum (bfloat16), for
// the float32 partial sums [splits, M, N] of ptl_rows_gemm_bf16: one workgroup a row, the row in
// registers (N % 8 == 0, N <= 8192). The product is rounded to bfloat16 first, as a product
// stored in bfloat16 would be; the sum with the residual and the statistics are float32, and
// the norm uses the unrounded sum (lite_llama/kernels/skip_rmsnorm.py:145-152).
template <int CH>
__global__ void __launch_bounds__(256)
sum_add_rmsnorm_kernel(bf16_t* __restrict__ y, const float* __restrict__ partials, int splits,
                       bf16_t* __restrict__ residual, const float* __restrict__ w, int M, int N, float eps) {
  __shared__ float scratch[16];
  const int m = blockIdx.x;
  const int nchunk = N >> 3;
  float v[CH][8];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int ci = threadIdx.x + c * blockDim.x;
    if (ci < nchunk) {
      float p[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      // four slices' loads under way at a time (one after the other they would each cost a trip
      // to L2), added in the order of the slices
      for (int s0 = 0; s0 < splits; s0 += 4) {
        float4 a[4], b[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float* at = partials + ((size_t)min(s0 + j, splits - 1) * M + m) * N + (size_t)ci * 8;
          a[j] = *reinterpret_cast<const float4*>(at);
          b[j] = *reinterpret_cast<const float4*>(at + 4);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if (s0 + j < splits) {
            p[0] += a[j].x; p[1] += a[j].y; p[2] += a[j].z; p[3] += a[j].w;
            p[4] += b[j].x; p[5] += b[j].y; p[6] += b[j].z; p[7] += b[j].w;
          }
        }
      }
      union { uint4 u; bf16_t e[8]; } r;
      r.u = *reinterpret_cast<const uint4*>(residual + (size_t)m * N + (size_t)ci * 8);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float f = round_to<bf16_t>(p[j]) + bf16_to_float(r.e[j]);
        r.e[j] = float_to_bf16(f);
        v[c][j] = f;
        ss += f * f;
      }
      *reinterpret_cast<uint4*>(residual + (size_t)m * N + (size_t)ci * 8) = r.u;
    }
  }
  ss = block_sum(ss, scratch);
  const float rr = 1.0f / sqrtf(ss / (float)N + eps);
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
      *reinterpret_cast<uint4*>(y + (size_t)m * N + (size_t)ci * 8) = o.u;
    }
  }
}

extern "C" int ptl_rows_sum_add_rmsnorm(void* y, const float* partials, int splits, void* residual,
                                        const float* w, int M, int N, float eps, hipStream_t stream) {
  if (M <= 0) return PTL_OK;
  if (N <= 0 || N % 8 || N > 8 * 256 * 4 || splits < 1 || !partials || !residual || !w ||
      ((uintptr_t)y | (uintptr_t)partials | (uintptr_t)residual | (uintptr_t)w) % 16)
    return PTL_ERR_ARG;
  const int nchunk = N / 8;
  int vt = 64;
  while (vt < 256 && vt < nchunk) vt <<= 1;
  const int ch = (nchunk + vt - 1) / vt;
#define GO(C) sum_add_rmsnorm_kernel<C><<<M, vt, 0, stream>>>((bf16_t*)y, partials, splits, (bf16_t*)residual, w, M, N, eps)
  if (ch <= 1) GO(1); else if (ch == 2) GO(2); else if (ch == 3) GO(3); else GO(4);
#undef GO
  return ptl_launch_status();
}

// The float32 partial sums [splits, M, (Hq + 2 Hkv) D] of a q | k | v projection, added up,
// rounded to bfloat16 (as a projection stored in bfloat16 is), q and k rotated by the angles
// position * inv_freq (pairs (j, j + D/2), float32 angles with the accurate sincosf;
// lite_llama/kernels/rope_emb.py:75-103), q written to q_out [M, Hq, D] and k, v into the cache
// pages at ``slots``. One thread a pair of elements.
__global__ void __launch_bounds__(256)
sum_rope_store_kernel(bf16_t* __restrict__ q_out, long ldq, const float* __restrict__ partials, int splits,
                      int M, const int32_t* __restrict__ positions, const float* __restrict__ inv_freq,
                      const int32_t* __restrict__ slots, bf16_t* __restrict__ k_cache,
                      bf16_t* __restrict__ v_cache, int Hq, int Hkv, int D, int page_size) {
  const int m = blockIdx.x, half = D >> 1;
  const int p = blockIdx.y * blockDim.x + threadIdx.x;
  const int heads = Hq + 2 * Hkv;
  if (p >= heads * half) return;
  const int head = p / half, j = p - head * half;
  const size_t width = (size_t)heads * D;
  float x1 = 0.f, x2 = 0.f;
  for (int s0 = 0; s0 < splits; s0 += 4) {       // (four slices' loads under way at a time)
    float a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float* at = partials + ((size_t)min(s0 + i, splits - 1) * M + m) * width + (size_t)head * D + j;
      a[i] = at[0];
      b[i] = at[half];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (s0 + i < splits) { x1 += a[i]; x2 += b[i]; }
  }
  x1 = round_to<bf16_t>(x1);
  x2 = round_to<bf16_t>(x2);
  const bool is_q = head < Hq, is_k = !is_q && head < Hq + Hkv;
  bf16_t* dst = nullptr;
  if (is_q) {
    dst = q_out + (size_t)m * ldq + (size_t)head * D;
  } else {
    const int slot = slots ? slots[m] : -1;
    if (slot >= 0) {
      const int kvh = is_k ? head - Hq : head - Hq - Hkv;
      const int page = slot / page_size, off = slot - page * page_size;
      dst = (is_k ? k_cache : v_cache) + (((size_t)page * Hkv + kvh) * page_size + off) * D;
    }
  }
  if (dst == nullptr) return;
  if ((is_q || is_k) && inv_freq) {
    float sn, cs;
    sincosf((float)positions[m] * inv_freq[j], &sn, &cs);
    const float a = x1 * cs - x2 * sn, b = x2 * cs + x1 * sn;
    x1 = a; x2 = b;
  }
  dst[j] = float_to_bf16(x1);
  dst[j + half] = float_to_bf16(x2);
}

extern "C" int ptl_rows_sum_rope_store(void* q_out, long ldq, const float* partials, int splits, int M,
                                       const int32_t* positions, const float* inv_freq, const int32_t* slots,
                                       void* k_cache, void* v_cache, int Hq, int Hkv, int D, int page_size,
                                       hipStream_t stream) {
  if (M <= 0) return PTL_OK;
  if (Hq <= 0 || Hkv <= 0 || D <= 0 || D % 2 || ldq < (long)Hq * D || page_size <= 0 || splits < 1 ||
      !partials || !positions || (slots && (!k_cache || !v_cache)))
    return PTL_ERR_ARG;
  const int pairs = (Hq + 2 * Hkv) * (D / 2);
  sum_rope_store_kernel<<<dim3(M, (pairs + 255) / 256), 256, 0, stream>>>(
      (bf16_t*)q_out, ldq, partials, splits, M, positions, inv_freq, slots, (bf16_t*)k_cache, (bf16_t*)v_cache,
      Hq, Hkv, D, page_size);
  return ptl_launch_status();
}
