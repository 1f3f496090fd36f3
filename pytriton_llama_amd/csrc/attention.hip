// Attention over the paged cache for a mixed batch: every query token of a
// sequence attends the keys of that sequence that lie in pages, up to and
// including its own position (its own key was written before the launch).
// A prompt portion and a single decoded token are the same case: q_len rows
// at positions ctx_len - q_len .. ctx_len - 1.
//
// Reference: scores q.k * scale, causal mask, online softmax with running max
// and denominator, float32 accumulators (lite_llama/kernels/flashattentionv2.py:
// 10-61,63-162); query head a reads kv head a / (Hq/Hkv) (:108); the decode
// case is lite_llama/kernels/flashdecoding.py:22-131. The mask of a portion
// with a cached prefix is k_pos <= prefix + q_idx
// (lite_llama/kernels/others/context_flashattention_nopad.py:83-92).
//
// Cache layout: [num_pages, Hkv, page_size, D]; key position p of a sequence is
// in page block_table[seq][p / page_size] at offset p % page_size.
// window > 0 limits a query at position p to keys p-window+1 .. p; pages left
// of every window may be gone (table entry < 0) and are never touched.
//
// ptl_attention_generic: vector-FMA kernel, float32 math, storage type T
// (float32 or bfloat16), any page size, any D up to 256.
#include "common.h"
#include "mfma.h"
#include <math.h>

#define BM 16

template <typename T, int BN>
__global__ void __launch_bounds__(256)
attn_generic_kernel(T* __restrict__ out, long out_stride, const T* __restrict__ q, long q_stride,
                    const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                    const int32_t* __restrict__ q_start, const int32_t* __restrict__ ctx_len,
                    const int32_t* __restrict__ block_table, int bt_stride,
                    const int32_t* __restrict__ work_seq, const int32_t* __restrict__ work_qoff,
                    int Hq, int Hkv, int D, int page_size, int window, float scale) {
  extern __shared__ float lds[];
  float* Qs = lds;                   // [BM][D]
  float* Ks = Qs + BM * D;           // [BN][D+1]
  float* Vs = Ks + BN * (D + 1);     // [BN][D]
  float* Ss = Vs + BN * D;           // [BM][BN]

  const int tid = threadIdx.x;
  const int head = blockIdx.y;
  const int seq = work_seq[blockIdx.x];
  const int qoff = work_qoff[blockIdx.x];
  const int qs = q_start[seq];
  const int qlen = q_start[seq + 1] - qs;
  const int ctx = ctx_len[seq];
  const int cached = ctx - qlen;
  const int rows = min(BM, qlen - qoff);
  if (rows <= 0) return;
  const int kvh = head / (Hq / Hkv);
  const int32_t* bt = block_table + (size_t)seq * bt_stride;

  for (int i = tid; i < BM * D; i += 256) {
    const int m = i / D, d = i - m * D;
    Qs[i] = m < rows ? to_float<T>(q[(size_t)(qs + qoff + m) * q_stride + head * D + d]) : 0.f;
  }

  const int tm = tid >> 4, tc = tid & 15;
  const bool row_valid = tm < rows;
  const int qpos = cached + qoff + tm;
  const int first_q = cached + qoff;
  const int k_end = min(ctx, first_q + rows);
  const int k_lo = window > 0 ? max(0, first_q - window + 1) : 0;
  const int k_begin = (k_lo / BN) * BN;
  const int nd = (D + 15) >> 4;

  float m_run = -INFINITY, l_run = 0.f;
  float acc[16];
#pragma unroll
  for (int j = 0; j < 16; ++j) acc[j] = 0.f;

  for (int k0 = k_begin; k0 < k_end; k0 += BN) {
    __syncthreads();
    for (int i = tid; i < BN * D; i += 256) {
      const int n = i / D, d = i - n * D;
      const int kp = k0 + n;
      float kv = 0.f, vv = 0.f;
      if (kp >= k_lo && kp < k_end) {
        const int page = bt[kp / page_size];
        if (page >= 0) {
          const size_t idx = (((size_t)page * Hkv + kvh) * page_size + (kp % page_size)) * D + d;
          kv = to_float<T>(k_cache[idx]);
          vv = to_float<T>(v_cache[idx]);
        }
      }
      Ks[n * (D + 1) + d] = kv;
      Vs[n * D + d] = vv;
    }
    __syncthreads();

    float s[BN / 16];
    float tmax = -INFINITY;
#pragma unroll
    for (int j = 0; j < BN / 16; ++j) {
      const int n = tc + 16 * j;
      const int kp = k0 + n;
      const float* qr = Qs + tm * D;
      const float* kr = Ks + n * (D + 1);
      float dot = 0.f;
      for (int d = 0; d < D; ++d) dot = fmaf(qr[d], kr[d], dot);
      const bool vis = row_valid && kp <= qpos && kp < ctx && (window <= 0 || kp > qpos - window);
      s[j] = vis ? dot * scale : -INFINITY;
      tmax = fmaxf(tmax, s[j]);
    }
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) tmax = fmaxf(tmax, __shfl_xor(tmax, o, 64));
    const float m_new = fmaxf(m_run, tmax);
    const float m_safe = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = expf(m_run - m_safe);
    float psum = 0.f;
#pragma unroll
    for (int j = 0; j < BN / 16; ++j) {
      const float p = expf(s[j] - m_safe);
      psum += p;
      Ss[tm * BN + tc + 16 * j] = p;
    }
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) psum += __shfl_xor(psum, o, 64);
    l_run = l_run * alpha + psum;
    m_run = m_new;
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[j] *= alpha;
    __syncthreads();

    const int n_lim = min(BN, k_end - k0);
    for (int n = 0; n < n_lim; ++n) {
      const float p = Ss[tm * BN + n];
      const float* vr = Vs + n * D + tc;
#pragma unroll
      for (int j = 0; j < 16; ++j)
        if (j < nd && tc + 16 * j < D) acc[j] = fmaf(p, vr[16 * j], acc[j]);
    }
  }

  if (row_valid) {
    const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
    T* o = out + (size_t)(qs + qoff + tm) * out_stride + head * D + tc;
#pragma unroll
    for (int j = 0; j < 16; ++j)
      if (j < nd && tc + 16 * j < D) o[16 * j] = from_float<T>(acc[j] * inv);
  }
}

template <typename T, int BN>
static int launch_generic(void* out, long out_stride, const void* q, long q_stride,
                          const void* k_cache, const void* v_cache, const int32_t* q_start,
                          const int32_t* ctx_len, const int32_t* block_table, int bt_stride,
                          const int32_t* work_seq, const int32_t* work_qoff, int n_work,
                          int Hq, int Hkv, int D, int page_size, int window, float scale,
                          hipStream_t stream) {
  const size_t lds = (size_t)(BM * D + BN * (D + 1) + BN * D + BM * BN) * sizeof(float);
  dim3 grid(n_work, Hq);
  attn_generic_kernel<T, BN><<<grid, 256, lds, stream>>>(
      (T*)out, out_stride, (const T*)q, q_stride, (const T*)k_cache, (const T*)v_cache, q_start,
      ctx_len, block_table, bt_stride, work_seq, work_qoff, Hq, Hkv, D, page_size, window, scale);
  return ptl_launch_status();
}

// work_seq / work_qoff list the 16-row query blocks: block i covers rows
// work_qoff[i] .. work_qoff[i]+15 of sequence work_seq[i].
extern "C" int ptl_attention_generic(void* out, long out_stride, const void* q, long q_stride,
                                     const void* k_cache, const void* v_cache,
                                     const int32_t* q_start, const int32_t* ctx_len,
                                     const int32_t* block_table, int bt_stride,
                                     const int32_t* work_seq, const int32_t* work_qoff, int n_work,
                                     int Hq, int Hkv, int D, int page_size, int window, float scale,
                                     int dtype, hipStream_t stream) {
  if (n_work <= 0) return PTL_OK;
  if (Hq <= 0 || Hkv <= 0 || Hq % Hkv || D <= 0 || D > 256 || page_size <= 0 ||
      Hq > 65535)
    return PTL_ERR_ARG;
#define GO(T, BN) launch_generic<T, BN>(out, out_stride, q, q_stride, k_cache, v_cache, q_start, \
                                        ctx_len, block_table, bt_stride, work_seq, work_qoff,   \
                                        n_work, Hq, Hkv, D, page_size, window, scale, stream)
  if (dtype == PTL_DTYPE_F32) return D <= 128 ? GO(float, 32) : GO(float, 16);
  if (dtype == PTL_DTYPE_BF16) return D <= 128 ? GO(bf16_t, 32) : GO(bf16_t, 16);
#undef GO
  return PTL_ERR_ARG;
}

// ===========================================================================
// ptl_attention_decode: one query token per sequence against its pages, the
// keys split over several workgroups (flash-decoding; the reference's stage 1
// and stage 2 are lite_llama/kernels/flashdecoding.py:22-131 and :171-231:
// every partition emits its accumulator with its running max and denominator,
// the merge weighs them by exp(max_p - max)).
//
// Grid (sequence, kv head x head group, split). A workgroup of four waves
// serves up to GT query heads that share one kv head, so every key and value
// is read once for all of them. A wave reads 64/LPK keys per turn: LPK lanes
// share a key, each lane owns 16 elements of the head dimension of that key
// and of the matching value, for all heads. Every key slot (LPK lanes) keeps
// an online softmax of its own; slots, waves and splits are merged at the end.
// Needs D % 16 == 0. Float32 math throughout.
// ===========================================================================
#define DEC_CHUNK 16

template <typename T> struct Chunk16 { float v[DEC_CHUNK]; };

template <typename T>
__device__ __forceinline__ void load_chunk(const T* __restrict__ p, float* out);

template <>
__device__ __forceinline__ void load_chunk<float>(const float* __restrict__ p, float* out) {
  const float4* p4 = reinterpret_cast<const float4*>(p);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float4 x = p4[i];
    out[4 * i] = x.x; out[4 * i + 1] = x.y; out[4 * i + 2] = x.z; out[4 * i + 3] = x.w;
  }
}

template <>
__device__ __forceinline__ void load_chunk<bf16_t>(const bf16_t* __restrict__ p, float* out) {
  const uint4* p4 = reinterpret_cast<const uint4*>(p);
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const uint4 x = p4[i];
    const uint32_t w[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      out[8 * i + 2 * j] = __uint_as_float(w[j] << 16);
      out[8 * i + 2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
    }
  }
}

template <typename T, int GT, int LPK>
__global__ void __launch_bounds__(256)
attn_decode_kernel(T* __restrict__ out, long out_stride, const T* __restrict__ q, long q_stride,
                   const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                   const int32_t* __restrict__ q_start, const int32_t* __restrict__ ctx_len,
                   const int32_t* __restrict__ block_table, int bt_stride,
                   float* __restrict__ part_acc, float* __restrict__ part_ml,
                   int Hq, int Hkv, int D, int page_size, int window, float scale,
                   int num_splits, int groups_per_kv) {
  constexpr int KPW = 64 / LPK;           // keys a wave reads per turn
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int seq = blockIdx.x;
  const int kvh = blockIdx.y / groups_per_kv;
  const int hg = blockIdx.y - kvh * groups_per_kv;
  const int split = blockIdx.z;
  const int G = Hq / Hkv;
  const int head0 = kvh * G + hg * GT;      // first query head of this workgroup
  const int nheads = min(GT, G - hg * GT);
  const int row = q_start[seq];
  const int ctx = ctx_len[seq];
  const int k_lo = window > 0 ? max(0, ctx - window) : 0;
  const int span = ctx - k_lo;
  const int tile = 4 * KPW;
  const int per_split = ((span + num_splits - 1) / num_splits + tile - 1) / tile * tile;
  const int k_begin = k_lo + split * per_split;
  const int k_end = min(ctx, k_begin + per_split);
  const int32_t* bt = block_table + (size_t)seq * bt_stride;

  const int c = lane % LPK;                 // which 16 elements of the head this lane owns
  const int ks = lane / LPK;                // key slot within the wave
  const bool active = c * DEC_CHUNK < D;

  float qf[GT][DEC_CHUNK];
#pragma unroll
  for (int h = 0; h < GT; ++h) {
    if (h < nheads && active) {
      load_chunk<T>(q + (size_t)row * q_stride + (size_t)(head0 + h) * D + c * DEC_CHUNK, qf[h]);
#pragma unroll
      for (int j = 0; j < DEC_CHUNK; ++j) qf[h][j] *= scale;
    } else {
#pragma unroll
      for (int j = 0; j < DEC_CHUNK; ++j) qf[h][j] = 0.f;
    }
  }
  float m[GT], l[GT], acc[GT][DEC_CHUNK];
#pragma unroll
  for (int h = 0; h < GT; ++h) {
    m[h] = -INFINITY; l[h] = 0.f;
#pragma unroll
    for (int j = 0; j < DEC_CHUNK; ++j) acc[h][j] = 0.f;
  }

  for (int kb = k_begin + wave * KPW; kb < k_end; kb += tile) {
    const int kp = kb + ks;
    const bool valid = kp < k_end;
    float kf[DEC_CHUNK], vf[DEC_CHUNK];
    if (valid && active) {
      const int page = bt[kp / page_size];
      const size_t idx = (((size_t)page * Hkv + kvh) * page_size + (kp % page_size)) * D + c * DEC_CHUNK;
      load_chunk<T>(k_cache + idx, kf);
      load_chunk<T>(v_cache + idx, vf);
    } else {
#pragma unroll
      for (int j = 0; j < DEC_CHUNK; ++j) { kf[j] = 0.f; vf[j] = 0.f; }
    }
#pragma unroll
    for (int h = 0; h < GT; ++h) {
      float s = 0.f;
#pragma unroll
      for (int j = 0; j < DEC_CHUNK; ++j) s = fmaf(qf[h][j], kf[j], s);
#pragma unroll
      for (int o = 1; o < LPK; o <<= 1) s += __shfl_xor(s, o, 64);
      if (valid) {
        if (s > m[h]) {
          const float alpha = expf(m[h] - s);     // exp(-inf) = 0 at the first key
          l[h] *= alpha;
#pragma unroll
          for (int j = 0; j < DEC_CHUNK; ++j) acc[h][j] *= alpha;
          m[h] = s;
        }
        const float p = expf(s - m[h]);
        l[h] += p;
#pragma unroll
        for (int j = 0; j < DEC_CHUNK; ++j) acc[h][j] = fmaf(p, vf[j], acc[h][j]);
      }
    }
  }

  // merge the key slots of the wave
#pragma unroll
  for (int o = LPK; o < 64; o <<= 1) {
#pragma unroll
    for (int h = 0; h < GT; ++h) {
      const float mo = __shfl_xor(m[h], o, 64);
      const float lo = __shfl_xor(l[h], o, 64);
      const float mn = fmaxf(m[h], mo);
      const float ms = mn == -INFINITY ? 0.f : mn;
      const float a = expf(m[h] - ms), b = expf(mo - ms);
      l[h] = l[h] * a + lo * b;
#pragma unroll
      for (int j = 0; j < DEC_CHUNK; ++j)
        acc[h][j] = acc[h][j] * a + __shfl_xor(acc[h][j], o, 64) * b;
      m[h] = mn;
    }
  }

  // merge the four waves through LDS
  extern __shared__ float lds[];
  float* w_acc = lds;                         // [4][GT][D]
  float* w_ml = lds + 4 * GT * D;             // [4][GT][2]
  if (ks == 0 && active) {
#pragma unroll
    for (int h = 0; h < GT; ++h) {
#pragma unroll
      for (int j = 0; j < DEC_CHUNK; ++j) w_acc[(wave * GT + h) * D + c * DEC_CHUNK + j] = acc[h][j];
      if (c == 0) { w_ml[(wave * GT + h) * 2] = m[h]; w_ml[(wave * GT + h) * 2 + 1] = l[h]; }
    }
  }
  __syncthreads();
  for (int i = tid; i < nheads * D; i += 256) {
    const int h = i / D, d = i - h * D;
    float mn = -INFINITY;
#pragma unroll
    for (int w = 0; w < 4; ++w) mn = fmaxf(mn, w_ml[(w * GT + h) * 2]);
    const float ms = mn == -INFINITY ? 0.f : mn;
    float ll = 0.f, a = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float f = expf(w_ml[(w * GT + h) * 2] - ms);
      ll += w_ml[(w * GT + h) * 2 + 1] * f;
      a += w_acc[(w * GT + h) * D + d] * f;
    }
    const int head = head0 + h;
    if (num_splits == 1) {
      out[(size_t)row * out_stride + (size_t)head * D + d] = from_float<T>(ll > 0.f ? a / ll : 0.f);
    } else {
      const size_t pi = ((size_t)seq * Hq + head) * num_splits + split;
      part_acc[pi * D + d] = a;
      if (d == 0) { part_ml[pi * 2] = mn; part_ml[pi * 2 + 1] = ll; }
    }
  }
}

template <typename T>
__global__ void __launch_bounds__(64)
attn_decode_merge_kernel(T* __restrict__ out, long out_stride, const int32_t* __restrict__ q_start,
                         const float* __restrict__ part_acc, const float* __restrict__ part_ml,
                         int Hq, int D, int num_splits) {
  // one wave per (sequence, head): lanes take the splits' (max, denominator) side by side,
  // then the head dimension, with the splits' weights in LDS. The partial results come from
  // other compute units' writes, a long way off: the first 16 splits of the lane's first
  // column are asked for before anything is computed, so that one wait covers them and the
  // (max, denominator) pairs.
  constexpr int AHEAD = 16;
  __shared__ float wgt[1024];
  const int seq = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const size_t base = ((size_t)seq * Hq + head) * num_splits;
  const float* pa0 = part_acc + base * D + lane;
  float first[AHEAD];
#pragma unroll
  for (int s = 0; s < AHEAD; ++s) first[s] = (s < num_splits && lane < D) ? pa0[(size_t)s * D] : 0.f;
  const int row = q_start[seq];
  float mn = -INFINITY;
  for (int s = lane; s < num_splits; s += 64) mn = fmaxf(mn, part_ml[(base + s) * 2]);
  mn = wave_max(mn);
  const float ms = mn == -INFINITY ? 0.f : mn;
  float ll = 0.f;
  for (int s = lane; s < num_splits; s += 64) {
    const float w = expf(part_ml[(base + s) * 2] - ms);
    if (s < 1024) wgt[s] = w;
    ll += part_ml[(base + s) * 2 + 1] * w;
  }
  ll = wave_sum(ll);
  __syncthreads();
  const float inv = ll > 0.f ? 1.0f / ll : 0.f;
  for (int d = lane; d < D; d += 64) {
    float a = 0.f;
    const float* pa = part_acc + base * D + d;
    int s = 0;
    if (d == lane) {
#pragma unroll
      for (; s < AHEAD; ++s)
        if (s < num_splits) a = fmaf(first[s], wgt[s], a);
    }
#pragma unroll 8
    for (; s < num_splits; ++s) a = fmaf(pa[(size_t)s * D], wgt[s], a);
    out[(size_t)row * out_stride + (size_t)head * D + d] = from_float<T>(a * inv);
  }
}

template <typename T, int LPK>
static int launch_decode(void* out, long out_stride, const void* q, long q_stride,
                         const void* k_cache, const void* v_cache, const int32_t* q_start,
                         const int32_t* ctx_len, const int32_t* block_table, int bt_stride,
                         float* part_acc, float* part_ml, int n_seq, int Hq, int Hkv, int D,
                         int page_size, int window, float scale, int num_splits, hipStream_t stream) {
  constexpr int GT = 4;
  const int G = Hq / Hkv;
  const int groups = (G + GT - 1) / GT;
  dim3 grid(n_seq, Hkv * groups, num_splits);
  const size_t lds = (size_t)(4 * GT * D + 4 * GT * 2) * sizeof(float);
  attn_decode_kernel<T, GT, LPK><<<grid, 256, lds, stream>>>(
      (T*)out, out_stride, (const T*)q, q_stride, (const T*)k_cache, (const T*)v_cache, q_start,
      ctx_len, block_table, bt_stride, part_acc, part_ml, Hq, Hkv, D, page_size, window, scale,
      num_splits, groups);
  if (hipGetLastError() != hipSuccess) return PTL_ERR_LAUNCH;
  if (num_splits > 1) {
    dim3 mgrid(n_seq, Hq);
    attn_decode_merge_kernel<T><<<mgrid, 64, 0, stream>>>((T*)out, out_stride, q_start, part_acc,
                                                         part_ml, Hq, D, num_splits);
  }
  return ptl_launch_status();
}

// Sequences 0..n_seq-1 of the tables each bring one query token (row q_start[s]).
// part_acc [n_seq, Hq, num_splits, D] and part_ml [n_seq, Hq, num_splits, 2] are
// float32 workspaces of the caller (unused when num_splits == 1).
extern "C" int ptl_attention_decode(void* out, long out_stride, const void* q, long q_stride,
                                    const void* k_cache, const void* v_cache,
                                    const int32_t* q_start, const int32_t* ctx_len,
                                    const int32_t* block_table, int bt_stride, float* part_acc,
                                    float* part_ml, int n_seq, int Hq, int Hkv, int D, int page_size,
                                    int window, float scale, int num_splits, int dtype,
                                    hipStream_t stream) {
  if (n_seq <= 0) return PTL_OK;
  if (Hq <= 0 || Hkv <= 0 || Hq % Hkv || D <= 0 || D % 16 || D > 256 || page_size <= 0 ||
      num_splits < 1 || num_splits > 1024 || (num_splits > 1 && (!part_acc || !part_ml)))
    return PTL_ERR_ARG;
  const int chunks = D / 16;
  int lpk = 1;
  while (lpk < chunks) lpk <<= 1;
#define GO(T, L) launch_decode<T, L>(out, out_stride, q, q_stride, k_cache, v_cache, q_start,      \
                                     ctx_len, block_table, bt_stride, part_acc, part_ml, n_seq,    \
                                     Hq, Hkv, D, page_size, window, scale, num_splits, stream)
#define BY_LPK(T)                                                                                  \
  switch (lpk) {                                                                                   \
    case 1: return GO(T, 1);                                                                       \
    case 2: return GO(T, 2);                                                                       \
    case 4: return GO(T, 4);                                                                       \
    case 8: return GO(T, 8);                                                                       \
    default: return GO(T, 16);                                                                     \
  }
  if (dtype == PTL_DTYPE_F32) { BY_LPK(float) }
  if (dtype == PTL_DTYPE_BF16) { BY_LPK(bf16_t) }
#undef BY_LPK
#undef GO
  return PTL_ERR_ARG;
}

// ===========================================================================
// ptl_attention_decode_mfma: the bfloat16 decode case on the matrix cores.
//
// Same grid and split scheme as ptl_attention_decode, but a wave takes UNR tiles of
// 16 keys per turn and all query heads of a kv head at once (up to 16 of them are
// the N side of the MFMA tiles, so grouped heads cost nothing extra):
//   S^T[key, head] = K[key, :] . Q[head, :]         v_mfma_f32_16x16x32_bf16,
//                                                   A = 16-byte loads of key rows
//   O^T[d, head]  += V^T[d, key] . P^T[key, head]   v_mfma_f32_16x16x16_bf16,
//                                                   B = P^T as it leaves the
//                                                   first product, A = V^T
// The value tiles go through a region of LDS that belongs to the wave: written as
// they lie in the cache (rows of D, 16-byte stores), read back transposed with
// ds_read_b64_tr_b16 (in a group of 16 lanes, lane s points at
// V[4 g + s/4][16 t + 4 (s%4)] and lane l receives V[4 g + 0..3][16 t + l]).
// Nothing in the loop waits for another wave. The keys and values of the next turn
// are on their way from global memory while this turn is computed, and the page
// numbers of the turn after that are read one turn earlier still.
// The softmax state of a head (running max, denominator) lives in the lanes of
// that head's column; the four waves and the splits are merged at the end as
// in ptl_attention_decode. Needs D % 32 == 0, D <= 128, Hq/Hkv <= 16, a page size
// that is a power of two, pages (of all kv heads) below 4 GiB.
// ===========================================================================
__device__ __forceinline__ void wave_lds_fence() {
  // orders this wave's LDS writes and reads for the compiler; the LDS itself runs a wave's
  // instructions in order
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <int NDT, int UNR>
__global__ void __launch_bounds__(256)
attn_decode_mfma_kernel(bf16_t* __restrict__ out, long out_stride, const bf16_t* __restrict__ q,
                        long q_stride, const bf16_t* __restrict__ k_cache,
                        const bf16_t* __restrict__ v_cache, const int32_t* __restrict__ q_start,
                        const int32_t* __restrict__ ctx_len, const int32_t* __restrict__ block_table,
                        int bt_stride, float* __restrict__ part_acc, float* __restrict__ part_ml,
                        int Hq, int Hkv, int page_size, int page_shift, int window, float scale_log2,
                        int num_splits) {
  constexpr int D = 32 * NDT;
  constexpr int NT = 2 * NDT;             // 16-wide tiles of the head dimension
  constexpr int TILE = 64 * UNR;          // keys per turn of the workgroup
  constexpr int VS = D + 16;              // row stride of a value tile in LDS, in elements
  constexpr int CPR = D / 8;              // 16-byte chunks per row
  constexpr int VCH = 16 * CPR / 64;      // chunks of a tile per lane
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int ln = lane & 15, lg = lane >> 4;
  const int seq = blockIdx.x, kvh = blockIdx.y, split = blockIdx.z;
  const int G = Hq / Hkv;
  const int head0 = kvh * G;
  const int row = q_start[seq];
  const int ctx = ctx_len[seq];
  const int k_lo = window > 0 ? max(0, ctx - window) : 0;
  const int span = ctx - k_lo;
  const int per_split = ((span + num_splits - 1) / num_splits + TILE - 1) / TILE * TILE;
  const int k_begin = k_lo + split * per_split;
  const int k_end = min(ctx, k_begin + per_split);
  const int turns = (k_end - k_begin + TILE - 1) / TILE;
  const int32_t* bt = block_table + (size_t)seq * bt_stride;
  const uint32_t page_bytes = (uint32_t)Hkv * page_size * D * 2;
  const int page_mask = page_size - 1;
  const char* k_head = reinterpret_cast<const char*>(k_cache) + (size_t)kvh * page_size * D * 2;
  const char* v_head = reinterpret_cast<const char*>(v_cache) + (size_t)kvh * page_size * D * 2;

  Frag8 qf[NDT];
#pragma unroll
  for (int kk = 0; kk < NDT; ++kk) {
    qf[kk].u = make_uint4(0, 0, 0, 0);
    if (ln < G)
      qf[kk].u = *reinterpret_cast<const uint4*>(q + (size_t)row * q_stride +
                                                 (size_t)(head0 + ln) * D + 32 * kk + 8 * lg);
  }
  f32x4_t o[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) o[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_part = 0.f;

  extern __shared__ float lds[];
  bf16_t* vl = reinterpret_cast<bf16_t*>(lds) + (size_t)wave * UNR * 16 * VS;
  // this lane's chunks of a value tile: row vrow[i], elements vcol[i] .. +7
  int vrow[VCH], vcol[VCH];
#pragma unroll
  for (int i = 0; i < VCH; ++i) {
    const int c = lane + 64 * i;
    vrow[i] = c / CPR;
    vcol[i] = (c - vrow[i] * CPR) * 8;
  }

  int pk[UNR], pv[UNR][VCH];            // pages of the key row and of the value chunks' rows
  uint4 vg[UNR][VCH];                   // values on their way to LDS
  auto first_key = [&](int turn) { return k_begin + turn * TILE + 16 * UNR * wave; };
  auto load_pages = [&](int turn) {
    const int kc = first_key(turn);
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      const int kp = kc + 16 * u + ln;
      pk[u] = (turn < turns && kp < k_end) ? bt[kp >> page_shift] : -1;
#pragma unroll
      for (int i = 0; i < VCH; ++i) {
        const int vp = kc + 16 * u + vrow[i];
        pv[u][i] = (turn < turns && vp < k_end) ? bt[vp >> page_shift] : -1;
      }
    }
  };
  auto issue_loads = [&](int turn, Frag8 (&kf)[UNR][NDT]) {
    const int kc = first_key(turn);
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      const int kp = kc + 16 * u + ln;
      const char* kr = k_head + (size_t)(uint32_t)max(pk[u], 0) * page_bytes +
                       (uint32_t)(((kp & page_mask) * D + 8 * lg) * 2);
#pragma unroll
      for (int kk = 0; kk < NDT; ++kk)
        kf[u][kk].u = pk[u] >= 0 ? load_once(kr + 64 * kk) : make_uint4(0, 0, 0, 0);
#pragma unroll
      for (int i = 0; i < VCH; ++i) {
        const int vp = kc + 16 * u + vrow[i];
        vg[u][i] = make_uint4(0, 0, 0, 0);              // rows past the end read as zeros
        if (pv[u][i] >= 0)
          vg[u][i] = load_once(v_head + (size_t)(uint32_t)pv[u][i] * page_bytes +
                               (uint32_t)(((vp & page_mask) * D + vcol[i]) * 2));
      }
    }
  };
  // one turn: the values that arrived go to LDS, the next turn's loads are issued, this
  // turn's keys (in kf) and values (in LDS) are used
  auto step = [&](int turn, Frag8 (&kf)[UNR][NDT], Frag8 (&kf_next)[UNR][NDT]) {
    wave_lds_fence();                                   // the last turn's reads are done
#pragma unroll
    for (int u = 0; u < UNR; ++u)
#pragma unroll
      for (int i = 0; i < VCH; ++i)
        *reinterpret_cast<uint4*>(vl + (u * 16 + vrow[i]) * VS + vcol[i]) = vg[u][i];
    wave_lds_fence();
    if (turn + 1 < turns) {
      issue_loads(turn + 1, kf_next);
      load_pages(turn + 2);
    }
    const int kc = first_key(turn);
    if (kc >= k_end) return;                            // wave-uniform: nothing of this turn is ours
    f32x4_t st[UNR];
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      st[u] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < NDT; ++kk)
        st[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[u][kk].v, qf[kk].v, st[u], 0, 0, 0);
    }
    float tmax = -INFINITY;
#pragma unroll
    for (int u = 0; u < UNR; ++u)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float sc = st[u][i] * scale_log2;
        sc = (kc + 16 * u + 4 * lg + i < k_end) ? sc : -INFINITY;
        st[u][i] = sc;
        tmax = fmaxf(tmax, sc);
      }
    tmax = max_with_lane_xor16(tmax);
    tmax = max_with_lane_xor32(tmax);
    if (tmax > m_run) {                                 // (finite: key kc is in range)
      const float alpha = __builtin_amdgcn_exp2f(m_run - tmax);
      m_run = tmax;
      l_part *= alpha;
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        o[t][0] *= alpha; o[t][1] *= alpha; o[t][2] *= alpha; o[t][3] *= alpha;
      }
    }
    s16x4_t pb[UNR];
#pragma unroll
    for (int u = 0; u < UNR; ++u)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = __builtin_amdgcn_exp2f(st[u][i] - m_run);
        l_part += p;
        pb[u][i] = (short)float_to_bf16(p);
      }
    const bf16_t* vp = vl + (4 * lg + (ln >> 2)) * VS + 4 * (ln & 3);
#pragma unroll
    for (int u = 0; u < UNR; ++u)
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const s16x4_t vf = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (__attribute__((address_space(3))) s16x4_t*)(vp + u * 16 * VS + 16 * t));
        o[t] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vf, pb[u], o[t], 0, 0, 0);
      }
  };

  Frag8 kfa[UNR][NDT], kfb[UNR][NDT];
  load_pages(0);
  issue_loads(0, kfa);
  load_pages(1);
  for (int turn = 0; turn < turns; turn += 2) {
    step(turn, kfa, kfb);
    if (turn + 1 < turns) step(turn + 1, kfb, kfa);
  }

  float l = l_part + __shfl_xor(l_part, 16, 64);
  l += __shfl_xor(l, 32, 64);

  // merge the four waves: [wave][head][D] accumulators, [wave][head][2] (max, denominator);
  // the region takes the place of the value tiles, which every wave has left by now
  __syncthreads();
  float* w_acc = lds;
  float* w_ml = lds + 4 * 16 * D;
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) w_acc[((wave * 16 + ln) * D) + 16 * t + 4 * lg + i] = o[t][i];
  if (lg == 0) { w_ml[(wave * 16 + ln) * 2] = m_run; w_ml[(wave * 16 + ln) * 2 + 1] = l; }
  __syncthreads();
  for (int i = tid; i < G * D; i += 256) {
    const int h = i / D, d = i - h * D;
    float mn = -INFINITY;
#pragma unroll
    for (int w = 0; w < 4; ++w) mn = fmaxf(mn, w_ml[(w * 16 + h) * 2]);
    const float ms = mn == -INFINITY ? 0.f : mn;
    float ll = 0.f, a = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float f = __builtin_amdgcn_exp2f(w_ml[(w * 16 + h) * 2] - ms);
      ll += w_ml[(w * 16 + h) * 2 + 1] * f;
      a += w_acc[(w * 16 + h) * D + d] * f;
    }
    const int head = head0 + h;
    if (num_splits == 1) {
      out[(size_t)row * out_stride + (size_t)head * D + d] = float_to_bf16(ll > 0.f ? a / ll : 0.f);
    } else {
      const size_t pi = ((size_t)seq * Hq + head) * num_splits + split;
      part_acc[pi * D + d] = a;
      // the merge kernel works with natural exponents
      if (d == 0) { part_ml[pi * 2] = mn * 0.6931471805599453f; part_ml[pi * 2 + 1] = ll; }
    }
  }
}

template <int NDT, int UNR>
static int launch_decode_mfma(void* out, long out_stride, const void* q, long q_stride,
                              const void* k_cache, const void* v_cache, const int32_t* q_start,
                              const int32_t* ctx_len, const int32_t* block_table, int bt_stride,
                              float* part_acc, float* part_ml, int n_seq, int Hq, int Hkv,
                              int page_size, int window, float scale, int num_splits,
                              hipStream_t stream) {
  constexpr int D = 32 * NDT;
  dim3 grid(n_seq, Hkv, num_splits);
  int page_shift = 0;
  while ((1 << page_shift) < page_size) ++page_shift;
  const size_t lds_merge = (size_t)(4 * 16 * D + 4 * 16 * 2) * sizeof(float);
  const size_t lds_values = (size_t)4 * UNR * 16 * (D + 16) * sizeof(bf16_t);
  const size_t lds = lds_merge > lds_values ? lds_merge : lds_values;
  attn_decode_mfma_kernel<NDT, UNR><<<grid, 256, lds, stream>>>(
      (bf16_t*)out, out_stride, (const bf16_t*)q, q_stride, (const bf16_t*)k_cache,
      (const bf16_t*)v_cache, q_start, ctx_len, block_table, bt_stride, part_acc, part_ml, Hq, Hkv,
      page_size, page_shift, window, scale * 1.4426950408889634f, num_splits);
  if (hipGetLastError() != hipSuccess) return PTL_ERR_LAUNCH;
  if (num_splits > 1) {
    dim3 mgrid(n_seq, Hq);
    attn_decode_merge_kernel<bf16_t><<<mgrid, 64, 0, stream>>>((bf16_t*)out, out_stride, q_start,
                                                              part_acc, part_ml, Hq, D, num_splits);
  }
  return ptl_launch_status();
}

// unroll: 16-key tiles a wave takes per turn, 1 or 2 (0: the kernel's choice).
extern "C" int ptl_attention_decode_mfma(void* out, long out_stride, const void* q, long q_stride,
                                         const void* k_cache, const void* v_cache,
                                         const int32_t* q_start, const int32_t* ctx_len,
                                         const int32_t* block_table, int bt_stride, float* part_acc,
                                         float* part_ml, int n_seq, int Hq, int Hkv, int D,
                                         int page_size, int window, float scale, int num_splits,
                                         int unroll, hipStream_t stream) {
  if (n_seq <= 0) return PTL_OK;
  if (Hq <= 0 || Hkv <= 0 || Hq % Hkv || Hq / Hkv > 16 || D <= 0 || D % 32 || D > 128 ||
      page_size <= 0 || (page_size & (page_size - 1)) ||
      (long)Hkv * page_size * D * 2 >= (1L << 32) || q_stride % 8 || num_splits < 1 ||
      num_splits > 1024 || (num_splits > 1 && (!part_acc || !part_ml)) || unroll < 0 || unroll > 2)
    return PTL_ERR_ARG;
  if (unroll == 0) unroll = 2;
#define GO(N, U) launch_decode_mfma<N, U>(out, out_stride, q, q_stride, k_cache, v_cache, q_start,    \
                                          ctx_len, block_table, bt_stride, part_acc, part_ml, n_seq, \
                                          Hq, Hkv, page_size, window, scale, num_splits, stream)
  if (unroll == 1) {
    switch (D / 32) {
      case 1: return GO(1, 1);
      case 2: return GO(2, 1);
      case 3: return GO(3, 1);
      default: return GO(4, 1);
    }
  }
  switch (D / 32) {
    case 1: return GO(1, 2);
    case 2: return GO(2, 2);
    case 3: return GO(3, 2);
    default: return GO(4, 2);
  }
#undef GO
}
