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
