// Rotary position encoding of q and k and the write of k, v into cache pages,
// one workgroup per token.
// Reference: lite_llama/models/RotaryEmbedding.py:200-220 (angle = pos * inv_freq
// in float32, both halves of a head share the angles) and
// lite_llama/kernels/rope_emb.py:75-103 (pairs (j, j + D/2):
// o1 = x1*cos - x2*sin, o2 = x2*cos + x1*sin); the cache write is
// lite_llama/kernels/update_kv_buffer.py:7-28. Here the rotation is done in
// float32 and rounded once.
//
// q, k, v are views of one row-major buffer: element (t, head, d) is at
// ptr[t*row_stride + head*D + d]. q is rotated in place. k (rotated) and v go
// to the caches laid out [num_pages, Hkv, page_size, D] at slot[t] =
// page*page_size + offset; slot < 0 skips the write. inv_freq == nullptr means
// no rotation (another position scheme was applied already, or none).
#include "common.h"

template <typename T>
__global__ void rope_store_kernel(T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
                                  long row_stride, const int32_t* __restrict__ positions,
                                  const float* __restrict__ inv_freq,
                                  const int32_t* __restrict__ slots,
                                  T* __restrict__ k_cache, T* __restrict__ v_cache,
                                  int Hq, int Hkv, int D, int page_size, int k_in_place) {
  const int t = blockIdx.x;
  const int half = D >> 1;
  const float pos = (float)positions[t];
  T* qrow = q + (size_t)t * row_stride;
  const T* krow = k + (size_t)t * row_stride;
  const T* vrow = v + (size_t)t * row_stride;
  const int64_t slot = slots ? slots[t] : -1;
  const int64_t page = slot >= 0 ? slot / page_size : 0;
  const int off = slot >= 0 ? (int)(slot - page * page_size) : 0;

  // q heads
  for (int i = threadIdx.x; i < Hq * half; i += blockDim.x) {
    const int h = i / half, j = i - h * half;
    if (inv_freq) {
      float s, c;
      sincosf(pos * inv_freq[j], &s, &c);
      const float x1 = to_float<T>(qrow[h * D + j]);
      const float x2 = to_float<T>(qrow[h * D + j + half]);
      qrow[h * D + j] = from_float<T>(x1 * c - x2 * s);
      qrow[h * D + j + half] = from_float<T>(x2 * c + x1 * s);
    }
  }
  // k heads: rotate, then store; v heads: store
  for (int i = threadIdx.x; i < Hkv * half; i += blockDim.x) {
    const int h = i / half, j = i - h * half;
    float k1 = to_float<T>(krow[h * D + j]);
    float k2 = to_float<T>(krow[h * D + j + half]);
    if (inv_freq) {
      float s, c;
      sincosf(pos * inv_freq[j], &s, &c);
      const float r1 = k1 * c - k2 * s;
      const float r2 = k2 * c + k1 * s;
      k1 = r1; k2 = r2;
    }
    if (k_in_place) {
      T* kw = const_cast<T*>(krow);
      kw[h * D + j] = from_float<T>(k1);
      kw[h * D + j + half] = from_float<T>(k2);
    }
    if (slot >= 0) {
      const size_t dst = (((size_t)page * Hkv + h) * page_size + off) * D;
      k_cache[dst + j] = from_float<T>(k1);
      k_cache[dst + j + half] = from_float<T>(k2);
      v_cache[dst + j] = vrow[h * D + j];
      v_cache[dst + j + half] = vrow[h * D + j + half];
    }
  }
}

extern "C" int ptl_rope_store(void* q, void* k, const void* v, long row_stride,
                              const int32_t* positions, const float* inv_freq,
                              const int32_t* slots, void* k_cache, void* v_cache,
                              int T_, int Hq, int Hkv, int D, int page_size, int k_in_place,
                              int dtype, hipStream_t stream) {
  if (T_ <= 0) return PTL_OK;
  if (Hq <= 0 || Hkv <= 0 || D <= 0 || (D & 1) || page_size <= 0) return PTL_ERR_ARG;
  if (slots && (!k_cache || !v_cache)) return PTL_ERR_ARG;
  const int work = Hq * (D / 2);
  int threads = 64;
  while (threads < 256 && threads < work) threads <<= 1;
  if (dtype == PTL_DTYPE_F32)
    rope_store_kernel<float><<<T_, threads, 0, stream>>>(
        (float*)q, (const float*)k, (const float*)v, row_stride, positions, inv_freq, slots,
        (float*)k_cache, (float*)v_cache, Hq, Hkv, D, page_size, k_in_place);
  else if (dtype == PTL_DTYPE_BF16)
    rope_store_kernel<bf16_t><<<T_, threads, 0, stream>>>(
        (bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v, row_stride, positions, inv_freq, slots,
        (bf16_t*)k_cache, (bf16_t*)v_cache, Hq, Hkv, D, page_size, k_in_place);
  else
    return PTL_ERR_ARG;
  return ptl_launch_status();
}
