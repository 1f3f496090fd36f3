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

// cs: [2 * (D/2)] floats of dynamic LDS: cosines, then sines, of this token's angles, computed
// once for all heads (sincosf of a large angle is some hundred instructions).
// VEC: elements a thread moves at once (8: 16-byte accesses for bfloat16, when D/2 and all the
// row strides are multiples of 8 and the pointers are aligned; 1: any even D).
template <typename T, int VEC>
__global__ void rope_store_kernel(T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
                                  long row_stride, const int32_t* __restrict__ positions,
                                  const float* __restrict__ inv_freq,
                                  const int32_t* __restrict__ slots,
                                  T* __restrict__ k_cache, T* __restrict__ v_cache,
                                  int Hq, int Hkv, int D, int page_size, int k_in_place) {
  extern __shared__ float cs[];
  const int t = blockIdx.x;
  const int half = D >> 1;
  const float pos = (float)positions[t];
  float* cosv = cs;
  float* sinv = cs + half;
  for (int j = threadIdx.x; j < half; j += blockDim.x) {
    float s = 0.f, c = 1.f;
    if (inv_freq) sincosf(pos * inv_freq[j], &s, &c);
    cosv[j] = c;
    sinv[j] = s;
  }
  __syncthreads();
  T* qrow = q + (size_t)t * row_stride;
  const T* krow = k + (size_t)t * row_stride;
  const T* vrow = v + (size_t)t * row_stride;
  const int64_t slot = slots ? slots[t] : -1;
  const int64_t page = slot >= 0 ? slot / page_size : 0;
  const int off = slot >= 0 ? (int)(slot - page * page_size) : 0;
  const int per_head = half / VEC;           // groups of VEC pairs in a head

  struct __attribute__((aligned(sizeof(T) * VEC))) Vec { T e[VEC]; };
  auto load = [](const T* p) { return *reinterpret_cast<const Vec*>(p); };
  auto store = [](T* p, const Vec& x) { *reinterpret_cast<Vec*>(p) = x; };
  auto rotate = [&](Vec& a, Vec& b, int j) {
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const float x1 = to_float<T>(a.e[i]), x2 = to_float<T>(b.e[i]);
      const float c = cosv[j + i], s = sinv[j + i];
      a.e[i] = from_float<T>(x1 * c - x2 * s);
      b.e[i] = from_float<T>(x2 * c + x1 * s);
    }
  };

  // q heads
  if (inv_freq) {
    for (int i = threadIdx.x; i < Hq * per_head; i += blockDim.x) {
      const int h = i / per_head, j = (i - h * per_head) * VEC;
      Vec a = load(qrow + h * D + j), b = load(qrow + h * D + j + half);
      rotate(a, b, j);
      store(qrow + h * D + j, a);
      store(qrow + h * D + j + half, b);
    }
  }
  // k heads: rotate, then store; v heads: store
  for (int i = threadIdx.x; i < Hkv * per_head; i += blockDim.x) {
    const int h = i / per_head, j = (i - h * per_head) * VEC;
    Vec a = load(krow + h * D + j), b = load(krow + h * D + j + half);
    if (inv_freq) rotate(a, b, j);
    if (k_in_place) {
      T* kw = const_cast<T*>(krow);
      store(kw + h * D + j, a);
      store(kw + h * D + j + half, b);
    }
    if (slot >= 0) {
      const size_t dst = (((size_t)page * Hkv + h) * page_size + off) * D;
      store(k_cache + dst + j, a);
      store(k_cache + dst + j + half, b);
      store(v_cache + dst + j, load(vrow + h * D + j));
      store(v_cache + dst + j + half, load(vrow + h * D + j + half));
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
  const size_t lds = (size_t)D * sizeof(float);
  const bool vec = dtype == PTL_DTYPE_BF16 && (D / 2) % 8 == 0 && row_stride % 8 == 0 &&
                   ((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)k_cache |
                    (uintptr_t)v_cache) % 16 == 0;
  const int work = Hq * (D / 2) / (vec ? 8 : 1);
  int threads = 64;
  while (threads < 256 && threads < work) threads <<= 1;
  if (dtype == PTL_DTYPE_F32)
    rope_store_kernel<float, 1><<<T_, threads, lds, stream>>>(
        (float*)q, (const float*)k, (const float*)v, row_stride, positions, inv_freq, slots,
        (float*)k_cache, (float*)v_cache, Hq, Hkv, D, page_size, k_in_place);
  else if (dtype == PTL_DTYPE_BF16 && vec)
    rope_store_kernel<bf16_t, 8><<<T_, threads, lds, stream>>>(
        (bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v, row_stride, positions, inv_freq, slots,
        (bf16_t*)k_cache, (bf16_t*)v_cache, Hq, Hkv, D, page_size, k_in_place);
  else if (dtype == PTL_DTYPE_BF16)
    rope_store_kernel<bf16_t, 1><<<T_, threads, lds, stream>>>(
        (bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v, row_stride, positions, inv_freq, slots,
        (bf16_t*)k_cache, (bf16_t*)v_cache, Hq, Hkv, D, page_size, k_in_place);
  else
    return PTL_ERR_ARG;
  return ptl_launch_status();
}
