// Token embedding lookup: out[t, :] = table[ids[t], :]
// (reference: nn.Embedding in lite_llama/models/llama.py:179,201).
#include "common.h"

template <typename T>
__global__ void embedding_kernel(T* __restrict__ out, const T* __restrict__ table,
                                 const int32_t* __restrict__ ids, int H, int V) {
  const int t = blockIdx.x;
  int id = ids[t];
  // ids are checked on the host; a bad id must still not read out of bounds
  if (id < 0 || id >= V) id = 0;
  const T* src = table + (size_t)id * H;
  T* dst = out + (size_t)t * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) dst[i] = src[i];
}

extern "C" int ptl_embedding(void* out, const void* table, const int32_t* ids,
                             int T_, int H, int V, int dtype, hipStream_t stream) {
  if (T_ <= 0) return PTL_OK;
  if (H <= 0 || V <= 0) return PTL_ERR_ARG;
  const int threads = H >= 1024 ? 256 : (H >= 256 ? 128 : 64);
  if (dtype == PTL_DTYPE_F32)
    embedding_kernel<float><<<T_, threads, 0, stream>>>((float*)out, (const float*)table, ids, H, V);
  else if (dtype == PTL_DTYPE_BF16)
    embedding_kernel<bf16_t><<<T_, threads, 0, stream>>>((bf16_t*)out, (const bf16_t*)table, ids, H, V);
  else
    return PTL_ERR_ARG;
  return ptl_launch_status();
}
