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

// ptl_stage_step: the integer tables of a step that replays a graph, from the host's pinned
// buffer into the static device buffer the graph reads: dst[i] = src[i] for i < n, except
// that dst[tok_at + j] = tokens[j] for j < n_tok when ``tokens`` (on the device) is given:
// the token ids of a step that is launched before the host knows them. ``src`` is pinned host
// memory, read by the kernel over the bus; one short kernel takes the place of two copies,
// each of which costs a step about 4 us. (The reference copies its decode inputs into the
// graph's static tensors one by one, lite_llama/executor/cuda_graph.py:107-122.)
__global__ void __launch_bounds__(256)
stage_step_kernel(int32_t* __restrict__ dst, const int32_t* __restrict__ src, int n,
                  const int32_t* __restrict__ tokens, int tok_at, int n_tok) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const int j = i - tok_at;
  dst[i] = (tokens != nullptr && j >= 0 && j < n_tok) ? tokens[j] : src[i];
}

extern "C" int ptl_stage_step(int32_t* dst, const int32_t* src, int n, const int32_t* tokens,
                              int tok_at, int n_tok, hipStream_t stream) {
  if (n <= 0) return PTL_OK;
  if (!dst || !src || (tokens && (tok_at < 0 || n_tok < 0 || tok_at + n_tok > n))) return PTL_ERR_ARG;
  stage_step_kernel<<<(n + 255) / 256, 256, 0, stream>>>(dst, src, n, tokens, tok_at, n_tok);
  return ptl_launch_status();
}
