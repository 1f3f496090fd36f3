// Sampling from float32 logits [R, V], one workgroup per row.
//
// ptl_argmax: greedy choice, ties to the lowest id (the reference's greedy
// branch is torch.argmax, lite_llama/generate_stream.py:150).
//
// ptl_sample_top_p: softmax(logits / temperature) (the reference's three-pass
// split softmax, lite_llama/kernels/softmax_split.py:7-77) followed by nucleus
// sampling with the rule of lite_llama/generate.py:30-43: in descending order of
// probability a token is kept while the mass before it is <= top_p, the kept
// ones are renormalised and one is drawn. The draw uses a uniform number
// u[r] in [0,1) given by the caller (seeded per request and step on the host),
// so a result does not depend on what else is in the batch.
//
// Instead of a sort the kernel finds the smallest kept probability by bisection
// over float bit patterns: mass_above(t) = sum of p > t never grows with t, and
// a token of probability p is kept iff mass_above(p) <= top_p. Tokens of equal
// probability are kept or dropped together; a sort would split such a tie at
// the edge of the nucleus by index.
#include "common.h"
#include <math.h>

// Two passes so that a row of vocabulary size is read by many workgroups: every
// chunk leaves its best (value, index), then one wave per row picks among them.
#define ARGMAX_CHUNK 4096

__device__ __forceinline__ void argmax_pick(float& best, int& bi, float v, int i) {
  if (v > best || (v == best && i < bi)) { best = v; bi = i; }
}

__global__ void __launch_bounds__(256)
argmax_partial_kernel(float* __restrict__ pv, int32_t* __restrict__ pi,
                      const float* __restrict__ logits, int V, long stride, int chunks) {
  __shared__ float sv[4];
  __shared__ int si[4];
  const float* row = logits + (size_t)blockIdx.y * stride;
  const int lo = blockIdx.x * ARGMAX_CHUNK, hi = min(V, lo + ARGMAX_CHUNK);
  float best = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = lo + threadIdx.x; i < hi; i += 256) {
    float v = row[i];
    if (v != v) v = -INFINITY;
    argmax_pick(best, bi, v, i);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) argmax_pick(best, bi, __shfl_xor(best, o, 64), __shfl_xor(bi, o, 64));
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (lane == 0) { sv[wave] = best; si[wave] = bi; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int i = 1; i < 4; ++i) argmax_pick(best, bi, sv[i], si[i]);
    pv[(size_t)blockIdx.y * chunks + blockIdx.x] = best;
    pi[(size_t)blockIdx.y * chunks + blockIdx.x] = bi;
  }
}

__global__ void __launch_bounds__(64)
argmax_final_kernel(int32_t* __restrict__ out, const float* __restrict__ pv,
                    const int32_t* __restrict__ pi, int chunks) {
  float best = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = threadIdx.x; i < chunks; i += 64)
    argmax_pick(best, bi, pv[(size_t)blockIdx.x * chunks + i], pi[(size_t)blockIdx.x * chunks + i]);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) argmax_pick(best, bi, __shfl_xor(best, o, 64), __shfl_xor(bi, o, 64));
  if (threadIdx.x == 0) out[blockIdx.x] = bi == 0x7fffffff ? 0 : bi;
}

// workspace: float [R, chunks] and int32 [R, chunks], chunks = ceil(V / 4096)
extern "C" int ptl_argmax(int32_t* out, const float* logits, int R, int V, long stride,
                          float* ws_val, int32_t* ws_idx, hipStream_t stream) {
  if (R <= 0) return PTL_OK;
  if (V <= 0 || stride < V || !ws_val || !ws_idx || R > 65535) return PTL_ERR_ARG;
  const int chunks = (V + ARGMAX_CHUNK - 1) / ARGMAX_CHUNK;
  dim3 grid(chunks, R);
  argmax_partial_kernel<<<grid, 256, 0, stream>>>(ws_val, ws_idx, logits, V, stride, chunks);
  if (hipGetLastError() != hipSuccess) return PTL_ERR_LAUNCH;
  argmax_final_kernel<<<R, 64, 0, stream>>>(out, ws_val, ws_idx, chunks);
  return ptl_launch_status();
}

// probs_out (optional, [R, V]) receives the renormalised nucleus distribution.
__global__ void __launch_bounds__(1024)
sample_top_p_kernel(int32_t* __restrict__ out, float* __restrict__ probs_out,
                    const float* __restrict__ logits, int V, long stride,
                    const float* __restrict__ temperature, const float* __restrict__ top_p,
                    const float* __restrict__ uniform) {
  __shared__ float scratch[16];
  __shared__ float chunk[1024];
  const int r = blockIdx.x;
  const float* row = logits + (size_t)r * stride;
  const float inv_t = 1.0f / temperature[r];
  const float tp = top_p[r];

  float mx = -INFINITY;
  for (int i = threadIdx.x; i < V; i += blockDim.x) mx = fmaxf(mx, row[i] * inv_t);
  mx = block_max(mx, scratch);
  float z = 0.f;
  for (int i = threadIdx.x; i < V; i += blockDim.x) z += expf(row[i] * inv_t - mx);
  z = block_sum(z, scratch);
  const float inv_z = 1.0f / z;

  // kept tokens: p > thr. lo keeps mass_above(lo) > top_p, hi keeps
  // mass_above(hi) <= top_p; when they are neighbouring floats no probability
  // lies between them and {p > lo} is exactly the nucleus.
  float thr = -1.0f;
  if (tp < 1.0f) {
    uint32_t lo = 0u, hi = __float_as_uint(1.0f);
    while (hi - lo > 1u) {
      const uint32_t mid = lo + ((hi - lo) >> 1);
      const float t = __uint_as_float(mid);
      float mass = 0.f;
      for (int i = threadIdx.x; i < V; i += blockDim.x) {
        const float p = expf(row[i] * inv_t - mx) * inv_z;
        if (p > t) mass += p;
      }
      mass = block_sum(mass, scratch);
      if (mass <= tp) hi = mid; else lo = mid;
    }
    thr = __uint_as_float(lo);
    // the most likely token is always kept (nothing lies before it)
    const float pmax = expf(0.f) * inv_z;
    if (thr >= pmax) thr = __uint_as_float(__float_as_uint(pmax) - 1u);
  }

  // inverse-CDF draw in vocabulary order over contiguous chunks
  const int per = (V + blockDim.x - 1) / blockDim.x;
  const int b = threadIdx.x * per, e = min(V, b + per);
  float mine = 0.f;
  for (int i = b; i < e; ++i) {
    const float p = expf(row[i] * inv_t - mx) * inv_z;
    if (p > thr) mine += p;
  }
  chunk[threadIdx.x] = mine;
  const float kept = block_sum(mine, scratch);  // has the barriers that publish chunk[]
  if (probs_out) {
    const float inv_kept = 1.0f / kept;
    float* po = probs_out + (size_t)r * V;
    for (int i = threadIdx.x; i < V; i += blockDim.x) {
      const float p = expf(row[i] * inv_t - mx) * inv_z;
      po[i] = p > thr ? p * inv_kept : 0.f;
    }
  }
  if (threadIdx.x == 0) {
    const float target = uniform[r] * kept;
    float run = 0.f;
    int c = -1, last_nonempty = 0;
    for (int i = 0; i < (int)blockDim.x; ++i) {
      if (chunk[i] > 0.f) {
        last_nonempty = i;
        if (run + chunk[i] > target) { c = i; break; }
      }
      run += chunk[i];
    }
    const bool past_end = c < 0;  // rounding pushed the target past the total
    if (past_end) c = last_nonempty;
    const int cb = c * per, ce = min(V, cb + per);
    int choice = -1, last_kept = -1;
    float acc = run;
    for (int i = cb; i < ce; ++i) {
      const float p = expf(row[i] * inv_t - mx) * inv_z;
      if (p > thr) {
        last_kept = i;
        acc += p;
        if (!past_end && acc > target) { choice = i; break; }
      }
    }
    if (choice < 0) choice = last_kept;
    out[r] = choice < 0 ? 0 : choice;
  }
}

extern "C" int ptl_sample_top_p(int32_t* out, float* probs_out, const float* logits, int R, int V,
                                long stride, const float* temperature, const float* top_p,
                                const float* uniform, hipStream_t stream) {
  if (R <= 0) return PTL_OK;
  if (V <= 0 || stride < V) return PTL_ERR_ARG;
  sample_top_p_kernel<<<R, 1024, 0, stream>>>(out, probs_out, logits, V, stride, temperature, top_p,
                                              uniform);
  return ptl_launch_status();
}
