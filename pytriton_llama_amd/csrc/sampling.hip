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
//
// How the nucleus is found without a sort. With e = exp(logit/T - max) (the unnormalised
// probability, kept in the work buffer), a token is kept iff the mass of the tokens with
// larger e is <= top_p * sum(e).
// (1) row max; (2) e and its sum; (3) three rounds of a 16-way split of the distance from
// the max, d = -ln e: round one splits [0, 32) into 16 buckets, finds the bucket in which
// the cumulative mass (most likely tokens first) crosses top_p, and the next rounds split
// that bucket again, down to a width of 1/128. Every thread adds into a column of its own
// in LDS (no atomics: LDS float atomics cost about a hundred cycles a wave here); (4) the
// tokens of the last crossing bucket (a few dozen for ordinary logits) are gathered and the
// exact cut among them is found by one wave bisecting over float bit patterns, ending with
// two neighbouring floats so that no e lies between them; (5) the waves sum their kept mass
// over contiguous ranges, a scan locates the wave whose range holds u * kept, and that wave
// walks its range with a running prefix. If the last bucket holds more tokens than fit (many
// equal logits), the bisection runs over the whole row: slower, same result.
#define SMP_THREADS 1024
#define SMP_FAN 16               // buckets per round
#define SMP_ROUNDS 3
#define SMP_SPAN 32.0f           // distance from the max that round one covers
#define SMP_LIST 4096

// exclusive prefix sum over the block; tmp holds 17 floats. Returns the prefix, total in *total.
__device__ __forceinline__ float block_exclusive_scan(float v, float* tmp, float* total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  float inc = v;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const float n = __shfl_up(inc, o, 64);
    if (lane >= o) inc += n;
  }
  __syncthreads();
  if (lane == 63) tmp[wave] = inc;
  __syncthreads();
  if (threadIdx.x == 0) {
    float run = 0.f;
    for (int i = 0; i < nw; ++i) { const float t = tmp[i]; tmp[i] = run; run += t; }
    tmp[16] = run;
  }
  __syncthreads();
  *total = tmp[16];
  return tmp[wave] + inc - v;
}

// Every pass over a row: four consecutive values a thread and step (one 16-byte load) when the
// row is 16-byte aligned, then the few values that are left; f(i, value).
template <typename F>
__device__ __forceinline__ void for_row(const float* __restrict__ p, int V, bool vec, F f) {
  if (vec) {
    const int n4 = V >> 2;
    const float4* p4 = reinterpret_cast<const float4*>(p);
    for (int i = threadIdx.x; i < n4; i += blockDim.x) {
      const float4 v = p4[i];
      f(4 * i, v.x); f(4 * i + 1, v.y); f(4 * i + 2, v.z); f(4 * i + 3, v.w);
    }
    for (int i = 4 * n4 + threadIdx.x; i < V; i += blockDim.x) f(i, p[i]);
  } else {
    for (int i = threadIdx.x; i < V; i += blockDim.x) f(i, p[i]);
  }
}

// work: float [R, V] scratch of the caller; it receives exp(logit/T - max) in the second
// pass, which the later passes read back instead of computing it again, and in the end (if
// want_probs) the renormalised nucleus distribution.
__global__ void __launch_bounds__(SMP_THREADS)
sample_top_p_kernel(int32_t* __restrict__ out, float* __restrict__ work, int want_probs,
                    const float* __restrict__ logits, int V, long stride,
                    const float* __restrict__ temperature, const float* __restrict__ top_p,
                    const float* __restrict__ uniform) {
  __shared__ float scratch[17];
  __shared__ float cols[SMP_FAN * SMP_THREADS];      // a column of bucket sums per thread
  __shared__ float part[SMP_FAN * 16];
  __shared__ float bucket[SMP_FAN];
  __shared__ float list[SMP_LIST];
  __shared__ int list_n;
  __shared__ int cross_bin;
  __shared__ float mass_before;
  __shared__ float thr_s;
  __shared__ int last_kept;
  const int tid = threadIdx.x;
  const int r = blockIdx.x;
  const float* row = logits + (size_t)r * stride;
  float* ex = work + (size_t)r * V;          // unnormalised probabilities e_i = exp(x_i/T - max)
  const float inv_t = 1.0f / temperature[r];
  const float c = inv_t * 1.4426950408889634f;

  const bool vec_in = (((uintptr_t)row) & 15) == 0, vec_ex = (((uintptr_t)ex) & 15) == 0;
  float mx = -INFINITY;
  for_row(row, V, vec_in, [&](int, float x) { mx = fmaxf(mx, x); });
  mx = block_max(mx, scratch);
  const float mc = mx * c;
  float z = 0.f;
  if (vec_in && vec_ex) {
    const int n4 = V >> 2;
    for (int i = tid; i < n4; i += SMP_THREADS) {
      const float4 x = reinterpret_cast<const float4*>(row)[i];
      float4 e;
      e.x = __builtin_amdgcn_exp2f(fmaf(x.x, c, -mc));
      e.y = __builtin_amdgcn_exp2f(fmaf(x.y, c, -mc));
      e.z = __builtin_amdgcn_exp2f(fmaf(x.z, c, -mc));
      e.w = __builtin_amdgcn_exp2f(fmaf(x.w, c, -mc));
      reinterpret_cast<float4*>(ex)[i] = e;
      z += (e.x + e.y) + (e.z + e.w);
    }
    for (int i = 4 * n4 + tid; i < V; i += SMP_THREADS) {
      const float e = __builtin_amdgcn_exp2f(fmaf(row[i], c, -mc));
      ex[i] = e;
      z += e;
    }
  } else {
    for (int i = tid; i < V; i += SMP_THREADS) {
      const float e = __builtin_amdgcn_exp2f(fmaf(row[i], c, -mc));
      ex[i] = e;
      z += e;
    }
  }
  z = block_sum(z, scratch);                 // (its barriers also publish ex[] to the block)
  const float tp = top_p[r] * z;             // all masses below are in units of e
  float thr = -1.0f;                         // kept: e > thr
  if (top_p[r] < 1.0f) {
    // Round q splits [lo[q], lo[q] + SMP_FAN / inv_w[q]) of d = -ln e into SMP_FAN buckets and
    // picks bucket pick[q]. A token belongs to a later round (and to the final list) iff the
    // same arithmetic put it into the picked bucket of every earlier round, so that no token
    // near a bucket's edge is counted twice or lost.
    float lo[SMP_ROUNDS], inv_w[SMP_ROUNDS];
    int pick[SMP_ROUNDS];
    float lo_d = 0.f, width = SMP_SPAN / SMP_FAN;
    float mb = 0.f;                          // mass of everything more likely than the bucket in hand
    bool found = true;
    if (tid == 0) list_n = 0;
    auto bucket_of = [&](float d, int q) -> int {
      float fb = (d - lo[q]) * inv_w[q];
      if (q == 0) fb = fminf(fmaxf(fb, 0.f), (float)(SMP_FAN - 1));   // far tokens: last bucket
      return (fb >= 0.f && fb < (float)SMP_FAN) ? (int)fb : -1;
    };
#pragma unroll
    for (int round = 0; round < SMP_ROUNDS; ++round) {
      if (!found) break;
      lo[round] = lo_d;
      inv_w[round] = 1.0f / width;
      for (int b = 0; b < SMP_FAN; ++b) cols[b * SMP_THREADS + tid] = 0.f;
      for_row(ex, V, vec_ex, [&](int, float e) {
        const float d = fmaxf(-__builtin_amdgcn_logf(e) * 0.6931471805599453f, 0.f);   // e may be a hair above 1
        bool in = true;
#pragma unroll
        for (int q = 0; q < round; ++q) in = in && bucket_of(d, q) == pick[q];
        const int bk = bucket_of(d, round);
        if (in && bk >= 0) cols[bk * SMP_THREADS + tid] += e;
      });
      // bucket sums: wave sums, then sixteen threads add the waves' partial sums
      for (int b = 0; b < SMP_FAN; ++b) {
        const float v = wave_sum(cols[b * SMP_THREADS + tid]);
        if ((tid & 63) == 0) part[b * 16 + (tid >> 6)] = v;
      }
      __syncthreads();
      if (tid < SMP_FAN) {
        float v = 0.f;
        for (int w = 0; w < 16; ++w) v += part[tid * 16 + w];
        bucket[tid] = v;
      }
      __syncthreads();
      if (tid == 0) {
        float run = mb;
        int cb = -1;
        for (int b = 0; b < SMP_FAN; ++b) {
          if (run + bucket[b] > tp) { cb = b; break; }
          run += bucket[b];
        }
        cross_bin = cb;
        mass_before = run;
      }
      __syncthreads();
      pick[round] = cross_bin;
      mb = mass_before;
      if (pick[round] < 0) { found = false; break; }   // rounding left the whole mass <= top_p
      lo_d += pick[round] * width;
      width *= 1.0f / SMP_FAN;
    }
    if (found) {
      for_row(ex, V, vec_ex, [&](int, float e) {
        const float d = fmaxf(-__builtin_amdgcn_logf(e) * 0.6931471805599453f, 0.f);   // e may be a hair above 1
        bool in = true;
#pragma unroll
        for (int q = 0; q < SMP_ROUNDS; ++q) in = in && bucket_of(d, q) == pick[q];
        if (in) {
          const int at = atomicAdd(&list_n, 1);
          if (at < SMP_LIST) list[at] = e;
        }
      });
      __syncthreads();
      const int n = list_n;
      // lo keeps mass_above(lo) > top_p, hi keeps mass_above(hi) <= top_p
      uint32_t lo = 0u, hi = __float_as_uint(2.0f);
      if (n <= SMP_LIST) {
        if (tid < 64) {                      // the list is short: one wave bisects it
          while (hi - lo > 1u) {
            const uint32_t mid = lo + ((hi - lo) >> 1);
            const float t = __uint_as_float(mid);
            float mass = 0.f;
            for (int i = tid; i < n; i += 64) mass += list[i] > t ? list[i] : 0.f;
            mass = wave_sum(mass) + mb;
            if (mass <= tp) hi = mid; else lo = mid;
          }
          if (tid == 0) thr_s = __uint_as_float(lo);
        }
        __syncthreads();
      } else {                               // too many tokens in one bucket: bisect over the whole row
        while (hi - lo > 1u) {
          const uint32_t mid = lo + ((hi - lo) >> 1);
          const float t = __uint_as_float(mid);
          float mass = 0.f;
          for (int i = tid; i < V; i += SMP_THREADS) {
            const float e = ex[i];
            if (e > t) mass += e;
          }
          mass = block_sum(mass, scratch);
          if (mass <= tp) hi = mid; else lo = mid;
        }
        if (tid == 0) thr_s = __uint_as_float(lo);
        __syncthreads();
      }
      thr = thr_s;
      // the most likely token (e = 1 up to rounding) is always kept: nothing lies before it
      if (thr >= 0.9999f) thr = 0.9999f;
    }
  }

  // inverse-CDF draw in vocabulary order. Every wave owns a contiguous range and reads it
  // 64 tokens at a time (coalesced); the waves' kept masses are scanned, and the wave whose
  // range holds u * kept walks it again with a running prefix.
  const int lane = tid & 63, wave = tid >> 6;
  const int per_wave = ((V + 15) / 16 + 63) / 64 * 64;
  const int wb = wave * per_wave, we = min(V, wb + per_wave);
  float mine = 0.f;
  for (int i = wb + lane; i < we; i += 64) {
    const float e = ex[i];
    if (e > thr) mine += e;
  }
  mine = wave_sum(mine);
  float kept;
  const float before = block_exclusive_scan(lane == 0 ? mine : 0.f, scratch, &kept);
  const float wave_before = __shfl(before, 0, 64);
  const float target = uniform[r] * kept;
  if (tid == 0) { out[r] = -1; last_kept = 0; }
  __syncthreads();
  if (mine > 0.f) {
    const bool owner = wave_before <= target && target < wave_before + mine;
    float run = wave_before;
    int choice = -1, my_last = -1;
    for (int i0 = wb; i0 < we; i0 += 64 * 8) {
      float ev[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) {           // eight loads in flight, then eight scans
        const int i = i0 + 64 * k + lane;
        ev[k] = (i < we) ? ex[i] : 0.f;
      }
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const int i = i0 + 64 * k + lane;
        const float v = ev[k] > thr ? ev[k] : 0.f;
        if (v > 0.f) my_last = i;
        if (owner && choice < 0) {
          float inc = v;
#pragma unroll
          for (int o = 1; o < 64; o <<= 1) {
            const float nb = __shfl_up(inc, o, 64);
            if (lane >= o) inc += nb;
          }
          const unsigned long long hit = __ballot(v > 0.f && run + inc > target);
          if (hit) choice = i0 + 64 * k + __ffsll((long long)hit) - 1;
          run += __shfl(inc, 63, 64);
        }
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) my_last = max(my_last, __shfl_xor(my_last, o, 64));
    if (lane == 0) {
      if (owner) out[r] = choice >= 0 ? choice : my_last;
      atomicMax(&last_kept, my_last);
    }
  }
  __syncthreads();
  // rounding may leave the target past the last kept token: take that token
  if (tid == 0 && out[r] < 0) out[r] = last_kept;
  if (want_probs) {
    const float inv_kept = 1.0f / kept;
    for (int i = tid; i < V; i += SMP_THREADS) {
      const float e = ex[i];
      ex[i] = e > thr ? e * inv_kept : 0.f;
    }
  }
#undef BIN
}

extern "C" int ptl_sample_top_p(int32_t* out, float* work, int want_probs, const float* logits, int R,
                                int V, long stride, const float* temperature, const float* top_p,
                                const float* uniform, hipStream_t stream) {
  if (R <= 0) return PTL_OK;
  if (V <= 0 || stride < V || !work) return PTL_ERR_ARG;
  sample_top_p_kernel<<<R, SMP_THREADS, 0, stream>>>(out, work, want_probs, logits, V, stride,
                                                     temperature, top_p, uniform);
  return ptl_launch_status();
}

// ptl_token_logprob: out[r] = log_softmax(logits[r])[tokens[r]], the log-probability the
// reference reports for a generated token (F.log_softmax of the step's logits gathered at
// the token, lite_llama/generete_with_probs.py:154-165). One workgroup a row.
__global__ void __launch_bounds__(1024)
token_logprob_kernel(float* __restrict__ out, const float* __restrict__ logits,
                     const int32_t* __restrict__ tokens, int V, long stride) {
  __shared__ float scratch[16];
  const float* row = logits + (size_t)blockIdx.x * stride;
  float mx = -INFINITY;
  for (int i = threadIdx.x; i < V; i += blockDim.x) mx = fmaxf(mx, row[i]);
  mx = block_max(mx, scratch);
  float z = 0.f;
  for (int i = threadIdx.x; i < V; i += blockDim.x) z += expf(row[i] - mx);
  z = block_sum(z, scratch);
  if (threadIdx.x == 0) {
    const int t = tokens[blockIdx.x];
    out[blockIdx.x] = (t >= 0 && t < V) ? row[t] - mx - logf(z) : -INFINITY;
  }
}

extern "C" int ptl_token_logprob(float* out, const float* logits, const int32_t* tokens, int R, int V,
                                 long stride, hipStream_t stream) {
  if (R <= 0) return PTL_OK;
  if (V <= 0 || stride < V) return PTL_ERR_ARG;
  token_logprob_kernel<<<R, 1024, 0, stream>>>(out, logits, tokens, V, stride);
  return ptl_launch_status();
}
