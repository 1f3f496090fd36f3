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
#include "no_alloc.h"
#include <math.h>
#include <mutex>

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
  if (hi - lo == ARGMAX_CHUNK && (reinterpret_cast<uintptr_t>(row + lo) & 15) == 0) {
    // a whole chunk with 16-byte aligned rows: a thread's four loads are asked for at once
    float4 v[ARGMAX_CHUNK / 1024];
#pragma unroll
    for (int k = 0; k < ARGMAX_CHUNK / 1024; ++k)
      v[k] = *reinterpret_cast<const float4*>(row + lo + 4 * (threadIdx.x + 256 * k));
#pragma unroll
    for (int k = 0; k < ARGMAX_CHUNK / 1024; ++k) {
      const float e[4] = {v[k].x, v[k].y, v[k].z, v[k].w};
#pragma unroll
      for (int j = 0; j < 4; ++j)
        argmax_pick(best, bi, e[j] != e[j] ? -INFINITY : e[j], lo + 4 * (threadIdx.x + 256 * k) + j);
    }
  } else {
    for (int i = lo + threadIdx.x; i < hi; i += 256) {
      float v = row[i];
      if (v != v) v = -INFINITY;
      argmax_pick(best, bi, v, i);
    }
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

// host_out (optional): pinned host memory that receives the choices as well, written over the
// bus by this kernel, so that the host needs no copy after it
__global__ void __launch_bounds__(64)
argmax_final_kernel(int32_t* __restrict__ out, const float* __restrict__ pv,
                    const int32_t* __restrict__ pi, int chunks, int32_t* __restrict__ host_out) {
  float best = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = threadIdx.x; i < chunks; i += 64)
    argmax_pick(best, bi, pv[(size_t)blockIdx.x * chunks + i], pi[(size_t)blockIdx.x * chunks + i]);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) argmax_pick(best, bi, __shfl_xor(best, o, 64), __shfl_xor(bi, o, 64));
  if (threadIdx.x == 0) {
    const int choice = bi == 0x7fffffff ? 0 : bi;
    out[blockIdx.x] = choice;
    if (host_out != nullptr) host_out[blockIdx.x] = choice;
  }
}

// workspace: float [R, chunks] and int32 [R, chunks], chunks = ceil(V / 4096)
extern "C" int ptl_argmax(int32_t* out, const float* logits, int R, int V, long stride,
                          float* ws_val, int32_t* ws_idx, int32_t* host_out, hipStream_t stream) {
  if (R <= 0) return PTL_OK;
  if (V <= 0 || stride < V || !ws_val || !ws_idx || R > 65535) return PTL_ERR_ARG;
  const int chunks = (V + ARGMAX_CHUNK - 1) / ARGMAX_CHUNK;
  dim3 grid(chunks, R);
  argmax_partial_kernel<<<grid, 256, 0, stream>>>(ws_val, ws_idx, logits, V, stride, chunks);
  if (hipGetLastError() != hipSuccess) return PTL_ERR_LAUNCH;
  argmax_final_kernel<<<R, 64, 0, stream>>>(out, ws_val, ws_idx, chunks, host_out);
  return ptl_launch_status();
}

// ptl_argmax with its workspace inside the library (see no_alloc.h): values in the first half of
// the array, indices in the second. Host code never uses the array's name as an address: the
// name is a host-side stand-in; the device address comes from hipGetSymbolAddress, once per
// device with that device current (every GPU holds a copy of its own), and is what the
// kernels are given.
static __device__ __align__(256) unsigned char argmax_scratch[PTL_ARGMAX_STATIC_MAX_PARTIALS * 8];
#define ARGMAX_STATIC_MAX_DEVICES 64
static void* argmax_scratch_at[ARGMAX_STATIC_MAX_DEVICES];
static std::mutex argmax_scratch_lock;

// The array's address on device ``dev``, looked up the first time with that device current.
// ``may_look_up`` false: only what is known already (a look-up may load the code object onto the
// device, which is no work for a stream that is being captured).
static int argmax_scratch_of(int dev, bool may_look_up, void** base) {
  if (dev < 0 || dev >= ARGMAX_STATIC_MAX_DEVICES) return PTL_ERR_LAUNCH;
  std::lock_guard<std::mutex> hold(argmax_scratch_lock);
  if (argmax_scratch_at[dev] == nullptr) {
    if (!may_look_up) return PTL_ERR_LAUNCH;
    int current = -1;
    if (hipGetDevice(&current) != hipSuccess) {
      (void)hipGetLastError();
      return PTL_ERR_LAUNCH;
    }
    if (current != dev && hipSetDevice(dev) != hipSuccess) {
      (void)hipGetLastError();
      return PTL_ERR_LAUNCH;
    }
    void* p = nullptr;
    const hipError_t found = hipGetSymbolAddress(&p, HIP_SYMBOL(argmax_scratch));
    if (current != dev) (void)hipSetDevice(current);
    if (found != hipSuccess || p == nullptr) {
      (void)hipGetLastError();
      return PTL_ERR_LAUNCH;
    }
    argmax_scratch_at[dev] = p;
  }
  *base = argmax_scratch_at[dev];
  return PTL_OK;
}

// The device a stream belongs to (the current device for the null stream).
static int device_of(hipStream_t stream) {
  int dev = -1;
  if (stream != nullptr && hipStreamGetDevice(stream, &dev) == hipSuccess) return dev;
  (void)hipGetLastError();
  if (hipGetDevice(&dev) != hipSuccess) {
    (void)hipGetLastError();
    return -1;
  }
  return dev;
}

extern "C" int ptl_argmax_static_init(void) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess) {
    (void)hipGetLastError();
    return PTL_ERR_LAUNCH;
  }
  void* base = nullptr;
  return argmax_scratch_of(dev, true, &base);
}

extern "C" int ptl_argmax_static(int32_t* out, const float* logits, int R, int V, long stride,
                                 int32_t* host_out, hipStream_t stream) {
  if (R <= 0) return PTL_OK;
  if (!out || !logits || V <= 0 || stride < V || R > 65535) return PTL_ERR_ARG;
  const long chunks = ((long)V + ARGMAX_CHUNK - 1) / ARGMAX_CHUNK;
  if ((long)R * chunks > PTL_ARGMAX_STATIC_MAX_PARTIALS) return PTL_ERR_ARG;
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &capturing) != hipSuccess) {
    (void)hipGetLastError();
    capturing = hipStreamCaptureStatusNone;
  }
  void* base = nullptr;
  const int rc = argmax_scratch_of(device_of(stream), capturing == hipStreamCaptureStatusNone, &base);
  if (rc != PTL_OK) return rc;
  float* ws_val = reinterpret_cast<float*>(base);
  int32_t* ws_idx = reinterpret_cast<int32_t*>(static_cast<unsigned char*>(base) +
                                               (size_t)PTL_ARGMAX_STATIC_MAX_PARTIALS * 4);
  return ptl_argmax(out, logits, R, V, stride, ws_val, ws_idx, host_out, stream);
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
    // (four loads under way at a time: a pass is a chain of L2 round trips otherwise)
    const int n4 = V >> 2;
    const int step = blockDim.x;
    const float4* p4 = reinterpret_cast<const float4*>(p);
    int i = threadIdx.x;
    for (; i + 3 * step < n4; i += 4 * step) {
      float4 v[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] = p4[i + j * step];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int at = 4 * (i + j * step);
        f(at, v[j].x); f(at + 1, v[j].y); f(at + 2, v[j].z); f(at + 3, v[j].w);
      }
    }
    for (; i < n4; i += step) {
      const float4 v = p4[i];
      f(4 * i, v.x); f(4 * i + 1, v.y); f(4 * i + 2, v.z); f(4 * i + 3, v.w);
    }
    for (int t = 4 * n4 + threadIdx.x; t < V; t += step) f(t, p[t]);
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
  // (a NaN logit counts as -inf: probability 0)
  float emax = 0.f;                          // the largest e (1 up to rounding)
  auto expo = [&](float x) {
    const float e = x != x ? 0.f : __builtin_amdgcn_exp2f(fmaf(x, c, -mc));
    emax = fmaxf(emax, e);
    return e;
  };
  if (vec_in && vec_ex) {
    const int n4 = V >> 2;
    auto exp4 = [&](int i, float4 x) {
      float4 e;
      e.x = expo(x.x);
      e.y = expo(x.y);
      e.z = expo(x.z);
      e.w = expo(x.w);
      reinterpret_cast<float4*>(ex)[i] = e;
      z += (e.x + e.y) + (e.z + e.w);
    };
    int i = tid;
    for (; i + 3 * SMP_THREADS < n4; i += 4 * SMP_THREADS) {
      float4 x[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) x[j] = reinterpret_cast<const float4*>(row)[i + j * SMP_THREADS];
#pragma unroll
      for (int j = 0; j < 4; ++j) exp4(i + j * SMP_THREADS, x[j]);
    }
    for (; i < n4; i += SMP_THREADS) exp4(i, reinterpret_cast<const float4*>(row)[i]);
    for (int i = 4 * n4 + tid; i < V; i += SMP_THREADS) {
      const float e = expo(row[i]);
      ex[i] = e;
      z += e;
    }
  } else {
    for (int i = tid; i < V; i += SMP_THREADS) {
      const float e = expo(row[i]);
      ex[i] = e;
      z += e;
    }
  }
  z = block_sum(z, scratch);                 // (its barriers also publish ex[] to the block)
  emax = block_max(emax, scratch);
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
      // the most likely token is always kept: nothing lies before it
      if (thr >= emax) thr = __uint_as_float(__float_as_uint(emax) - 1u);
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

// ===========================================================================
// ptl_sample_top_p_wide: the same rule for rows of vocabulary size, spread over the chip.
//
// One workgroup reads a row of 128k logits at a small part of what the chip can deliver, and
// the kernel above passes over the row seven times. Here a row is cut into chunks of 4096
// logits, a workgroup a chunk, and the passes become kernels:
//   (1) minmax:  every chunk's largest and smallest finite logit;
//   (2) exp:     e = exp(x/T - max) into the work buffer, the chunk's sum, and the chunk's
//                histogram of mass over 2048 buckets of x, equally wide, from the row's max
//                down to its min (at most 32 T below the max; what lies further goes to the
//                last bucket). The histogram is summed in LDS in fixed point (2^-40) with
//                integer atomics, so that it does not depend on the order of the threads;
//   (3) combine: the chunks' histograms added in chunk order;
//   (4) gather:  every workgroup finds the bucket in which the mass, most likely tokens first,
//                passes top_p (same code, same numbers: same answer), adds up what its chunk
//                has above that bucket and hands on its tokens inside it (at most 256);
//   (5) draw:    one workgroup a row bisects over the bit patterns of x among the tokens handed
//                on (a few hundred) for the exact edge of the nucleus, adds the kept mass chunk
//                by chunk, finds the chunk that holds u * kept and walks it;
//   (6) probs:   only if asked for, the renormalised nucleus distribution.
// A token is kept iff it lies in a bucket above the crossing one, or in it and above the edge;
// equal logits are kept or dropped together. If a chunk has more than 256 tokens in the crossing
// bucket, or the row more than 4096 (many equal logits), the draw kernel bisects over the whole
// row instead: slower, same result. Everything is added in a fixed order: the same logits,
// parameters and u give the same token.
// ===========================================================================
#define SW_CHUNK 4096
#define SW_THREADS 256
#define SW_PER (SW_CHUNK / SW_THREADS)
#define SW_BUCKETS 2048
#define SW_SEG 256
#define SW_LIST 4096
#define SW_SPAN 32.0f
#define SW_FIXED 1099511627776.0f        // 2^40

// where a row's pieces lie in the workspace (all 4-byte words)
struct SwRow {
  float *cmax, *cmin, *csum, *ckept, *hist, *tot, *seg_x, *result;
  int32_t *ccount, *seg_i;
};
__host__ __device__ static inline size_t sw_row_words(int S) {
  return (size_t)5 * S + (size_t)S * SW_BUCKETS + SW_BUCKETS + (size_t)2 * S * SW_SEG + 8;
}
__device__ __forceinline__ SwRow sw_row(float* ws, int r, int S) {
  float* p = ws + (size_t)r * sw_row_words(S);
  SwRow w;
  w.cmax = p; p += S;
  w.cmin = p; p += S;
  w.csum = p; p += S;
  w.ckept = p; p += S;
  w.ccount = reinterpret_cast<int32_t*>(p); p += S;
  w.hist = p; p += (size_t)S * SW_BUCKETS;
  w.tot = p; p += SW_BUCKETS;
  w.seg_x = p; p += (size_t)S * SW_SEG;
  w.seg_i = reinterpret_cast<int32_t*>(p); p += (size_t)S * SW_SEG;
  w.result = p;        // [0] edge key (bits), [1] crossing bucket (bits), [2] kept mass, [3] mass before
                       // the crossing bucket, [4] row max, [5] buckets per unit of x, [6] sum of e
  return w;
}

// bit patterns that order as the floats do
__device__ __forceinline__ uint32_t sw_key(float x) {
  const uint32_t b = __float_as_uint(x);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
// a NaN logit counts as -inf; -0 and +0 are one value (their bit patterns differ)
__device__ __forceinline__ float sw_clean(float x) { return x != x ? -INFINITY : (x == 0.f ? 0.f : x); }

struct SwScale {
  float mx, inv_w, c, mc, z;               // row max, buckets per unit of x, log2(e)/T, mx*c, sum of e
};
// Every wave of every workgroup of a row computes this from the same numbers in the same order:
// lane c takes chunk c (S <= 64), and the lanes meet in a butterfly, which gives all of them
// the same bits.
__device__ __forceinline__ SwScale sw_scale(const SwRow& w, int S, float T, bool with_sum) {
  const int lane = threadIdx.x & 63;
  const float mx = wave_max(lane < S ? w.cmax[lane] : -INFINITY);
  const float mn = -wave_max(lane < S ? -w.cmin[lane] : -INFINITY);
  SwScale s;
  s.z = with_sum ? wave_sum(lane < S ? w.csum[lane] : 0.f) : 0.f;
  s.mx = mx;
  s.c = 1.4426950408889634f / T;
  s.mc = mx * s.c;
  const float span = fminf(mx - mn, SW_SPAN * T);
  s.inv_w = span > 0.f ? (float)SW_BUCKETS / span : 0.f;
  return s;
}
__device__ __forceinline__ int sw_bucket(float x, const SwScale& s) {
  const float fb = (s.mx - x) * s.inv_w;                 // (NaN when -inf meets inv_w 0: bucket 0)
  return (int)fminf(fmaxf(fb, 0.f), (float)(SW_BUCKETS - 1));
}
__device__ __forceinline__ bool sw_kept(float x, const SwScale& s, int cross, uint32_t edge) {
  const int b = sw_bucket(x, s);
  return b < cross || (b == cross && sw_key(x) > edge);
}

__global__ void __launch_bounds__(SW_THREADS)
sw_minmax_kernel(float* __restrict__ ws, const float* __restrict__ logits, int V, long stride, int S) {
  __shared__ float scratch[16];
  const int r = blockIdx.y, c = blockIdx.x;
  const SwRow w = sw_row(ws, r, S);
  const float* row = logits + (size_t)r * stride;
  const int lo = c * SW_CHUNK;
  float mx = -INFINITY, mn = INFINITY;
#pragma unroll
  for (int j = 0; j < SW_PER; ++j) {
    const int i = lo + j * SW_THREADS + threadIdx.x;
    const float x = i < V ? sw_clean(row[i]) : -INFINITY;
    mx = fmaxf(mx, x);
    if (x > -INFINITY) mn = fminf(mn, x);
  }
  mx = block_max(mx, scratch);
  mn = -block_max(-mn, scratch);
  if (threadIdx.x == 0) { w.cmax[c] = mx; w.cmin[c] = mn; }
}

__global__ void __launch_bounds__(SW_THREADS)
sw_exp_hist_kernel(float* __restrict__ ws, float* __restrict__ work, const float* __restrict__ logits,
                   int V, long stride, int S, const float* __restrict__ temperature) {
  __shared__ unsigned long long hist[SW_BUCKETS];
  __shared__ float scratch[16];
  const int r = blockIdx.y, c = blockIdx.x;
  const SwRow w = sw_row(ws, r, S);
  const float* row = logits + (size_t)r * stride;
  float* ex = work + (size_t)r * V;
  const SwScale s = sw_scale(w, S, temperature[r], false);
  for (int b = threadIdx.x; b < SW_BUCKETS; b += SW_THREADS) hist[b] = 0ull;
  __syncthreads();
  const int lo = c * SW_CHUNK;
  float x[SW_PER];
#pragma unroll
  for (int j = 0; j < SW_PER; ++j) {
    const int i = lo + j * SW_THREADS + threadIdx.x;
    x[j] = i < V ? sw_clean(row[i]) : -INFINITY;
  }
  float z = 0.f;
#pragma unroll
  for (int j = 0; j < SW_PER; ++j) {
    const int i = lo + j * SW_THREADS + threadIdx.x;
    if (i < V) {
      const float e = __builtin_amdgcn_exp2f(fmaf(x[j], s.c, -s.mc));
      ex[i] = e;
      z += e;
      atomicAdd(&hist[sw_bucket(x[j], s)], (unsigned long long)(e * SW_FIXED + 0.5f));
    }
  }
  z = block_sum(z, scratch);               // (its barriers also complete the histogram)
  if (threadIdx.x == 0) w.csum[c] = z;
  float* out = w.hist + (size_t)c * SW_BUCKETS;
  for (int b = threadIdx.x; b < SW_BUCKETS; b += SW_THREADS) out[b] = (float)hist[b] * (1.0f / SW_FIXED);
}

__global__ void __launch_bounds__(SW_THREADS)
sw_combine_kernel(float* __restrict__ ws, int S) {
  const SwRow w = sw_row(ws, blockIdx.y, S);
  const int b = blockIdx.x * SW_THREADS + threadIdx.x;
  float t = 0.f;
  for (int c0 = 0; c0 < S; c0 += 8) {      // eight loads under way, added in chunk order
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = c0 + j < S ? w.hist[(size_t)(c0 + j) * SW_BUCKETS + b] : 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) t += v[j];
  }
  w.tot[b] = t;
}

// The bucket in which the mass, most likely tokens first, passes tp, and the mass before it;
// SW_BUCKETS if it never does (everything is kept). The first SW_THREADS threads work, every
// thread of the block must call (barriers). tmp: 8 floats and 2 ints of LDS.
__device__ __forceinline__ void sw_crossing(const float* __restrict__ tot, float tp, float* tmp,
                                            int* itmp, int* cross, float* before) {
  constexpr int PER = SW_BUCKETS / SW_THREADS;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const bool works = tid < SW_THREADS;
  float v[PER], mine = 0.f;
  if (works) {
#pragma unroll
    for (int j = 0; j < PER; ++j) { v[j] = tot[tid * PER + j]; mine += v[j]; }
  }
  float inc = mine;
  if (works) {
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const float n = __shfl_up(inc, o, 64);
      if (lane >= o) inc += n;
    }
  }
  if (tid == 0) { itmp[0] = SW_BUCKETS; }
  if (works && lane == 63) tmp[wave] = inc;
  __syncthreads();
  float run = 0.f;
  if (works) {
    for (int i = 0; i < wave; ++i) run += tmp[i];
    run += inc - mine;                     // mass before this thread's buckets
    int first = SW_BUCKETS;
    float r2 = run;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      if (first == SW_BUCKETS && r2 + v[j] > tp) first = tid * PER + j;
      if (first == SW_BUCKETS) r2 += v[j];
    }
    if (first < SW_BUCKETS) atomicMin(&itmp[0], first);
  }
  __syncthreads();
  const int cb = itmp[0];
  if (works && cb < SW_BUCKETS && cb / PER == tid) {
    float r2 = run;
    for (int j = 0; j < cb - tid * PER; ++j) r2 += v[j];
    tmp[4] = r2;
  }
  __syncthreads();
  *cross = cb;
  *before = cb < SW_BUCKETS ? tmp[4] : 0.f;
}

__global__ void __launch_bounds__(SW_THREADS)
sw_gather_kernel(float* __restrict__ ws, const float* __restrict__ work, const float* __restrict__ logits,
                 int V, long stride, int S, const float* __restrict__ temperature,
                 const float* __restrict__ top_p) {
  __shared__ float tmp[17];
  __shared__ int itmp[2];
  const int r = blockIdx.y, c = blockIdx.x;
  const SwRow w = sw_row(ws, r, S);
  const float* row = logits + (size_t)r * stride;
  const float* ex = work + (size_t)r * V;
  const SwScale s = sw_scale(w, S, temperature[r], true);
  int cross = SW_BUCKETS;
  float before = 0.f;
  if (top_p[r] < 1.0f) sw_crossing(w.tot, top_p[r] * s.z, tmp, itmp, &cross, &before);
  const int lo = c * SW_CHUNK;
  float x[SW_PER], e[SW_PER];
#pragma unroll
  for (int j = 0; j < SW_PER; ++j) {
    const int i = lo + j * SW_THREADS + threadIdx.x;
    x[j] = i < V ? sw_clean(row[i]) : -INFINITY;
    e[j] = i < V ? ex[i] : 0.f;
  }
  float sure = 0.f;
  int mine = 0;
  bool in[SW_PER];
#pragma unroll
  for (int j = 0; j < SW_PER; ++j) {
    const int i = lo + j * SW_THREADS + threadIdx.x;
    const int b = sw_bucket(x[j], s);
    in[j] = i < V && b == cross;
    if (i < V && b < cross) sure += e[j];
    mine += in[j] ? 1 : 0;
  }
  float total;
  const int at0 = (int)block_exclusive_scan((float)mine, tmp, &total);   // (counts up to 4096: exact)
  sure = block_sum(sure, tmp);
  if (threadIdx.x == 0) {
    w.ckept[c] = sure;
    w.ccount[c] = (int)total;
    if (c == 0) {                          // what every workgroup of the row found, for the draw
      w.result[1] = __int_as_float(cross);
      w.result[3] = before;
      w.result[4] = s.mx;
      w.result[5] = s.inv_w;
      w.result[6] = s.z;
    }
  }
  int at = at0;
#pragma unroll
  for (int j = 0; j < SW_PER; ++j) {
    if (in[j]) {
      if (at < SW_SEG) {
        w.seg_x[(size_t)c * SW_SEG + at] = x[j];
        w.seg_i[(size_t)c * SW_SEG + at] = lo + j * SW_THREADS + threadIdx.x;
      }
      ++at;
    }
  }
}

// inclusive prefix over the lanes of a wave, in a fixed order
__device__ __forceinline__ float wave_inclusive_scan(float v) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const float n = __shfl_up(v, o, 64);
    if (lane >= o) v += n;
  }
  return v;
}

__global__ void __launch_bounds__(SW_THREADS)
sw_draw_kernel(int32_t* __restrict__ out, float* __restrict__ ws, const float* __restrict__ work,
               const float* __restrict__ logits, int V, long stride, int S,
               const float* __restrict__ temperature, const float* __restrict__ top_p,
               const float* __restrict__ uniform) {
  __shared__ float tmp[17];
  __shared__ float list_x[SW_LIST], list_e[SW_LIST];
  __shared__ int seg_at[65];
  __shared__ uint32_t edge_s, vote_key[4];
  __shared__ int vote_low[4];
  __shared__ int pick_chunk, last_kept, choice_s;
  __shared__ float pick_before, kept_s;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = blockIdx.x;
  const SwRow w = sw_row(ws, r, S);
  const float* row = logits + (size_t)r * stride;
  const float* ex = work + (size_t)r * V;
  // what the gather kernel's workgroups agreed on
  const int cross = __float_as_int(w.result[1]);
  const float before = w.result[3];
  SwScale s;
  s.mx = w.result[4];
  s.inv_w = w.result[5];
  s.z = w.result[6];
  s.c = 1.4426950408889634f / temperature[r];
  s.mc = s.mx * s.c;
  const float tp = top_p[r] * s.z;
  const int my_count = lane < S ? w.ccount[lane] : 0;
  const float my_sure = lane < S ? w.ckept[lane] : 0.f;
  if (tid == 0) { last_kept = -1; choice_s = -1; }

  uint32_t edge = 0u;                      // kept inside the crossing bucket: key > edge
  bool whole_row = false;
  int n = 0;
  if (cross < SW_BUCKETS) {
    // where every chunk's tokens go in the list (every wave computes the same)
    const int fits = min(my_count, SW_SEG);
    const int upto = (int)wave_inclusive_scan((float)fits);          // (small integers: exact)
    n = __shfl(upto, 63, 64);
    whole_row = __any(my_count > SW_SEG) || n > SW_LIST;
    if (wave == 0 && lane < S) { seg_at[lane] = upto - fits; seg_at[lane + 1] = upto; }
    __syncthreads();
    // lo keeps mass_above(lo) > tp, hi keeps mass_above(hi) <= tp (mass_above counts key > t)
    uint32_t lo = 0u, hi = 0xffffffffu;
    if (!whole_row) {
      for (int c = tid >> 3; c < S; c += SW_THREADS / 8) {            // eight threads a chunk
        const int base = seg_at[c], k = seg_at[c + 1] - base;
        for (int j = tid & 7; j < k; j += 8) {
          const int i = w.seg_i[(size_t)c * SW_SEG + j];
          list_x[base + j] = w.seg_x[(size_t)c * SW_SEG + j];
          list_e[base + j] = ex[i];
        }
      }
      __syncthreads();
      if (n <= SW_THREADS) {
        // Few tokens: every one of them asks directly whether it is kept (the mass of the
        // tokens above it, added in list order, and what lies before the bucket); the edge is
        // the smallest kept key, less one.
        uint32_t lowest = 0xffffffffu;
        for (int i = tid; i < n; i += SW_THREADS) {
          const uint32_t k = sw_key(list_x[i]);
          float mass = 0.f;
          for (int j = 0; j < n; ++j) mass += sw_key(list_x[j]) > k ? list_e[j] : 0.f;
          if (mass + before <= tp) lowest = min(lowest, k);
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) lowest = min(lowest, (uint32_t)__shfl_xor((int)lowest, o, 64));
        if (lane == 0) vote_key[wave] = lowest;
        __syncthreads();
        lowest = min(min(vote_key[0], vote_key[1]), min(vote_key[2], vote_key[3]));
        edge = lowest - 1u;                // (no token kept: 0xfffffffe, nothing in the bucket passes)
        if (lowest == 0xffffffffu) edge = 0xffffffffu;
      } else {
        // The edge lies between the list's smallest key (less one: everything above it is the
        // whole list) and its largest (nothing above it). Four waves try four keys a round.
        uint32_t kmin = 0xffffffffu, kmax = 0u;
        for (int i = lane; i < n; i += 64) {
          const uint32_t k = sw_key(list_x[i]);
          kmin = min(kmin, k);
          kmax = max(kmax, k);
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
          kmin = min(kmin, (uint32_t)__shfl_xor((int)kmin, o, 64));
          kmax = max(kmax, (uint32_t)__shfl_xor((int)kmax, o, 64));
        }
        lo = kmin - 1u;
        hi = kmax;
        while (hi - lo > 1u) {
          // gap keys lie strictly between lo and hi; wave v tries one of them: all of them
          // when there are at most four, else four spread evenly
          const uint32_t gap = hi - lo - 1u;
          const bool mine = gap > 4u || (uint32_t)wave < gap;
          const uint32_t mid = gap > 4u
              ? lo + 1u + (uint32_t)(((unsigned long long)gap * (uint32_t)(wave + 1)) / 5u)
              : lo + 1u + (uint32_t)wave;
          float mass = 0.f;
          if (mine) {
            for (int i = lane; i < n; i += 64) mass += sw_key(list_x[i]) > mid ? list_e[i] : 0.f;
            mass = wave_sum(mass) + before;
          }
          __syncthreads();
          if (lane == 0) { vote_key[wave] = mine ? mid : 0u; vote_low[wave] = !mine ? -1 : (mass > tp ? 1 : 0); }
          __syncthreads();
          uint32_t nlo = lo, nhi = hi;
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            if (vote_low[v] == 1) nlo = max(nlo, vote_key[v]);
            if (vote_low[v] == 0) nhi = min(nhi, vote_key[v]);
          }
          lo = nlo; hi = nhi;
        }
        edge = lo;
      }
    } else {                               // too many tokens in one bucket: bisect over the whole row
      while (hi - lo > 1u) {
        const uint32_t mid = lo + ((hi - lo) >> 1);
        float mass = 0.f;
        for (int i = tid; i < V; i += SW_THREADS) {
          const float x = sw_clean(row[i]);
          if (sw_bucket(x, s) == cross && sw_key(x) > mid) mass += ex[i];
        }
        mass = block_sum(mass, tmp) + before;
        if (mass <= tp) hi = mid; else lo = mid;
      }
      edge = lo;
    }
    // the most likely token is always kept: nothing lies before it
    if (cross == 0 && edge >= sw_key(s.mx)) edge = sw_key(s.mx) - 1u;
  }

  // kept mass chunk by chunk: what lies above the crossing bucket, and the kept part of it;
  // wave 0 (lane c: chunk c) adds them up and finds the chunk that holds the target
  float extra = 0.f;
  if (whole_row) {
    for (int c = 0; c < S; ++c) {
      float part = 0.f;
      for (int i = c * SW_CHUNK + tid; i < min(V, (c + 1) * SW_CHUNK); i += SW_THREADS) {
        const float x = sw_clean(row[i]);
        if (sw_bucket(x, s) == cross && sw_key(x) > edge) part += ex[i];
      }
      part = block_sum(part, tmp);
      if (lane == c) extra = part;
    }
  } else if (cross < SW_BUCKETS && lane < S) {
    for (int j = seg_at[lane]; j < seg_at[lane + 1]; ++j) extra += sw_key(list_x[j]) > edge ? list_e[j] : 0.f;
  }
  if (wave == 0) {
    const float mass = my_sure + extra;
    const float upto = wave_inclusive_scan(mass);
    const float kept = __shfl(upto, 63, 64);
    const float target = uniform[r] * kept;
    const unsigned long long holds = __ballot(mass > 0.f && upto > target);
    const unsigned long long any = __ballot(mass > 0.f);
    if (lane == 0) {
      int pc;
      if (holds) {
        pc = __ffsll((long long)holds) - 1;
      } else {                             // rounding: past the last kept token
        pc = any ? 63 - __clzll((long long)any) : 0;
      }
      pick_chunk = pc;
      kept_s = kept;
      w.result[0] = __uint_as_float(edge);
      w.result[2] = kept;
    }
    if (holds && lane == __ffsll((long long)holds) - 1) pick_before = upto - mass;
    if (!holds && lane == 0) pick_before = -INFINITY;
  }
  __syncthreads();
  // walk the chunk that holds the target: sixteen consecutive tokens a thread
  const int c0 = pick_chunk * SW_CHUNK;
  const float target = uniform[r] * kept_s - pick_before;
  float xv[SW_PER], v[SW_PER], mine = 0.f;
  int my_last = -1;
#pragma unroll
  for (int k = 0; k < SW_PER; ++k) {
    const int i = c0 + SW_PER * tid + k;
    xv[k] = i < V ? sw_clean(row[i]) : -INFINITY;
    v[k] = i < V ? ex[i] : 0.f;
  }
#pragma unroll
  for (int k = 0; k < SW_PER; ++k) {
    const int i = c0 + SW_PER * tid + k;
    // (as a select: written as "if (!(...)) v[k] = 0" this loop kept what it should drop)
    const bool keep = i < V && sw_kept(xv[k], s, cross, edge);
    v[k] = keep ? v[k] : 0.f;
    if (v[k] > 0.f) my_last = i;
    mine += v[k];
  }
  float total;
  const float run = block_exclusive_scan(mine, tmp, &total);
  if (mine > 0.f && run <= target && target < run + mine) {
    int choice = my_last;
    float upto = run;
    bool found = false;
#pragma unroll
    for (int k = 0; k < SW_PER; ++k) {
      upto += v[k];
      if (!found && v[k] > 0.f && upto > target) { choice = c0 + SW_PER * tid + k; found = true; }
    }
    choice_s = choice;
  }
  if (my_last >= 0) atomicMax(&last_kept, my_last);
  __syncthreads();
  // rounding may leave the target past the chunk's last kept token: take that token
  if (tid == 0) out[r] = choice_s >= 0 ? choice_s : max(last_kept, 0);
}

__global__ void __launch_bounds__(SW_THREADS)
sw_probs_kernel(float* __restrict__ ws, float* __restrict__ work, const float* __restrict__ logits,
                int V, long stride, int S, const float* __restrict__ temperature) {
  const int r = blockIdx.y, c = blockIdx.x;
  const SwRow w = sw_row(ws, r, S);
  const float* row = logits + (size_t)r * stride;
  float* ex = work + (size_t)r * V;
  SwScale s;
  s.mx = w.result[4];
  s.inv_w = w.result[5];
  const uint32_t edge = __float_as_uint(w.result[0]);
  const int cross = __float_as_int(w.result[1]);
  const float inv_kept = 1.0f / w.result[2];
#pragma unroll
  for (int j = 0; j < SW_PER; ++j) {
    const int i = c * SW_CHUNK + j * SW_THREADS + threadIdx.x;
    if (i < V) ex[i] = sw_kept(sw_clean(row[i]), s, cross, edge) ? ex[i] * inv_kept : 0.f;
  }
}

// bytes of workspace ptl_sample_top_p_wide needs for R rows of V logits
extern "C" size_t ptl_sample_top_p_wide_workspace(int R, int V) {
  const int S = (V + SW_CHUNK - 1) / SW_CHUNK;
  return (size_t)R * sw_row_words(S) * sizeof(float);
}

// As ptl_sample_top_p; ws: ptl_sample_top_p_wide_workspace(R, V) bytes, 16-byte aligned.
// Rows of up to 64 chunks (262,144 logits).
extern "C" int ptl_sample_top_p_wide(int32_t* out, float* work, int want_probs, const float* logits,
                                     int R, int V, long stride, const float* temperature,
                                     const float* top_p, const float* uniform, float* ws,
                                     hipStream_t stream) {
  if (R <= 0) return PTL_OK;
  const int S = (V + SW_CHUNK - 1) / SW_CHUNK;
  if (V <= 0 || stride < V || !work || !ws || S > 64 || R > 65535) return PTL_ERR_ARG;
  const dim3 chunks(S, R);
  sw_minmax_kernel<<<chunks, SW_THREADS, 0, stream>>>(ws, logits, V, stride, S);
  sw_exp_hist_kernel<<<chunks, SW_THREADS, 0, stream>>>(ws, work, logits, V, stride, S, temperature);
  sw_combine_kernel<<<dim3(SW_BUCKETS / SW_THREADS, R), SW_THREADS, 0, stream>>>(ws, S);
  sw_gather_kernel<<<chunks, SW_THREADS, 0, stream>>>(ws, work, logits, V, stride, S, temperature, top_p);
  sw_draw_kernel<<<R, SW_THREADS, 0, stream>>>(out, ws, work, logits, V, stride, S, temperature, top_p, uniform);
  if (want_probs)
    sw_probs_kernel<<<chunks, SW_THREADS, 0, stream>>>(ws, work, logits, V, stride, S, temperature);
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
