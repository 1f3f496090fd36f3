// Attention of prompt portions over the paged cache on the matrix cores (bfloat16).
// The cache layout, the meaning of the arguments and the reference formulas are those of
// attention.hip; this kernel has a source file of its own because it is compiled with one more
// option (see max2 below).
#include "common.h"
#include "mfma.h"
#include <math.h>
#include <type_traits>

// ===========================================================================
// ptl_attention_prefill_mfma: bfloat16 prompt portions on the matrix cores.
//
// A workgroup of four waves takes 64 or 128 query rows of one head (16 or 32 per
// wave) and walks the sequence's keys in tiles of 64. Key and value tiles go
// through LDS as they lie in the cache (rows of D), in two buffers: while tile t
// is used, tile t+1 is on its way from global memory straight into the other
// buffer (global_load_lds_dwordx4, no register in between; its page numbers were
// read one tile earlier still), so a tile costs one barrier. Both products are
// computed transposed so that the scores leave the first MFMA in the register
// layout the second one wants, without a shuffle:
//   S^T[key, query] = K[key, :] . Q[query, :]      (A = K tile, B = Q^T)
//   O^T[d, query]  += V^T[d, key] . P^T[key, query] (A = V^T tile, B = P^T)
// with v_mfma_f32_16x16x32_bf16: a lane holds 8 consecutive k-values of row
// (lane % 16), k-group (lane / 16); the result tile holds rows 4*(lane/16)+i,
// column lane % 16. The V^T fragments come from the row-major value tile through
// ds_read_b64_tr_b16: in a group of 16 lanes, lane s gives the address of four
// consecutive elements E[s][0..3], and lane l receives E[4i + l/4][l%4], i = 0..3;
// with lane s pointing at V[key0 + s/4][d0 + 4*(s%4)], lane l gets
// V[key0 + 0..3][d0 + l]. Softmax is the online one of
// lite_llama/kernels/flashattentionv2.py:10-61 in base 2 (scale * log2 e folded
// into the scores, exp2), float32 max / denominator / accumulator; P is rounded
// to bfloat16 for the second product as there (:55). The running maximum is a
// stabiliser, not a result: it follows the scores only when they pass it by more
// than 8 (in the exponent's units), so that what is kept is rescaled rarely.
// Needs D % 32 == 0, D <= 128, a page size that is a power of two.
// ===========================================================================

#define PF_BN 64


// (This file is compiled with -fno-honor-nans: fmaxf then is one v_max, or half a v_max3,
// without a quieting v_max(x, x) in front of every score that comes out of an MFMA. No inline
// assembly for it: the compiler inserts the wait states between an MFMA and the first read of
// its result only for instructions it knows.)
__device__ __forceinline__ float max2(float a, float b) { return fmaxf(a, b); }
__device__ __forceinline__ s16x4_t lds_read_tr16(const bf16_t* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)p);
}

// RT: 16-row query tiles per wave; the workgroup takes 64 * RT query rows.
template <int NDT, int RT>
__global__ void __launch_bounds__(256, NDT <= 2 ? 3 : 2)
attn_prefill_mfma_kernel(bf16_t* __restrict__ out, long out_stride, const bf16_t* __restrict__ q,
                         long q_stride, const bf16_t* __restrict__ k_cache,
                         const bf16_t* __restrict__ v_cache, const int32_t* __restrict__ q_start,
                         const int32_t* __restrict__ ctx_len, const int32_t* __restrict__ block_table,
                         int bt_stride, const int32_t* __restrict__ work_seq,
                         const int32_t* __restrict__ work_qoff, int n_work, int Hq, int Hkv,
                         int page_size, int page_shift, int window, float scale_log2) {
  constexpr int D = 32 * NDT;
  constexpr int PBM = 64 * RT;
  constexpr int CPR = D / 8;           // 16-byte chunks per row
  constexpr int NCH = PF_BN * CPR / 256;   // chunks of a tile per thread
  // Tiles lie in LDS as rows of D elements without padding; the 16-byte chunks of a row are
  // permuted (chunk c of row r lies at c ^ swz(r)) so that neither the row-wise reads of the
  // first product nor the transposing reads of the second meet in a bank. Two buffers each,
  // as separate arrays: the compiler then knows that a load into one does not touch the other.
  constexpr bool SW8 = CPR % 8 == 0;
  __shared__ __attribute__((aligned(1024))) bf16_t Ks0[PF_BN * D];
  __shared__ __attribute__((aligned(1024))) bf16_t Ks1[PF_BN * D];
  __shared__ __attribute__((aligned(1024))) bf16_t Vs0[PF_BN * D];
  __shared__ __attribute__((aligned(1024))) bf16_t Vs1[PF_BN * D];
  auto swz = [](int row) { return SW8 ? (row & 7) : ((row >> 1) & 3); };

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int ln = lane & 15, lg = lane >> 4;
  // Heads run along x, the fast index of the launch, so that workgroups started one after the
  // other land on the eight XCDs in turn; the heads are dealt out so that XCD c gets heads
  // c * Hq/8 .. (c+1) * Hq/8 - 1: the query heads of a kv head meet in one L2, which then holds
  // an eighth of the keys and values instead of all of them.
  const int head = (Hq % 8 == 0) ? (blockIdx.x % 8) * (Hq / 8) + blockIdx.x / 8 : blockIdx.x;
  const int group_at = blockIdx.y, n_groups = gridDim.y;
  // The work list is sorted, the blocks with the most keys first. The n_groups workgroups of a
  // head walk it as a snake: forwards in even rounds, backwards in odd ones, so that the
  // workgroup with the longest block of one round takes the shortest of the next.
  for (int round = 0;; ++round) {
  const int item = round * n_groups + ((round & 1) ? n_groups - 1 - group_at : group_at);
  if (item >= n_work) break;       // (and so is every later item of this workgroup)
  const int seq = work_seq[item];
  const int qoff = work_qoff[item];
  const int qs = q_start[seq];
  const int qlen = q_start[seq + 1] - qs;
  const int ctx = ctx_len[seq];
  const int cached = ctx - qlen;
  const int rows = min(PBM, qlen - qoff);
  if (rows <= 0) continue;
  const int kvh = head / (Hq / Hkv);
  const int32_t* bt = block_table + (size_t)seq * bt_stride;
  const int first_q = cached + qoff;

  // query rows of this lane: tile r covers rows 16*(RT*wave + r) .. +15 of the block
  int qpos[RT];
  bool row_ok[RT];
  Frag8 qf[RT][NDT];
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    const int my_row = 16 * (RT * wave + r) + ln;
    row_ok[r] = my_row < rows;
    const int qrow = row_ok[r] ? my_row : 0;       // rows past the end repeat row 0; never stored
    qpos[r] = first_q + qrow;
    const bf16_t* qp = q + (size_t)(qs + qoff + qrow) * q_stride + (size_t)head * D + 8 * lg;
#pragma unroll
    for (int kk = 0; kk < NDT; ++kk) qf[r][kk].u = *reinterpret_cast<const uint4*>(qp + 32 * kk);
  }
  const int wave_first_row = 16 * RT * wave;
  const bool wave_has_rows = wave_first_row < rows;
  const int wave_min_q = first_q + (wave_has_rows ? wave_first_row : 0);
  const int wave_max_q = first_q + min(rows, wave_first_row + 16 * RT) - 1;

  // The softmax denominator: o[r][2 NDT] is one more tile of the second product, whose
  // "values" are all one; it sums the probabilities as the product sees them (rounded to
  // bfloat16; float32 sums) and is rescaled with the numerators.
  f32x4_t o[RT][2 * NDT + 1];
  float m_run[RT];
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    m_run[r] = -INFINITY;
#pragma unroll
    for (int t = 0; t <= 2 * NDT; ++t) o[r][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }
  Frag8 ones;
#pragma unroll
  for (int j = 0; j < 8; ++j) ones.v[j] = (__bf16)1.0f;
  // the running maximum follows the scores only when they pass it by more than this (raw
  // units): until then exp2 of a score minus the maximum stays below 2^8, which float32 sums
  // and bfloat16 probabilities hold as well as values below 1, and nothing is rescaled
  const float lazy = 8.0f / scale_log2;

  const int k_end = min(ctx, first_q + rows);
  const int k_lo = window > 0 ? max(0, first_q - window + 1) : 0;
  const int k_begin = (k_lo / PF_BN) * PF_BN;
  const int n_tiles = (k_end - k_begin + PF_BN - 1) / PF_BN;

  // This thread's chunks of a tile. A wave's load instruction fills 64 consecutive 16-byte
  // slots of LDS, lane l the l-th; slot s holds row s / CPR, chunk (s % CPR) ^ swz(row).
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  int crow[NCH], ccol[NCH];
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int slot = 64 * (wave_u * NCH + i) + lane;
    crow[i] = slot / CPR;
    ccol[i] = ((slot - crow[i] * CPR) ^ swz(crow[i])) * 8;
  }
  const bf16_t* k_head = k_cache + (size_t)kvh * page_size * D;
  const bf16_t* v_head = v_cache + (size_t)kvh * page_size * D;

  int pg[NCH];                  // pages of the chunks' rows, read one tile ahead of the rows
  const uint32_t page_bytes = (uint32_t)Hkv * page_size * D * 2;     // < 4 GiB, checked by the host
  const int page_mask = page_size - 1;                                // page sizes are powers of two
  // a tile that lies wholly inside the keys this block sees needs no tests (uniform)
  auto whole = [&](int t) {
    const int k0 = k_begin + t * PF_BN;
    return t < n_tiles && k0 >= k_lo && k0 + PF_BN <= k_end;
  };
  auto load_pages = [&](int t) {
    const int k0 = k_begin + t * PF_BN;
    if (whole(t)) {
#pragma unroll
      for (int i = 0; i < NCH; ++i) pg[i] = bt[(k0 + crow[i]) >> page_shift];
    } else {
#pragma unroll
      for (int i = 0; i < NCH; ++i) {
        const int kp = k0 + crow[i];
        pg[i] = -1;
        if (t < n_tiles && kp >= k_lo && kp < k_end) pg[i] = bt[kp >> page_shift];
      }
    }
  };
  // global memory -> LDS without a register in between (global_load_lds_dwordx4): every lane
  // names its own 16 bytes of global memory, the wave's 64 chunks land side by side in LDS
  auto to_lds = [&](const bf16_t* base, uint64_t at, bf16_t* tile_lds, int i) {
    __builtin_amdgcn_global_load_lds(
        (const __attribute__((address_space(1))) void*)(reinterpret_cast<const char*>(base) + at),
        (__attribute__((address_space(3))) void*)(tile_lds + 512 * (wave_u * NCH + i)), 16, 0, 0);
  };
  auto fetch = [&](int t, bf16_t* Kb, bf16_t* Vb) {
    const int k0 = k_begin + t * PF_BN;
    if (whole(t)) {
#pragma unroll
      for (int i = 0; i < NCH; ++i) {
        const uint32_t in_page = (uint32_t)(((k0 + crow[i]) & page_mask) * D + ccol[i]) * 2;
        const uint64_t at = (uint64_t)(uint32_t)pg[i] * page_bytes + in_page;
        to_lds(k_head, at, Kb, i);
        to_lds(v_head, at, Vb, i);
      }
    } else {
#pragma unroll
      for (int i = 0; i < NCH; ++i) {
        if (pg[i] >= 0) {
          const uint32_t in_page = (uint32_t)(((k0 + crow[i]) & page_mask) * D + ccol[i]) * 2;
          const uint64_t at = (uint64_t)(uint32_t)pg[i] * page_bytes + in_page;
          to_lds(k_head, at, Kb, i);
          to_lds(v_head, at, Vb, i);
        } else {                                  // rows outside the keys read as zeros
          const int slot = 64 * (wave_u * NCH + i) + lane;
          *reinterpret_cast<uint4*>(Kb + 8 * slot) = make_uint4(0, 0, 0, 0);
          *reinterpret_cast<uint4*>(Vb + 8 * slot) = make_uint4(0, 0, 0, 0);
        }
      }
    }
  };
  // where this lane reads: the first product takes row 16 kt + ln, chunk 4 kk + lg; the second
  // points at row 32 half + 16 j + 4 lg + ln / 4, elements 16 dt + 4 (ln % 4) .. +3
  int k_at[NDT], v_at[2 * NDT];
  {
    const int sw = swz(ln);
#pragma unroll
    for (int kk = 0; kk < NDT; ++kk) k_at[kk] = ln * D + 8 * ((4 * kk + lg) ^ sw);
    const int vrow = 4 * lg + (ln >> 2);
    const int vsw = swz(vrow);
#pragma unroll
    for (int dt = 0; dt < 2 * NDT; ++dt)
      v_at[dt] = vrow * D + 8 * ((2 * dt + ((ln & 3) >> 1)) ^ vsw) + 4 * (ln & 1);
  }

  // one key tile for this wave's rows; MASKED: the tile touches the diagonal, the end of the
  // keys or a window's edge
  auto tile = [&](int k0, const bf16_t* Kb, const bf16_t* Vb, auto masked_tag) {
    constexpr bool MASKED = decltype(masked_tag)::value;
    f32x4_t st[RT][4];
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
#pragma unroll
      for (int r = 0; r < RT; ++r) st[r][kt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < NDT; ++kk) {
        Frag8 a;
        a.u = *reinterpret_cast<const uint4*>(Kb + 16 * kt * D + k_at[kk]);
#pragma unroll
        for (int r = 0; r < RT; ++r)
          st[r][kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, qf[r][kk].v, st[r][kt], 0, 0, 0);
      }
    }
    Frag8 pb[RT][2];
#pragma unroll
    for (int r = 0; r < RT; ++r) {
      if (MASKED) {
#pragma unroll
        for (int kt = 0; kt < 4; ++kt)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int key = k0 + 16 * kt + 4 * lg + i;
            const bool vis = key <= qpos[r] && key < k_end && (window <= 0 || key > qpos[r] - window);
            st[r][kt][i] = vis ? st[r][kt][i] : -INFINITY;
          }
      }
      // the running max is kept in units of the raw scores; scale * log2(e) enters in the
      // exponent's multiply-add
      float tm[4];
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
        tm[kt] = max2(max2(st[r][kt][0], st[r][kt][1]), max2(st[r][kt][2], st[r][kt][3]));
      float tmax = max2(max2(tm[0], tm[1]), max2(tm[2], tm[3]));
      tmax = max_with_lane_xor16(tmax);
      tmax = max_with_lane_xor32(tmax);
      // the maximum moved far enough for this lane's row: rescale what is kept. (A branch per
      // lane, not per wave: the lanes that skip it keep their registers, so nothing is copied
      // where it joins.)
      if (tmax > m_run[r] + lazy) {
        const float alpha = __builtin_amdgcn_exp2f((m_run[r] - tmax) * scale_log2);
        m_run[r] = tmax;
#pragma unroll
        for (int t = 0; t <= 2 * NDT; ++t) {
          o[r][t][0] *= alpha; o[r][t][1] *= alpha; o[r][t][2] *= alpha; o[r][t][3] *= alpha;
        }
      }
      // (a row that has seen no key yet and sees none in this tile: all its scores are -inf)
      const float mc = (MASKED && m_run[r] == -INFINITY) ? 0.f : -m_run[r] * scale_log2;
#pragma unroll
      for (int half = 0; half < 2; ++half)
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float p = __builtin_amdgcn_exp2f(fmaf(st[r][2 * half + t][i], scale_log2, mc));
            pb[r][half].v[4 * t + i] = (__bf16)p;
          }
    }
    // V^T fragments: lane (ln, lg) points at V[key0 + ln/4][16 dt + 4 (ln%4)] and receives
    // V[key0 + 0..3][16 dt + ln], key0 = 32 half + 16 t + 4 lg: the keys of P^T's element 4 t + i
#pragma unroll
    for (int half = 0; half < 2; ++half)
#pragma unroll
      for (int dt = 0; dt < 2 * NDT; ++dt) {
        Frag8 a;
        a.s[0] = lds_read_tr16(Vb + (32 * half) * D + v_at[dt]);
        a.s[1] = lds_read_tr16(Vb + (32 * half + 16) * D + v_at[dt]);
#pragma unroll
        for (int r = 0; r < RT; ++r)
          o[r][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, pb[r][half].v, o[r][dt], 0, 0, 0);
      }
#pragma unroll
    for (int half = 0; half < 2; ++half)
#pragma unroll
      for (int r = 0; r < RT; ++r)
        o[r][2 * NDT] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones.v, pb[r][half].v, o[r][2 * NDT], 0, 0, 0);
  };

  // one turn: tile t + 1 sets out for the other buffer (everyone left it before the last
  // barrier), tile t is used, and what was loaded is waited for before the barrier
  auto turn = [&](int t, bf16_t* Kb, bf16_t* Vb, bf16_t* Kn, bf16_t* Vn) {
    const int k0 = k_begin + t * PF_BN;
    if (t + 1 < n_tiles) {
      fetch(t + 1, Kn, Vn);
      load_pages(t + 2);
    }
    // a wave whose rows all lie before this tile has nothing to do in it
    if (wave_has_rows && k0 <= wave_max_q) {
      const bool need_mask = (k0 + PF_BN - 1 > wave_min_q) || (k0 + PF_BN > k_end) || window > 0;
      if (need_mask)
        tile(k0, Kb, Vb, std::true_type{});
      else
        tile(k0, Kb, Vb, std::false_type{});
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);      // vmcnt(0): this wave's loads into LDS have landed
    __syncthreads();
  };
  load_pages(0);
  fetch(0, Ks0, Vs0);
  load_pages(1);
  __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();
  for (int t = 0; t < n_tiles; t += 2) {
    turn(t, Ks0, Vs0, Ks1, Vs1);
    if (t + 1 < n_tiles) turn(t + 1, Ks1, Vs1, Ks0, Vs0);
  }

#pragma unroll
  for (int r = 0; r < RT; ++r) {
    const float l = o[r][2 * NDT][0];          // every row of that tile holds the column's sum
    if (row_ok[r]) {
      const float inv = l > 0.f ? 1.0f / l : 0.f;
      const int my_row = 16 * (RT * wave + r) + ln;
      bf16_t* op = out + (size_t)(qs + qoff + my_row) * out_stride + (size_t)head * D + 4 * lg;
#pragma unroll
      for (int dt = 0; dt < 2 * NDT; ++dt) {
        union { uint2 u; bf16_t e[4]; } rr;
#pragma unroll
        for (int i = 0; i < 4; ++i) rr.e[i] = float_to_bf16(o[r][dt][i] * inv);
        *reinterpret_cast<uint2*>(op + 16 * dt) = rr.u;
      }
    }
  }
  }   // work items
}

template <int NDT, int RT>
static int launch_prefill_mfma(void* out, long out_stride, const void* q, long q_stride,
                               const void* k_cache, const void* v_cache, const int32_t* q_start,
                               const int32_t* ctx_len, const int32_t* block_table, int bt_stride,
                               const int32_t* work_seq, const int32_t* work_qoff, int n_work,
                               int n_groups, int Hq, int Hkv, int page_size, int window, float scale,
                               hipStream_t stream) {
  dim3 grid(Hq, n_groups < 65535 ? n_groups : 65535);
  int page_shift = -1;
  for (int sh = 0; sh < 31; ++sh)
    if ((1 << sh) == page_size) page_shift = sh;
  attn_prefill_mfma_kernel<NDT, RT><<<grid, 256, 0, stream>>>(
      (bf16_t*)out, out_stride, (const bf16_t*)q, q_stride, (const bf16_t*)k_cache,
      (const bf16_t*)v_cache, q_start, ctx_len, block_table, bt_stride, work_seq, work_qoff,
      n_work, Hq, Hkv, page_size, page_shift, window, scale * 1.4426950408889634f);
  return ptl_launch_status();
}

// work_seq / work_qoff list query blocks of ``block_rows`` rows (64 or 128), the longest first;
// n_groups workgroups a head share them (1 <= n_groups <= n_work). bfloat16 only;
// q rows must be 16-byte aligned and output rows 8-byte (q_stride % 8, out_stride % 4); the
// page size is a power of two and a page of all kv heads is smaller than 4 GiB.
extern "C" int ptl_attention_prefill_mfma(void* out, long out_stride, const void* q, long q_stride,
                                          const void* k_cache, const void* v_cache,
                                          const int32_t* q_start, const int32_t* ctx_len,
                                          const int32_t* block_table, int bt_stride,
                                          const int32_t* work_seq, const int32_t* work_qoff,
                                          int n_work, int n_groups, int block_rows, int Hq,
                                          int Hkv, int D,
                                          int page_size, int window, float scale,
                                          hipStream_t stream) {
  if (n_work <= 0) return PTL_OK;
  if (Hq <= 0 || Hkv <= 0 || Hq % Hkv || D % 32 || D <= 0 || D > 128 || page_size <= 0 ||
      (page_size & (page_size - 1)) || (long)Hkv * page_size * D * 2 >= (1L << 32) ||
      Hq > 65535 || n_groups < 1 || n_groups > n_work || q_stride % 8 || out_stride % 4 ||
      (block_rows != 64 && block_rows != 128))
    return PTL_ERR_ARG;
#define GO(N, R) launch_prefill_mfma<N, R>(out, out_stride, q, q_stride, k_cache, v_cache, q_start, \
                                           ctx_len, block_table, bt_stride, work_seq, work_qoff,  \
                                           n_work, n_groups, Hq, Hkv, page_size, window, scale, stream)
  if (block_rows == 64) {
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
