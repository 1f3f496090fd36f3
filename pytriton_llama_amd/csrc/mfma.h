// Register types of the matrix-core kernels.
//
// v_mfma_f32_16x16x32_bf16 (A [16 x 32] . B [32 x 16] -> C [16 x 16]): lane l holds, of A, the
// eight consecutive k-values 8*(l/16) .. +7 of row l % 16; of B, the same k-values of column
// l % 16; of C, rows 4*(l/16) + i (i = 0..3) of column l % 16.
#pragma once
#include <hip/hip_runtime.h>

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));

// eight bfloat16 of one lane: as loaded (16 bytes, or two halves) and as the MFMA takes them
union Frag8 {
  uint4 u;
  uint2 h[2];
  s16x4_t s[2];
  bf16x8_t v;
};

// The larger of x in this lane and in lane ^ 16 (lane ^ 32): gfx950 swaps the odd rows of 16 (32)
// lanes of one register with the even rows of another in one VALU instruction; with both
// registers holding x, one then holds the even rows' values everywhere and the other the odd
// rows'. A ds_bpermute for the same costs a trip through the LDS crossbar, some hundred cycles
// in the chain of every key tile.
__device__ __forceinline__ float max_with_lane_xor16(float x) {
  const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float max_with_lane_xor32(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
