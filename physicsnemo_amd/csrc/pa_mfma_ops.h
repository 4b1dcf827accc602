// MFMA operand types and small helpers shared by the bf16 kernels (v_mfma_f32_32x32x16_bf16, gfx950).
//
// Register layouts (lane = 32*g + i, i = lane % 32, g = lane / 32):
//   A operand (32 x 16): lane holds row i, k = 8g + j, j = 0..7.      B operand (16 x 32): column i, k = 8g + j.
//   C/D (32 x 32): lane holds column i; register r = 0..15 is row  rowmap(r, g) = 8*(r/4) + 4*g + r%4.
// A C/D tile converted to bf16 is directly a pair of A (or B) operands of a following MFMA whose reduction index is
// the C/D row index taken in the order kperm(kk, g, j), provided the other operand uses the same permutation.
#pragma once

#include "pa_common.h"

namespace pa {
namespace mfma {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ f32x16 mma(u32x4 a, u32x4 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

__device__ __forceinline__ int rowmap(int r, int g) { return 8 * (r >> 2) + 4 * g + (r & 3); }
__device__ __forceinline__ int kperm(int kk, int g, int j) { return 16 * kk + 8 * (j >> 2) + 4 * g + (j & 3); }

// registers 8*HALF .. 8*HALF+7 of an accumulator, scaled, as 8 bf16 (round to nearest even)
template <int HALF>
__device__ __forceinline__ u32x4 pack_half(const f32x16 &v, float scale = 1.f) {
  bf16x8 o;
#pragma unroll
  for (int j = 0; j < 8; ++j) o[j] = (__bf16)(v[8 * HALF + j] * scale);
  return __builtin_bit_cast(u32x4, o);
}

__device__ __forceinline__ uint16_t to_bf16_bits(float f) { return __builtin_bit_cast(uint16_t, (__bf16)f); }

// value of lane l combined with the value of lane l ^ 32, without a trip through LDS: v_permlane32_swap hands every
// lane the lower-half and the upper-half value of its column
__device__ __forceinline__ float half_max(float v) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float half_sum(float v) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// A 32 x 32 accumulator tile (lane (i, g) <-> point i, register r <-> channel rowmap(r, g)) to bf16 rows in natural
// layout: `row` points at channel 0 of this lane's point.  Registers 4q..4q+3 hold channels 8q + 4g .. + 3; swapping
// halves with lane ^ 32 gives each lane 8 consecutive channels (g = 0: 0-7 and 8-15, g = 1: 16-23 and 24-31), so a
// point's 64 bytes leave as four 16-byte stores.  `nch` = valid channels (32, or 16: the lower half only).
__device__ __forceinline__ void store_tile_natural(const f32x16 &v, uint16_t *row, int g, bool ok, int nch = 32) {
  uint32_t p[4][2];
#pragma unroll
  for (int q = 0; q < 4; ++q)
#pragma unroll
    for (int w = 0; w < 2; ++w)
      p[q][w] = (uint32_t)to_bf16_bits(v[4 * q + 2 * w]) | ((uint32_t)to_bf16_bits(v[4 * q + 2 * w + 1]) << 16);
  u32x4 s0, s1;
#pragma unroll
  for (int w = 0; w < 2; ++w) {
    // lower half-wave: (own piece 0, partner's piece 0); upper half-wave: (partner's piece 2, own piece 2)
    const auto a = __builtin_amdgcn_permlane32_swap(p[0][w], p[2][w], false, false);
    s0[w] = a[0];
    s0[2 + w] = a[1];
    const auto b = __builtin_amdgcn_permlane32_swap(p[1][w], p[3][w], false, false);
    s1[w] = b[0];
    s1[2 + w] = b[1];
  }
  if (ok && (g == 0 || nch > 16)) {
    *reinterpret_cast<u32x4 *>(row + 16 * g) = s0;
    *reinterpret_cast<u32x4 *>(row + 16 * g + 8) = s1;
  }
}

}  // namespace mfma
}  // namespace pa
