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

// ------------------------------------------------------------------------------------------------
// The slice weights of one head for one tile of 32 points, formed in registers: logits, temperature softmax, bf16
// operand chunks.  chunk[cq] (cq = 0 .. S/16 - 1) is what the slice-softmax kernels store: as an A operand its rows
// are the points and its reduction index the slices 16 cq + kperm order; the same registers serve as a B operand
// whose columns are the points.  The kernels that use this recompute the weights from x_mid instead of passing them through
// memory (S/16 KB per point and head group written once and read twice otherwise).  The token sums use
// bf16(e_s / sum e), the hand-back bf16(e_s) divided by the sum of those rounded values: the same softmax, each rounded
// once.
// ------------------------------------------------------------------------------------------------
// DEFER: the chunks hold bf16(exp2(..)) without the division by their sum; the caller divides what it forms from them
// by the sum of the same rounded values (one more MFMA column), which saves a pass over the S values per point.
template <int S, bool DEFER = false>
__device__ __forceinline__ void slice_weights_of_tile(const u32x4 *__restrict__ wsl, const float *__restrict__ bsl,
                                                      u32x4 xm0, u32x4 xm1, float sc, bool valid, int lane, int g,
                                                      u32x4 (&chunk)[S / 16]) {
  constexpr int ST = (S + 31) / 32, NCH = S / 16;
  f32x16 lg[ST];
#pragma unroll
  for (int st = 0; st < ST; ++st) {
#pragma unroll
    for (int r = 0; r < 16; ++r) lg[st][r] = bsl[32 * st + rowmap(r, g)];
    lg[st] = mma(wsl[(st * 2 + 0) * 64 + lane], xm0, lg[st]);
    lg[st] = mma(wsl[(st * 2 + 1) * 64 + lane], xm1, lg[st]);
  }
  float mx = -INFINITY;
#pragma unroll
  for (int st = 0; st < ST; ++st)
#pragma unroll
    for (int r = 0; r < 16; ++r) mx = fmaxf(mx, lg[st][r]);
  mx = half_max(mx);
  const float off = mx * sc;
  if constexpr (DEFER) {
#pragma unroll
    for (int st = 0; st < ST; ++st)
#pragma unroll
      for (int r = 0; r < 16; ++r) lg[st][r] = __builtin_amdgcn_exp2f(fmaf(lg[st][r], sc, -off));
#pragma unroll
    for (int cq = 0; cq < NCH; ++cq) chunk[cq] = (cq & 1) ? pack_half<1>(lg[cq >> 1]) : pack_half<0>(lg[cq >> 1]);
  } else {
    float sum = 0.f;
#pragma unroll
    for (int st = 0; st < ST; ++st)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float e = __builtin_amdgcn_exp2f(fmaf(lg[st][r], sc, -off));
        lg[st][r] = e;
        sum += e;
      }
    sum = half_sum(sum);
    const float inv = valid ? __builtin_amdgcn_rcpf(sum) : 0.f;
#pragma unroll
    for (int cq = 0; cq < NCH; ++cq) chunk[cq] = (cq & 1) ? pack_half<1>(lg[cq >> 1], inv) : pack_half<0>(lg[cq >> 1], inv);
  }
}

// W_slice as A operands and the slice bias in LDS, as slice_weights_of_tile reads them; the reduction index runs over
// d in natural order (x_mid read from its rows) or in kperm order (PACKED_X: x_mid read as packed operand tiles)
template <int S, bool PACKED_X>
__device__ __forceinline__ void stage_slice_projection(const float *__restrict__ w_slice, const float *__restrict__ b_slice,
                                                       u32x4 *wsl, float *bsl) {
  constexpr int ST = (S + 31) / 32;
  for (int u = threadIdx.x; u < ST * 2 * 64; u += blockDim.x) {
    const int ul = u & 63, ui = ul & 31, ug = ul >> 5, f = u >> 6, st = f >> 1, kk = f & 1;
    const int s = 32 * st + ui;
    bf16x8 e;
#pragma unroll
    for (int j = 0; j < 8; ++j)
      e[j] = (__bf16)(s < S ? w_slice[s * 32 + (PACKED_X ? kperm(kk, ug, j) : 16 * kk + 8 * ug + j)] : 0.f);
    wsl[u] = __builtin_bit_cast(u32x4, e);
  }
  for (int s = threadIdx.x; s < ST * 32; s += blockDim.x) bsl[s] = s < S ? b_slice[s] : -1e30f;  // slices beyond S: weight 0
}

}  // namespace mfma
}  // namespace pa
