// Float32 products on the bf16 matrix cores: operand splitting and the small helpers shared by the float32 row kernels.
//
// A float32 value is cut into three bf16 pieces a = a1 + a2 + a3 (8 significant bits each, exact); a . b is taken as
// a1 b1 + a1 b2 + a2 b1 + a2 b2 + a1 b3 + a3 b1 with float32 accumulation: six v_mfma_f32_32x32x16_bf16 per 16 reduction
// indices (48 passes) where v_mfma_f32_32x32x2_f32 needs 128.  The dropped products are below 2^-23 |a b|.
#pragma once

#include <utility>

#include "pa_mfma_ops.h"

namespace pa {
namespace split {

using mfma::f32x16;
using mfma::u32x4;

// v = f1 + f2 + f3, each with at most 8 significant bits (exact: every difference below is representable)
__device__ __forceinline__ void split3(float v, uint32_t (&h)[3]) {
  const uint32_t u = __float_as_uint(v);
  const float r1 = v - __uint_as_float(u & 0xffff0000u);
  const uint32_t u1 = __float_as_uint(r1);
  const float r2 = r1 - __uint_as_float(u1 & 0xffff0000u);
  h[0] = u >> 16;
  h[1] = u1 >> 16;
  h[2] = __float_as_uint(r2) >> 16;
}

// 8 floats (an operand's k = 8 g .. 8 g + 7) as the three bf16 operands
__device__ __forceinline__ void split8(const float (&v)[8], u32x4 (&pl)[3]) {
  uint32_t h[8][3];
#pragma unroll
  for (int e = 0; e < 8; ++e) split3(v[e], h[e]);
#pragma unroll
  for (int p = 0; p < 3; ++p)
#pragma unroll
    for (int q = 0; q < 4; ++q) pl[p][q] = h[2 * q][p] | (h[2 * q + 1][p] << 16);
}

// 3 KB (1 KB per instruction) from src + 16 lane to LDS byte address lds + 16 lane; the instruction offset advances
// both addresses.  Asynchronous, counted by vmcnt; sbase and lds are wave-uniform.
__device__ __forceinline__ void load_3k_to_lds(const void *sbase, unsigned lane16, unsigned lds) {
  asm volatile(
      "s_mov_b32 m0, %2\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %1, %0\n\t"
      "global_load_lds_dwordx4 %1, %0 offset:1024\n\t"
      "global_load_lds_dwordx4 %1, %0 offset:2048" ::"s"(sbase),
      "v"(lane16), "s"(lds)
      : "memory");
}

// A float32 weight as A-operand fragments: units of 12 KB = one k-step (16 reduction indices) of 128 output rows,
// [tile 0..3][piece 0..2][lane].
constexpr int kUnit = 4 * 3 * 64;  // 16-byte elements of a unit

// One unit of a 128-row block of a float32 weight: thread `v` (0 .. 255) packs tile v / 64, lane v % 64 = (i, g):
// row 32 tile + i, reduction indices k0 + 8 g + j (natural) or k0 rounded down to 32 + mfma::kperm((k0 / 16) % 2, g, j).
__device__ __forceinline__ void pack_unit(const float *w, int64_t ld, int k0, bool permuted, u32x4 *unit, int v) {
  const int ot = v >> 6, lane = v & 63, i = lane & 31, g = lane >> 5;
  const float *row = w + (int64_t)(32 * ot + i) * ld;
  float e[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) e[j] = row[permuted ? (k0 & ~31) + mfma::kperm((k0 >> 4) & 1, g, j) : k0 + 8 * g + j];
  u32x4 pl[3];
  split8(e, pl);
#pragma unroll
  for (int p = 0; p < 3; ++p) unit[(ot * 3 + p) * 64 + lane] = pl[p];
}

template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F &&f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

__device__ __forceinline__ f32x16 mma32(float a, float b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

}  // namespace split
}  // namespace pa
