// Shared device helpers for the PhysicsAttention kernels (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/physattn.h"

namespace pa {

constexpr float kSliceNormEps = 1e-2f;  // PA.py:185
constexpr float kTempMin = 0.5f;        // PA.py:173
constexpr float kTempMax = 5.0f;
constexpr float kLog2e = 1.4426950408889634f;

// bf16 stored as raw 16 bits; conversions are round-to-nearest-even like torch's.
struct bf16 {
  uint16_t bits;
};

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }

__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);  // quiet NaN
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

__device__ __forceinline__ float load_as_f32(const float *p) { return *p; }
__device__ __forceinline__ float load_as_f32(const bf16 *p) { return bf16_bits_to_f32(p->bits); }
__device__ __forceinline__ void store_from_f32(float *p, float v) { *p = v; }
__device__ __forceinline__ void store_from_f32(bf16 *p, float v) { p->bits = f32_to_bf16_bits(v); }

// value after a round trip through the storage type (what a later kernel will read back)
__device__ __forceinline__ float round_to(const float *, float v) { return v; }
__device__ __forceinline__ float round_to(const bf16 *, float v) { return bf16_bits_to_f32(f32_to_bf16_bits(v)); }

// GELU in its erf form (torch.nn.GELU default, activations.py:198)
__device__ __forceinline__ float gelu_erf(float v) { return 0.5f * v * (1.f + erff(v * 0.70710678118654752f)); }

// GELU(x) = x * Phi(x) for the bf16 MFMA kernels, Phi in the logistic form 1 / (1 + exp(-2 x P(x^2))) with P fitted to
// the exact erf form: max |error| 2.6e-5 over all x (the plain tanh form has 4.7e-4); |x| is clamped where Phi is 0 or
// 1 in fp32.  Two transcendental instructions and five multiply-adds.
__device__ __forceinline__ float gelu_logistic(float x) {
  const float x2 = fminf(x * x, 81.f);  // beyond |x| = 9 Phi is 0 or 1 in fp32; keeps x P(x^2) monotone
  // -2 * log2(e) * (c0 + c1 x^2 + c2 x^4)
  float p = fmaf(-3.51902394e-04f * -2.f * kLog2e, x2, 3.70080200e-02f * -2.f * kLog2e);
  p = fmaf(p, x2, 7.97505275e-01f * -2.f * kLog2e);
  const float e = __builtin_amdgcn_exp2f(x * p);
  return x * __builtin_amdgcn_rcpf(1.f + e);
}

// its derivative: Phi(v) + v phi(v)
__device__ __forceinline__ float gelu_erf_grad(float v) {
  return 0.5f * (1.f + erff(v * 0.70710678118654752f)) + v * 0.3989422804014327f * expf(-0.5f * v * v);
}

// Accesses to tensors that a kernel streams through once (activations in, activations out, the packed slice
// weights): the non-temporal hint keeps them from displacing what the L2 is for -- weights, tables, partial sums --
// and measured 9 % off kernel (d) and 5 % off the layer.  Any trivially copyable vector type.
template <class T>
__device__ __forceinline__ T load_streaming(const T *p) {
  return __builtin_nontemporal_load(p);
}
template <class T>
__device__ __forceinline__ void store_streaming(T *p, T v) {
  __builtin_nontemporal_store(v, p);
}

// e4m3fn (OCP): 1 sign, 4 exponent (bias 7), 3 mantissa bits; exponent 0 is subnormal (2^-6 * m/8); 0x7f / 0xff are
// NaN; there are no infinities.
__device__ __forceinline__ float decode_e4m3fn(uint8_t v) {
  const int e = (v >> 3) & 15, m = v & 7;
  float mag;
  if (e == 15 && m == 7) mag = __uint_as_float(0x7fc00000u);
  else if (e == 0) mag = (float)m * 0.001953125f;                             // m/8 * 2^-6
  else mag = __uint_as_float((uint32_t)(e + 120) << 23 | (uint32_t)m << 20);  // 2^(e-7) * (1 + m/8)
  return (v & 0x80) ? -mag : mag;
}

// A large weight matrix as the repacking kernels read it: bf16 bits (scale == nullptr), or fp8-e4m3 bytes with one
// float32 scale per output row.  Element (row, col) as bf16 bits: the stored bits, or bf16(scale[row] * e4m3) rounded
// to nearest even -- the value an expansion to bf16 followed by an ordinary bf16 repack would have produced.
struct WeightView {
  const void *w;
  const float *scale;
  int64_t ld;  // elements per row
};
__device__ __forceinline__ uint16_t weight_bits(const WeightView &v, int64_t row, int64_t col) {
  const int64_t at = row * v.ld + col;
  if (!v.scale) return static_cast<const uint16_t *>(v.w)[at];
  return f32_to_bf16_bits(v.scale[row] * decode_e4m3fn(static_cast<const uint8_t *>(v.w)[at]));
}
// eight consecutive elements of a row (col a multiple of 8) as four packed pairs
__device__ __forceinline__ void weight_bits8(const WeightView &v, int64_t row, int64_t col, uint32_t out[4]) {
  const int64_t at = row * v.ld + col;
  if (!v.scale) {
    const uint4 q = *reinterpret_cast<const uint4 *>(static_cast<const uint16_t *>(v.w) + at);
    out[0] = q.x; out[1] = q.y; out[2] = q.z; out[3] = q.w;
    return;
  }
  const uint2 q = *reinterpret_cast<const uint2 *>(static_cast<const uint8_t *>(v.w) + at);
  const float sc = v.scale[row];
  const uint32_t b[2] = {q.x, q.y};
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const uint32_t lo = (b[k >> 1] >> (16 * (k & 1))) & 0xffu, hi = (b[k >> 1] >> (16 * (k & 1) + 8)) & 0xffu;
    out[k] = (uint32_t)f32_to_bf16_bits(sc * decode_e4m3fn((uint8_t)lo)) |
             ((uint32_t)f32_to_bf16_bits(sc * decode_e4m3fn((uint8_t)hi)) << 16);
  }
}

__device__ __forceinline__ float clamp_temperature(float t) { return fminf(fmaxf(t, kTempMin), kTempMax); }

// wave64 butterfly reductions
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace pa
