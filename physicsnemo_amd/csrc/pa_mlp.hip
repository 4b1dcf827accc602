// Fused block MLP on gfx950 MFMA:  y = W2 . gelu(W1 . u + b1) + b2  [+ residual]  [-> LayerNorm(y)]
// for bf16 rows u (M x C), hidden width F, C in {128, 256}, F a multiple of 64.
// Replaces the reference's `ln_mlp1[1](ln) + fx` (physicsnemo/models/transolver/transolver.py:301-303; Mlp:
// physicsnemo/nn/module/mlp_layers.py:139-173, GELU = exact erf form, activations.py:188-243) and hands the
// LayerNorm of the result to the next consumer (next block's ln_1 or the output head's LayerNorm).
//
// One workgroup of 4 waves per CU, one wave per SIMD (512 registers per lane); wave w owns 64 rows of a block of
// 256 rows:
//   * its rows of u stay in registers as B operands for the whole block (lane <-> row, k <-> channel);
//   * the weights stream through LDS in chunks of 64 hidden units, fetched with direct global -> LDS loads one chunk
//     ahead (two buffers, one barrier per chunk); every weight fragment read from LDS feeds two MFMAs (the wave's two
//     32-row halves), which keeps LDS at half its bandwidth;
//   * h^T (64 hidden x rows) = W1_chunk . u^T comes out with lanes <-> rows and registers <-> hidden units, so
//     gelu(h) rounded to bf16 is directly the B operand of  y^T (C x rows) += W2_chunk . gelu(h)^T;
//   * the y^T accumulators of all C channels (2 * C/32 * 16 = 256 registers for C = 256) live in the accumulation
//     registers for the whole block;
//   * epilogue: y^T -> bf16 -> this wave's share of the idle weight buffer (granule-swizzled transpose) -> row-major
//     rows: + residual, LayerNorm statistics by DPP reductions, full-row coalesced stores.
#include "pa_common.h"
#include "pa_host.h"
#include "pa_mfma_ops.h"

#include <type_traits>

namespace pa {
namespace mlp {

using namespace pa::mfma;

constexpr int kRowsPerBlock = 256;  // 4 waves x 64 rows

// 16-byte units of one weight chunk: W1 fragments [n 2][ks C/16][lane], then W2 fragments [ct C/32][k4 4][lane]
__host__ __device__ constexpr int chunk_units(int C) { return (2 * (C / 16) + (C / 32) * 4) * 64; }

// W1 (F x C) and W2 (C x F), bf16 row-major -> fragment order, chunk after chunk.
//   W1 fragment (n, ks): lane (i, g) holds W1[64c + 32n + i][16ks + 8g + j]
//   W2 fragment (ct, k4 = 2n + kk): lane (i, g) holds W2[32ct + i][64c + 32n + kperm(kk, g, j)]
__global__ __launch_bounds__(256) void pack_kernel(const uint16_t *__restrict__ w1, const uint16_t *__restrict__ w2,
                                                   u32x4 *__restrict__ blob, int C, int F) {
  const int KS = C / 16, NF1 = 2 * KS, CU = chunk_units(C);
  const int64_t total = (int64_t)(F / 64) * CU;
  for (int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x; u < total; u += (int64_t)gridDim.x * 256) {
    const int c = (int)(u / CU), r = (int)(u - (int64_t)c * CU), frag = r >> 6, lane = r & 63, i = lane & 31, g = lane >> 5;
    uint16_t e[8];
    if (frag < NF1) {
      const int n = frag / KS, ks = frag - n * KS;
      const uint16_t *src = w1 + (int64_t)(64 * c + 32 * n + i) * C + 16 * ks + 8 * g;
#pragma unroll
      for (int j = 0; j < 8; ++j) e[j] = src[j];
    } else {
      const int q = frag - NF1, ct = q >> 2, k4 = q & 3, n = k4 >> 1, kk = k4 & 1;
      const uint16_t *src = w2 + (int64_t)(32 * ct + i) * F + 64 * c + 32 * n;
#pragma unroll
      for (int j = 0; j < 8; ++j) e[j] = src[kperm(kk, g, j)];
    }
    u32x4 v;
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = (uint32_t)e[2 * j] | ((uint32_t)e[2 * j + 1] << 16);
    blob[u] = v;
  }
}

// 64 x 16 bytes, one per lane, from global memory straight into LDS at lds_wave_base + lane (no registers).
// The load is asynchronous and counted by vmcnt; its data must not be read before a wait and a barrier.
__device__ __forceinline__ void load_to_lds(const u32x4 *gsrc_lane, u32x4 *lds_wave_base) {
  const unsigned lds = __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)lds_wave_base);
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds), "v"(gsrc_lane) : "memory");
}

// exact-erf GELU; erf by Abramowitz-Stegun 7.1.26 (|error| < 2e-7 in fp32)
__device__ __forceinline__ float gelu_erf(float x) {
  const float z = x * 0.70710678118654752f, a = fabsf(z);
  const float t = __builtin_amdgcn_rcpf(fmaf(0.3275911f, a, 1.f));
  float p = fmaf(1.061405429f, t, -1.453152027f);
  p = fmaf(p, t, 1.421413741f);
  p = fmaf(p, t, -0.284496736f);
  p = fmaf(p, t, 0.254829592f);
  p *= t;
  const float e = __builtin_amdgcn_exp2f(a * a * -kLog2e);
  const float er = copysignf(fmaf(-p, e, 1.f), z);
  const float hx = 0.5f * x;
  return fmaf(hx, er, hx);
}

// sum over the 64 lanes, returned in every lane: DPP steps inside each row of 16, then the four row totals
__device__ __forceinline__ float wave_sum_dpp(float v) {
  auto step = [](float x, auto ctrl) {
    constexpr int c = decltype(ctrl)::value;
    return x + __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(x), c, 0xf, 0xf, true));
  };
  v = step(v, std::integral_constant<int, 0xB1>{});   // quad_perm [1,0,3,2]
  v = step(v, std::integral_constant<int, 0x4E>{});   // quad_perm [2,3,0,1]
  v = step(v, std::integral_constant<int, 0x141>{});  // row_half_mirror
  v = step(v, std::integral_constant<int, 0x140>{});  // row_mirror
  auto row_total = [&](int l) { return __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(v), l)); };
  return (row_total(0) + row_total(16)) + (row_total(32) + row_total(48));
}

template <int C, int TAIL>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void mlp_kernel(
    const u32x4 *__restrict__ blob, const float *__restrict__ b1, const float *__restrict__ b2,
    const uint16_t *__restrict__ u, uint16_t *__restrict__ y, const uint16_t *__restrict__ residual,
    const float *__restrict__ ln_gamma, const float *__restrict__ ln_beta, float ln_eps, uint16_t *__restrict__ ln_out,
    int64_t M, int F, int64_t nblocks) {
  constexpr bool HAS_RES = TAIL == 1 || TAIL == 2, HAS_LN = TAIL == 1 || TAIL == 3;
  constexpr int KS = C / 16, CT = C / 32, NF1 = 2 * KS, CU = chunk_units(C);
  constexpr int WU = CU / 4;     // units of a chunk fetched by each wave = its staging share in the epilogue
  constexpr int NDMA = WU / 64;  // direct-to-LDS loads per wave and chunk
  constexpr int CPL = C / 64;    // consecutive channels per lane in the row-major epilogue
  constexpr int G4 = C / 4;      // 8-byte granules (4 channels) per staged row
  static_assert(WU * 16 == 32 * C * 2, "a wave's share of a chunk buffer must hold 32 bf16 rows");
  extern __shared__ u32x4 smem[];
  u32x4 *wbuf = smem;  // 2 * CU
  float *b1s = reinterpret_cast<float *>(smem + 2 * CU);
  float *b2s = b1s + F;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, i = lane & 31, g = lane >> 5;
  const int NC = F / 64;

  for (int k = tid; k < F; k += 256) b1s[k] = b1[k];
  for (int k = tid; k < C; k += 256) b2s[k] = b2[k];
  float gam[CPL], bet[CPL];
#pragma unroll
  for (int k = 0; k < CPL; ++k) {
    gam[k] = HAS_LN ? ln_gamma[lane * CPL + k] : 1.f;
    bet[k] = HAS_LN ? ln_beta[lane * CPL + k] : 0.f;
  }

  auto fetch_chunk = [&](int64_t gc, int c) {  // this wave's share of chunk c into buffer gc & 1
    const u32x4 *src = blob + (int64_t)c * CU + wave * WU + lane;
    u32x4 *dst = wbuf + (gc & 1) * CU + wave * WU;
#pragma unroll
    for (int q = 0; q < NDMA; ++q) load_to_lds(src + q * 64, dst + q * 64);
  };

  int64_t gc = 0;  // chunks processed so far by this workgroup (buffer parity)
  if ((int64_t)blockIdx.x < nblocks) fetch_chunk(0, 0);
  for (int64_t mb = blockIdx.x; mb < nblocks; mb += gridDim.x) {
    // this wave's rows as B operands: lane (i, g) holds row 32m + i, channels 16ks + 8g .. + 7
    const int64_t row0 = mb * kRowsPerBlock + wave * 64;
    u32x4 ub[2][KS];
#pragma unroll
    for (int m = 0; m < 2; ++m) {
      int64_t r = row0 + 32 * m + i;
      if (r >= M) r = M - 1;
      const uint16_t *src = u + r * C + 8 * g;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) ub[m][ks] = *reinterpret_cast<const u32x4 *>(src + 16 * ks);
    }
    f32x16 yacc[2][CT];
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
      for (int ct = 0; ct < CT; ++ct)
#pragma unroll
        for (int r = 0; r < 16; ++r) yacc[m][ct][r] = 0.f;

    for (int c = 0; c < NC; ++c, ++gc) {
      // chunk gc has landed (every wave waits for its own share, then all meet); the other buffer is free
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      if (c + 1 < NC) fetch_chunk(gc + 1, c + 1);
      else if (mb + gridDim.x < nblocks) fetch_chunk(gc + 1, 0);
      const u32x4 *wb = wbuf + (gc & 1) * CU + lane;

      // h^T = W1_chunk . u^T + b1: two tiles of 32 hidden units for each of the two row halves
      f32x16 hacc[2][2];
#pragma unroll
      for (int n = 0; n < 2; ++n)
#pragma unroll
        for (int r = 0; r < 16; ++r) hacc[0][n][r] = hacc[1][n][r] = b1s[64 * c + 32 * n + rowmap(r, g)];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int n = 0; n < 2; ++n) {
          const u32x4 a = wb[(n * KS + ks) * 64];
          hacc[0][n] = mma(a, ub[0][ks], hacc[0][n]);
          hacc[1][n] = mma(a, ub[1][ks], hacc[1][n]);
        }
      // gelu, rounded to bf16: B operands of the second product (k4 = 2n + kk)
      u32x4 hb[2][4];
#pragma unroll
      for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int n = 0; n < 2; ++n) {
#pragma unroll
          for (int r = 0; r < 16; ++r) hacc[m][n][r] = gelu_erf(hacc[m][n][r]);
          hb[m][2 * n] = pack_half<0>(hacc[m][n]);
          hb[m][2 * n + 1] = pack_half<1>(hacc[m][n]);
        }
      // y^T += W2_chunk . gelu(h)^T
#pragma unroll
      for (int k4 = 0; k4 < 4; ++k4)
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
          const u32x4 a = wb[(NF1 + ct * 4 + k4) * 64];
          yacc[0][ct] = mma(a, hb[0][k4], yacc[0][ct]);
          yacc[1][ct] = mma(a, hb[1][k4], yacc[1][ct]);
        }
    }

    // ---- epilogue: the buffer of the last chunk is idle once every wave is past its last MFMA ----
    __syncthreads();
    uint32_t *stg = reinterpret_cast<uint32_t *>(wbuf + ((gc - 1) & 1) * CU + wave * WU);  // [32 rows][C/2 words]
#pragma unroll
    for (int m = 0; m < 2; ++m) {
      // y^T + b2 -> bf16 -> staged rows; granule gr (4 channels) of row i sits at gr ^ ((2i) % G4)
#pragma unroll
      for (int ct = 0; ct < CT; ++ct)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int ch = 32 * ct + 8 * q + 4 * g;
          const float v0 = yacc[m][ct][4 * q + 0] + b2s[ch + 0], v1 = yacc[m][ct][4 * q + 1] + b2s[ch + 1];
          const float v2 = yacc[m][ct][4 * q + 2] + b2s[ch + 2], v3 = yacc[m][ct][4 * q + 3] + b2s[ch + 3];
          const int gr = (ch >> 2) ^ ((2 * i) & (G4 - 1));
          u32x2 pk;
          pk[0] = (uint32_t)to_bf16_bits(v0) | ((uint32_t)to_bf16_bits(v1) << 16);
          pk[1] = (uint32_t)to_bf16_bits(v2) | ((uint32_t)to_bf16_bits(v3) << 16);
          *reinterpret_cast<u32x2 *>(stg + i * (C / 2) + gr * 2) = pk;
        }
      __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup");  // staged rows are read back by other lanes of this wave
      __builtin_amdgcn_wave_barrier();
      // rows, 8 at a time: lane holds CPL consecutive channels
      constexpr int RB = 8;
#pragma unroll 1
      for (int rb = 0; rb < 32; rb += RB) {
        uint32_t rsd[RB][CPL / 2];
        if constexpr (HAS_RES) {
#pragma unroll
          for (int rr = 0; rr < RB; ++rr) {
            int64_t r = row0 + 32 * m + rb + rr;
            if (r >= M) r = M - 1;
#pragma unroll
            for (int w = 0; w < CPL / 2; ++w)
              rsd[rr][w] = *reinterpret_cast<const uint32_t *>(residual + r * C + lane * CPL + 2 * w);
          }
        }
#pragma unroll
        for (int rr = 0; rr < RB; ++rr) {
          const int row = rb + rr;
          const int64_t r = row0 + 32 * m + row;
          const bool ok = r < M;
          float v[CPL];
          uint32_t ob[CPL / 2];
#pragma unroll
          for (int w = 0; w < CPL / 2; ++w) {
            const int word = lane * (CPL / 2) + w;  // word of the row; granule = word / 2
            const uint32_t sv = stg[row * (C / 2) + ((((word >> 1) ^ ((2 * row) & (G4 - 1))) << 1) | (word & 1))];
            float t0 = bf16_bits_to_f32((uint16_t)(sv & 0xffffu)), t1 = bf16_bits_to_f32((uint16_t)(sv >> 16));
            if constexpr (HAS_RES) {  // the MLP output is a bf16 tensor; the sum is rounded again
              t0 += bf16_bits_to_f32((uint16_t)(rsd[rr][w] & 0xffffu));
              t1 += bf16_bits_to_f32((uint16_t)(rsd[rr][w] >> 16));
            }
            const uint16_t o0 = to_bf16_bits(t0), o1 = to_bf16_bits(t1);
            v[2 * w] = bf16_bits_to_f32(o0);
            v[2 * w + 1] = bf16_bits_to_f32(o1);
            ob[w] = (uint32_t)o0 | ((uint32_t)o1 << 16);
          }
          if (ok) {
#pragma unroll
            for (int w = 0; w < CPL / 2; ++w) *reinterpret_cast<uint32_t *>(y + r * C + lane * CPL + 2 * w) = ob[w];
          }
          if constexpr (HAS_LN) {
            float s1 = 0.f;
#pragma unroll
            for (int k = 0; k < CPL; ++k) s1 += v[k];
            const float mean = wave_sum_dpp(s1) * (1.f / C);
            float s2 = 0.f;
#pragma unroll
            for (int k = 0; k < CPL; ++k) {
              const float dl = v[k] - mean;
              s2 = fmaf(dl, dl, s2);
            }
            const float rstd = rsqrtf(wave_sum_dpp(s2) * (1.f / C) + ln_eps);
            if (ok) {
#pragma unroll
              for (int w = 0; w < CPL / 2; ++w) {
                const uint16_t l0 = to_bf16_bits((v[2 * w] - mean) * rstd * gam[2 * w] + bet[2 * w]);
                const uint16_t l1 = to_bf16_bits((v[2 * w + 1] - mean) * rstd * gam[2 * w + 1] + bet[2 * w + 1]);
                *reinterpret_cast<uint32_t *>(ln_out + r * C + lane * CPL + 2 * w) = (uint32_t)l0 | ((uint32_t)l1 << 16);
              }
            }
          }
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup");  // rows read before the other half overwrites the stage
      __builtin_amdgcn_wave_barrier();
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing may still be landing in LDS when the workgroup ends
}

// ---------------------------------------------------------------------------------------------------------------
bool supported(int dtype, int64_t rows, int64_t C, int64_t F) {
  return dtype == PA_BF16 && rows > 0 && (C == 128 || C == 256) && F >= 64 && F % 64 == 0 && F <= 8192;
}

int64_t blob_bytes(int64_t C, int64_t F) { return (F / 64) * (int64_t)chunk_units((int)C) * 16; }

static size_t lds_bytes(int C, int F) { return (size_t)2 * chunk_units(C) * 16 + (size_t)(F + C) * 4; }

int pack(int64_t C, int64_t F, const void *w1, const void *w2, void *blob, hipStream_t st) {
  const int64_t total = (F / 64) * (int64_t)chunk_units((int)C);
  const int grid = (int)((total + 255) / 256 < 1024 ? (total + 255) / 256 : 1024);
  hipLaunchKernelGGL(pack_kernel, dim3(grid), dim3(256), 0, st, static_cast<const uint16_t *>(w1),
                     static_cast<const uint16_t *>(w2), static_cast<u32x4 *>(blob), (int)C, (int)F);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? PA_OK : (int)e;
}

template <int C, int TAIL>
static int launch(int64_t rows, int F, const void *blob, const float *b1, const float *b2, const void *u, void *y,
                  const pa_block_tail *tail, int num_cu, hipStream_t st) {
  const size_t lds = lds_bytes(C, F);
  if (lds > kMaxLdsBytes) return PA_ERR_UNSUPPORTED;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(mlp_kernel<C, TAIL>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return (int)e;
  const int64_t nblocks = (rows + kRowsPerBlock - 1) / kRowsPerBlock;
  const int64_t grid = nblocks < num_cu ? nblocks : num_cu;
  hipLaunchKernelGGL((mlp_kernel<C, TAIL>), dim3((unsigned)grid), dim3(256), lds, st, static_cast<const u32x4 *>(blob),
                     b1, b2, static_cast<const uint16_t *>(u), static_cast<uint16_t *>(y),
                     tail ? static_cast<const uint16_t *>(tail->residual) : nullptr, tail ? tail->ln_gamma : nullptr,
                     tail ? tail->ln_beta : nullptr, tail ? tail->ln_eps : 0.f,
                     tail ? static_cast<uint16_t *>(tail->ln_out) : nullptr, rows, F, nblocks);
  e = hipGetLastError();
  return e == hipSuccess ? PA_OK : (int)e;
}

template <int C>
static int launch_c(int64_t rows, int F, const void *blob, const float *b1, const float *b2, const void *u, void *y,
                    const pa_block_tail *tail, int num_cu, hipStream_t st) {
  const bool res = tail && tail->residual, ln = tail && tail->ln_out;
  if (res && ln) return launch<C, 1>(rows, F, blob, b1, b2, u, y, tail, num_cu, st);
  if (res) return launch<C, 2>(rows, F, blob, b1, b2, u, y, tail, num_cu, st);
  if (ln) return launch<C, 3>(rows, F, blob, b1, b2, u, y, tail, num_cu, st);
  return launch<C, 0>(rows, F, blob, b1, b2, u, y, nullptr, num_cu, st);
}

int forward(int64_t rows, int64_t C, int64_t F, const void *blob, const float *b1, const float *b2, const void *u,
            void *y, const pa_block_tail *tail, int num_cu, hipStream_t st) {
  if (C == 256) return launch_c<256>(rows, (int)F, blob, b1, b2, u, y, tail, num_cu, st);
  if (C == 128) return launch_c<128>(rows, (int)F, blob, b1, b2, u, y, tail, num_cu, st);
  return PA_ERR_UNSUPPORTED;
}

}  // namespace mlp
}  // namespace pa
