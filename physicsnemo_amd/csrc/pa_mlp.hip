// Fused block MLP on gfx950 MFMA:  y = W2 . gelu(W1 . u + b1) + b2  [+ residual]  [-> LayerNorm(y)]
// for bf16 rows u (M x C), hidden width F, C in {128, 256}, F a multiple of 64.
// Replaces the reference's `ln_mlp1[1](ln) + fx` (physicsnemo/models/transolver/transolver.py:301-303; Mlp:
// physicsnemo/nn/module/mlp_layers.py:139-173, GELU = erf form, activations.py:188-243) and hands the
// LayerNorm of the result to the next consumer (next block's ln_1 or the output head's LayerNorm).
//
// One workgroup of 4 waves per CU, one wave per SIMD (256 vector + 256 accumulation registers per lane).  A block
// of 128 rows is shared by two pairs of waves; the waves (rg, p = 0 / 1) of a pair own the same 64 rows:
//   * the rows of u stay in registers as B operands for the whole block (lane <-> row, k <-> channel);
//   * the weights stream through LDS in slots of 64 hidden units, fetched with direct global -> LDS loads one slot
//     ahead (two buffers); every weight fragment read from LDS feeds two MFMAs (the two 32-row halves), which
//     keeps LDS at half its bandwidth;
//   * wave p computes hidden tile p (32 units) of the slot: h^T = W1_tile . u^T comes out with lanes <-> rows and
//     registers <-> hidden units, so gelu(h) rounded to bf16 is directly a B operand of the second product; the
//     partner's tile comes through LDS;
//   * wave p accumulates y^T (C/2 channels x 64 rows) += W2[channel half p, slot] . gelu(h)^T in accumulation
//     registers for the whole block.  The second product runs one slot behind the first, so the VALU work of the
//     activation of slot c is issued behind the MFMAs of the second product of slot c-1 (slot c of the packed
//     weights therefore holds W1 of hidden chunk c and W2 of hidden chunk c-1);
//   * epilogue: y^T -> bf16 -> the idle weight buffer (granule-swizzled transpose, both waves of a pair) ->
//     row-major rows: + residual, LayerNorm statistics by DPP reductions, full-row coalesced stores.
#include "pa_common.h"
#include "pa_host.h"
#include "pa_mfma_ops.h"

#include <type_traits>
#include <utility>

namespace pa {
namespace mlp {

using namespace pa::mfma;

constexpr int kRowsPerBlock = 128;  // 2 pairs of waves x 64 rows

// 16-byte units of one weight slot: W1 fragments [n 2][ks C/16][lane], then W2 fragments [ct C/32][k4 4][lane]
__host__ __device__ constexpr int slot_units(int C) { return (2 * (C / 16) + (C / 32) * 4) * 64; }

// W1 (F x C) and W2 (C x F), bf16 row-major -> fragment order, F/64 + 1 slots: slot c holds W1 of hidden chunk c
// (zeros in the last slot) and W2 of hidden chunk c - 1 (zeros in the first).
//   W1 fragment (n, ks): lane (i, g) holds W1[64c + 32n + i][16ks + 8g + j]
//   W2 fragment (ct, k4 = 2n + kk): lane (i, g) holds W2[32ct + i][64(c-1) + 32n + kperm(kk, g, j)]
__global__ __launch_bounds__(256) void pack_kernel(const uint16_t *__restrict__ w1, const uint16_t *__restrict__ w2,
                                                   u32x4 *__restrict__ blob, int C, int F) {
  const int KS = C / 16, NF1 = 2 * KS, SU = slot_units(C), NC = F / 64;
  const int64_t total = (int64_t)(NC + 1) * SU;
  for (int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x; u < total; u += (int64_t)gridDim.x * 256) {
    const int c = (int)(u / SU), r = (int)(u - (int64_t)c * SU), frag = r >> 6, lane = r & 63, i = lane & 31, g = lane >> 5;
    uint16_t e[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) e[j] = 0;
    if (frag < NF1) {
      if (c < NC) {
        const int n = frag / KS, ks = frag - n * KS;
        const uint16_t *src = w1 + (int64_t)(64 * c + 32 * n + i) * C + 16 * ks + 8 * g;
#pragma unroll
        for (int j = 0; j < 8; ++j) e[j] = src[j];
      }
    } else if (c > 0) {
      const int q = frag - NF1, ct = q >> 2, k4 = q & 3, n = k4 >> 1, kk = k4 & 1;
      const uint16_t *src = w2 + (int64_t)(32 * ct + i) * F + 64 * (c - 1) + 32 * n;
#pragma unroll
      for (int j = 0; j < 8; ++j) e[j] = src[kperm(kk, g, j)];
    }
    u32x4 v;
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = (uint32_t)e[2 * j] | ((uint32_t)e[2 * j + 1] << 16);
    blob[u] = v;
  }
}

// One direct global -> LDS load of 64 x 16 bytes (no registers): the wave's lanes read sbase + voff (voff = 16 * lane)
// and the data land at LDS byte address lds + 16 * lane.  sbase and lds are wave-uniform.  The load is asynchronous
// and counted by vmcnt; its data must not be read before a wait and a barrier.
__device__ __forceinline__ void load_to_lds(const void *sbase, unsigned voff, unsigned lds) {
  asm volatile(
      "s_mov_b32 m0, %2\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %1, %0" ::"s"(sbase),
      "v"(voff), "s"(lds)
      : "memory");
}

// f(integral_constant<int, 0>{}), ..., f(integral_constant<int, N - 1>{}): a loop whose index is a constant expression
template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F &&f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

__device__ __forceinline__ float gelu(float x) { return gelu_logistic(x); }

// 8 floats -> 8 bf16 (round to nearest even)
__device__ __forceinline__ u32x4 pack8(const float (&v)[8]) {
  bf16x8 o;
#pragma unroll
  for (int j = 0; j < 8; ++j) o[j] = (__bf16)v[j];
  return __builtin_bit_cast(u32x4, o);
}

// sum over the 32 lanes of this lane's half of the wave, returned in every lane of the half: DPP steps inside each
// row of 16 lanes, then v_permlane16_swap pairs the two rows of the half
__device__ __forceinline__ float half_wave_sum(float v) {
  auto step = [](float x, auto ctrl) {
    constexpr int c = decltype(ctrl)::value;
    return x + __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(x), c, 0xf, 0xf, true));
  };
  v = step(v, std::integral_constant<int, 0xB1>{});   // quad_perm [1,0,3,2]
  v = step(v, std::integral_constant<int, 0x4E>{});   // quad_perm [2,3,0,1]
  v = step(v, std::integral_constant<int, 0x141>{});  // row_half_mirror
  v = step(v, std::integral_constant<int, 0x140>{});  // row_mirror
  const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

template <int C, int TAIL>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void mlp_kernel(
    const u32x4 *__restrict__ blob, const float *__restrict__ b1, const float *__restrict__ b2,
    const uint16_t *__restrict__ u, uint16_t *__restrict__ y, const uint16_t *__restrict__ residual,
    const float *__restrict__ ln_gamma, const float *__restrict__ ln_beta, float ln_eps, uint16_t *__restrict__ ln_out,
    int64_t M, int F, int64_t nblocks) {
  constexpr bool HAS_RES = TAIL == 1 || TAIL == 2, HAS_LN = TAIL == 1 || TAIL == 3;
  constexpr int KS = C / 16, CT = C / 32, CTH = CT / 2, NF1 = 2 * KS, SU = slot_units(C);
  constexpr int WU = SU / 4;     // units of a slot fetched by each wave
  constexpr int NDMA = WU / 64;  // direct-to-LDS loads per wave and slot
  constexpr int CPH = C / 32;    // consecutive channels per lane in the row-major epilogue (half a wave per row)
  constexpr int WPH = CPH / 2;   // 32-bit words per lane and row
  constexpr int G4 = C / 4;      // 8-byte granules (4 channels) per staged row
  static_assert(SU * 16 == 128 * C * 2, "a slot buffer must hold the 128 bf16 rows of a block in the epilogue");
  extern __shared__ u32x4 smem[];
  u32x4 *wbuf = smem;            // 2 * SU
  u32x4 *xch = wbuf + 2 * SU;    // [wave 4][m 2][kk 2][lane]: gelu(h) tiles handed to the partner wave
  float *b1s = reinterpret_cast<float *>(xch + 4 * 4 * 64);
  float *b2s = b1s + F;
  const int tid = threadIdx.x, lane = tid & 63, i = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: addresses derived from it stay scalar
  const int rg = wave >> 1, p = wave & 1;
  const int NC = F / 64;

  for (int k = tid; k < F; k += 256) b1s[k] = b1[k];
  for (int k = tid; k < C; k += 256) b2s[k] = b2[k];
  const int half = lane >> 5;  // in the epilogue each half of the wave finishes one row per step
  float gam[CPH], bet[CPH];
#pragma unroll
  for (int k = 0; k < CPH; ++k) {
    gam[k] = HAS_LN ? ln_gamma[i * CPH + k] : 1.f;
    bet[k] = HAS_LN ? ln_beta[i * CPH + k] : 0.f;
  }

  static_assert(NDMA == KS, "one direct-to-LDS load per step of the first phase");
  // piece q of this wave's share of slot c into buffer gs & 1
  auto fetch_piece = [&](int64_t gs, int c, int q) {
    const u32x4 *src = blob + (int64_t)c * SU + wave * WU + q * 64;
    const unsigned dst = (unsigned)(uintptr_t)(wbuf + (gs & 1) * SU + wave * WU + q * 64);
    load_to_lds(src, lane * 16, dst);
  };
  auto load_rows = [&](int64_t mb, u32x4(&ub)[2][KS]) {  // the pair's rows of block mb as B operands
    const int64_t row0 = mb * kRowsPerBlock + rg * 64;
#pragma unroll
    for (int m = 0; m < 2; ++m) {
      int64_t r = row0 + 32 * m + i;
      if (r >= M) r = M - 1;
      const uint16_t *src = u + r * C + 8 * g;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) ub[m][ks] = *reinterpret_cast<const u32x4 *>(src + 16 * ks);
    }
  };

  int64_t gs = 0;  // slots processed so far by this workgroup (buffer parity)
  if ((int64_t)blockIdx.x < nblocks) {
#pragma unroll
    for (int q = 0; q < NDMA; ++q) fetch_piece(0, 0, q);
  }
  // lane (i, g) holds row 32m + i, channels 16ks + 8g .. + 7
  u32x4 ub[2][KS];
  if ((int64_t)blockIdx.x < nblocks) load_rows(blockIdx.x, ub);
  for (int64_t mb = blockIdx.x; mb < nblocks; mb += gridDim.x) {
    const int64_t row0 = mb * kRowsPerBlock + rg * 64;
    f32x16 yacc[2][CTH];  // channels 32 * (CTH * p + ct) + rowmap(r, g)
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
      for (int ct = 0; ct < CTH; ++ct)
#pragma unroll
        for (int r = 0; r < 16; ++r) yacc[m][ct][r] = 0.f;
    // gelu(h) of hidden chunk c-1 as B operands [m][kk]: this wave's tile and the partner's
    u32x4 hown[2][2], hpar[2][2];
    float hrest[2][8];  // second half (registers 8..15) of this wave's h tile of chunk c-1, before the activation
#pragma unroll
    for (int m = 0; m < 2; ++m) {
      hown[m][0] = u32x4{0, 0, 0, 0};
#pragma unroll
      for (int j = 0; j < 8; ++j) hrest[m][j] = 0.f;
    }

    for (int c = 0; c <= NC; ++c, ++gs) {
      // slot gs has landed (every wave waits for its own share, then all meet) and the other buffer is free.  The
      // first slot of a later block was waited for before the epilogue of the block before it, whose stores may
      // still be in flight here.
      if (c > 0 || gs == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      const bool has_next = c < NC || mb + gridDim.x < nblocks;
      const int c_next = c < NC ? c + 1 : 0;
      const u32x4 *wb = wbuf + (gs & 1) * SU + lane;
      // this wave's fragments of the slot: W1 of hidden tile p; W2 of its channel half, hidden tile p ("own") first
      const u32x4 *w1f = wb + p * KS * 64;
      const u32x4 *w2own = wb + (NF1 + p * CTH * 4 + 2 * p) * 64, *w2par = wb + (NF1 + p * CTH * 4 + 2 * (1 - p)) * 64;

      // One slot = 2 phases of KS resp. 4 * CTH steps; a step = one weight fragment (read from LDS AHEAD steps
      // early), two MFMAs and, behind them, one or two gelu evaluations:
      //   phase 1   h^T tile p of hidden chunk c += W1 fragment . u^T (both row halves);
      //             gelu of the second half of the tile of chunk c-1 -> the tile is complete, goes to the partner
      //   phase 2   y^T += W2 fragment(ct, k4) of hidden chunk c-1 . gelu(h)^T (own tile, then the partner's);
      //             gelu of the first half of the tile of chunk c
      constexpr int RING = 6, AHEAD = 5;
      f32x16 hacc[2];
#pragma unroll
      for (int r = 0; r < 16; ++r) hacc[0][r] = hacc[1][r] = b1s[(c < NC ? 64 * c : 0) + 32 * p + rowmap(r, g)];
      {
        constexpr int EV = 16 / KS > 0 ? 16 / KS : 1;  // evaluations per step (16 over KS steps)
        static_assert(KS * EV == 16 || KS == 16, "phase 1 must cover 16 evaluations");
        u32x4 fr[RING];
        static_for<AHEAD>([&](auto q) { fr[decltype(q)::value] = w1f[decltype(q)::value * 64]; });
        // the first fragments and the bias are on their way: now the next slot's fetch, whose issue keeps the wave
        // busy for a while (its buffer was last read in phase 2 of the slot before this one)
        if (has_next) {
#pragma unroll
          for (int q = 0; q < NDMA; ++q) fetch_piece(gs + 1, c_next, q);
        }
        static_for<KS>([&](auto st) {
          constexpr int step = decltype(st)::value;
          if constexpr (step + AHEAD < KS) fr[(step + AHEAD) % RING] = w1f[(step + AHEAD) * 64];
          const u32x4 a = fr[step % RING];
          hacc[0] = mma(a, ub[0][step], hacc[0]);
          hacc[1] = mma(a, ub[1][step], hacc[1]);
          static_for<(KS == 16 ? 1 : 16 / KS)>([&](auto q) {
            constexpr int E = step * (KS == 16 ? 1 : 16 / KS) + decltype(q)::value, m = E / 8, j = E % 8;
            hrest[m][j] = gelu(hrest[m][j]);
            if constexpr (j == 7) hown[m][1] = pack8(hrest[m]);
          });
          __builtin_amdgcn_sched_barrier(0);  // keeps the issue order as written
        });
      }
      // the tile of chunk c-1 is complete: hand it to the partner, take the partner's
#pragma unroll
      for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) xch[((wave * 2 + m) * 2 + kk) * 64 + lane] = hown[m][kk];
      {
        constexpr int NS2 = 4 * CTH, EV = 16 / NS2 > 0 ? 16 / NS2 : 1;
        static_assert(NS2 * EV == 16, "phase 2 must cover 16 evaluations");
        float fl[2][8];
        u32x4 hfirst[2];
        auto frag2 = [&](auto st) {  // step -> (k4' = step / CTH, ct = step % CTH); k4' < 2: own tile, kk = k4' % 2
          constexpr int t = decltype(st)::value, k4 = t / CTH, ct = t % CTH;
          return (k4 < 2 ? w2own : w2par)[(ct * 4 + (k4 & 1)) * 64];
        };
        u32x4 fr[RING];
        static_for<AHEAD>([&](auto q) { fr[decltype(q)::value] = frag2(q); });
        static_for<NS2>([&](auto st) {
          constexpr int t = decltype(st)::value, k4 = t / CTH, ct = t % CTH, kk = k4 & 1;
          if constexpr (t == 2 * CTH - 2) {  // two steps before the partner's tile (written before phase 2) is needed
            __syncthreads();
#pragma unroll
            for (int m = 0; m < 2; ++m)
#pragma unroll
              for (int k = 0; k < 2; ++k) hpar[m][k] = xch[(((wave ^ 1) * 2 + m) * 2 + k) * 64 + lane];
          }
          if constexpr (t + AHEAD < NS2) fr[(t + AHEAD) % RING] = frag2(std::integral_constant<int, t + AHEAD>{});
          const u32x4 a = fr[t % RING];
          yacc[0][ct] = mma(a, k4 < 2 ? hown[0][kk] : hpar[0][kk], yacc[0][ct]);
          yacc[1][ct] = mma(a, k4 < 2 ? hown[1][kk] : hpar[1][kk], yacc[1][ct]);
          static_for<EV>([&](auto q) {
            constexpr int E = t * EV + decltype(q)::value, m = E / 8, j = E % 8;
            fl[m][j] = gelu(hacc[m][j]);
            if constexpr (j == 7) hfirst[m] = pack8(fl[m]);
          });
          __builtin_amdgcn_sched_barrier(0);
        });
#pragma unroll
        for (int m = 0; m < 2; ++m) {
          hown[m][0] = hfirst[m];
#pragma unroll
          for (int j = 0; j < 8; ++j) hrest[m][j] = hacc[m][8 + j];
        }
      }
    }

    // ---- epilogue: the buffer of the last slot is idle once every wave is past its last MFMA ----
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's share of the next block's first slot has landed
    __syncthreads();
    // the rows of this workgroup's next block travel while the epilogue runs (past the end: this block again)
    load_rows(mb + gridDim.x < nblocks ? mb + gridDim.x : mb, ub);
    uint32_t *stg = reinterpret_cast<uint32_t *>(wbuf + ((gs - 1) & 1) * SU) + rg * 64 * (C / 2);  // [64 rows][C/2 words]
    // y^T + b2 -> bf16 -> staged rows; granule gr (4 channels) of row rw sits at gr ^ ((2 rw) % G4)
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
      for (int ct = 0; ct < CTH; ++ct)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int ch = 32 * (CTH * p + ct) + 8 * q + 4 * g, rw = 32 * m + i;
          const float v0 = yacc[m][ct][4 * q + 0] + b2s[ch + 0], v1 = yacc[m][ct][4 * q + 1] + b2s[ch + 1];
          const float v2 = yacc[m][ct][4 * q + 2] + b2s[ch + 2], v3 = yacc[m][ct][4 * q + 3] + b2s[ch + 3];
          const int gr = (ch >> 2) ^ ((2 * rw) & (G4 - 1));
          u32x2 pk;
          pk[0] = (uint32_t)to_bf16_bits(v0) | ((uint32_t)to_bf16_bits(v1) << 16);
          pk[1] = (uint32_t)to_bf16_bits(v2) | ((uint32_t)to_bf16_bits(v3) << 16);
          *reinterpret_cast<u32x2 *>(stg + rw * (C / 2) + gr * 2) = pk;
        }
    __syncthreads();  // both waves of a pair have staged their channel halves
    // wave p finishes rows 32p .. 32p+31 of the pair, two per step: lanes 0-31 one row, lanes 32-63 the next, CPH
    // consecutive channels per lane (16-byte accesses for C = 256)
    typedef uint32_t rowv __attribute__((ext_vector_type(WPH)));
    constexpr int NRS = 16;
    rowv rsd[NRS];
    if constexpr (HAS_RES) {
#pragma unroll
      for (int rr = 0; rr < NRS; ++rr) {
        int64_t r = row0 + 32 * p + 2 * rr + half;
        if (r >= M) r = M - 1;
        rsd[rr] = *reinterpret_cast<const rowv *>(residual + r * C + i * CPH);
      }
    }
#pragma unroll
    for (int rr = 0; rr < NRS; ++rr) {
      const int rw = 32 * p + 2 * rr + half;
      const int64_t r = row0 + rw;
      const bool ok = r < M;
      // granules (4 channels) i*CPH/4 .. of row rw; the swizzle flips an even number, so they stay adjacent
      const rowv sv = *reinterpret_cast<const rowv *>(stg + rw * (C / 2) + (((i * CPH / 4) ^ ((2 * rw) & (G4 - 1))) << 1));
      float v[CPH];
      rowv ob;
#pragma unroll
      for (int w = 0; w < WPH; ++w) {
        float t0 = bf16_bits_to_f32((uint16_t)(sv[w] & 0xffffu)), t1 = bf16_bits_to_f32((uint16_t)(sv[w] >> 16));
        if constexpr (HAS_RES) {  // the MLP output is a bf16 tensor; the sum is rounded again
          t0 += bf16_bits_to_f32((uint16_t)(rsd[rr][w] & 0xffffu));
          t1 += bf16_bits_to_f32((uint16_t)(rsd[rr][w] >> 16));
        }
        const uint16_t o0 = to_bf16_bits(t0), o1 = to_bf16_bits(t1);
        v[2 * w] = bf16_bits_to_f32(o0);
        v[2 * w + 1] = bf16_bits_to_f32(o1);
        ob[w] = (uint32_t)o0 | ((uint32_t)o1 << 16);
      }
      if (ok) *reinterpret_cast<rowv *>(y + r * C + i * CPH) = ob;
      if constexpr (HAS_LN) {
        float s1 = 0.f;
#pragma unroll
        for (int k = 0; k < CPH; ++k) s1 += v[k];
        const float mean = half_wave_sum(s1) * (1.f / C);
        float s2 = 0.f;
#pragma unroll
        for (int k = 0; k < CPH; ++k) {
          const float dl = v[k] - mean;
          s2 = fmaf(dl, dl, s2);
        }
        const float rstd = rsqrtf(half_wave_sum(s2) * (1.f / C) + ln_eps);
        rowv lb;
#pragma unroll
        for (int w = 0; w < WPH; ++w) {
          const uint16_t l0 = to_bf16_bits((v[2 * w] - mean) * rstd * gam[2 * w] + bet[2 * w]);
          const uint16_t l1 = to_bf16_bits((v[2 * w + 1] - mean) * rstd * gam[2 * w + 1] + bet[2 * w + 1]);
          lb[w] = (uint32_t)l0 | ((uint32_t)l1 << 16);
        }
        if (ok) *reinterpret_cast<rowv *>(ln_out + r * C + i * CPH) = lb;
      }
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing may still be landing in LDS when the workgroup ends
}

// ---------------------------------------------------------------------------------------------------------------
bool supported(int dtype, int64_t rows, int64_t C, int64_t F) {
  return dtype == PA_BF16 && rows > 0 && (C == 128 || C == 256) && F >= 64 && F % 64 == 0 && F <= 8192;
}

int64_t blob_bytes(int64_t C, int64_t F) { return (F / 64 + 1) * (int64_t)slot_units((int)C) * 16; }

static size_t lds_bytes(int C, int F) { return (size_t)(2 * slot_units(C) + 4 * 4 * 64) * 16 + (size_t)(F + C) * 4; }

int pack(int64_t C, int64_t F, const void *w1, const void *w2, void *blob, hipStream_t st) {
  const int64_t total = (F / 64 + 1) * (int64_t)slot_units((int)C);
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
