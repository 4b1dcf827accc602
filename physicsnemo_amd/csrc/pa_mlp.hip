// Fused block MLP on gfx950 MFMA:  y = W2 . gelu(W1 . u + b1) + b2  [+ residual]  [-> LayerNorm(y)]
// for bf16 rows u (M x C), hidden width F (a multiple of 64).
// Replaces the reference's `ln_mlp1[1](ln) + fx` (physicsnemo/models/transolver/transolver.py:301-303; Mlp:
// physicsnemo/nn/module/mlp_layers.py:139-173, GELU = erf form, activations.py:188-243) and hands the
// LayerNorm of the result to the next consumer (next block's ln_1 or the output head's LayerNorm).
//
// Three tilings, chosen by C (namespace rows holds the two in which a wave owns its rows outright, together with the
// row GEMMs of the 512-wide layer built on the same skeleton):
//   C = 128   mlp_kernel        pairs of waves share 64 rows and split hidden tiles and output channels (below)
//   C = 256   mlp_rows2_kernel  32 rows per wave, two waves per SIMD
//   C = 512   mlp_rows_kernel   32 rows per wave, one wave per SIMD, the two products interleaved
//
// mlp_kernel:
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
__global__ __launch_bounds__(256) void pack_kernel(WeightView w1, WeightView w2, u32x4 *__restrict__ blob, int C, int F) {
  const int KS = C / 16, NF1 = 2 * KS, SU = slot_units(C), NC = F / 64;
  const int64_t total = (int64_t)(NC + 1) * SU;
  for (int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x; u < total; u += (int64_t)gridDim.x * 256) {
    const int c = (int)(u / SU), r = (int)(u - (int64_t)c * SU), frag = r >> 6, lane = r & 63, i = lane & 31, g = lane >> 5;
    uint32_t e[4] = {0, 0, 0, 0};
    if (frag < NF1) {
      if (c < NC) {
        const int n = frag / KS, ks = frag - n * KS;
        weight_bits8(w1, 64 * c + 32 * n + i, 16 * ks + 8 * g, e);
      }
    } else if (c > 0) {
      const int q = frag - NF1, ct = q >> 2, k4 = q & 3, n = k4 >> 1, kk = k4 & 1;
      const int64_t row2 = 32 * ct + i, col2 = 64 * (c - 1) + 32 * n;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        e[j] = (uint32_t)weight_bits(w2, row2, col2 + kperm(kk, g, 2 * j)) |
               ((uint32_t)weight_bits(w2, row2, col2 + kperm(kk, g, 2 * j + 1)) << 16);
    }
    blob[u] = u32x4{e[0], e[1], e[2], e[3]};
  }
}

// Four direct global -> LDS loads of 64 x 16 bytes each (no registers): the wave's lanes read sbase + 1024 q + 16 lane
// (q = 0..3) and the data land at LDS byte address lds + 1024 q + 16 lane; the instruction offset advances the
// global and the LDS address alike.  sbase and lds are wave-uniform.  The loads are asynchronous and counted by
// vmcnt; their data must not be read before a wait and a barrier.
__device__ __forceinline__ void load_4k_to_lds(const void *sbase, unsigned lane16, unsigned lds) {
  asm volatile(
      "s_mov_b32 m0, %2\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %1, %0\n\t"
      "global_load_lds_dwordx4 %1, %0 offset:1024\n\t"
      "global_load_lds_dwordx4 %1, %0 offset:2048\n\t"
      "global_load_lds_dwordx4 %1, %0 offset:3072" ::"s"(sbase),
      "v"(lane16), "s"(lds)
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

// 8 floats -> 8 bf16 (round to nearest even)
__device__ __forceinline__ u32x4 pack8(const float (&v)[8]) {
  bf16x8 o;
#pragma unroll
  for (int j = 0; j < 8; ++j) o[j] = (__bf16)v[j];
  return __builtin_bit_cast(u32x4, o);
}

// 2 floats -> 2 bf16 (round to nearest even), the first in the low half
__device__ __forceinline__ uint32_t pack2(float a, float b) {
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  bf16x2 o;
  o[0] = (__bf16)a;
  o[1] = (__bf16)b;
  return __builtin_bit_cast(uint32_t, o);
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

  static_assert(NDMA % 4 == 0 && NDMA / 4 <= KS / 4, "the fetch of a slot is issued in groups of four loads");
  // pieces 4k .. 4k+3 (1 KB each) of this wave's share of slot c into buffer gs & 1
  auto fetch_quad = [&](int64_t gs, int c, int k) {
    const u32x4 *src = blob + (int64_t)c * SU + wave * WU + k * 256;
    const unsigned dst = (unsigned)(uintptr_t)(wbuf + (gs & 1) * SU + wave * WU + k * 256);
    load_4k_to_lds(src, lane * 16, dst);
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
    for (int k = 0; k < NDMA / 4; ++k) fetch_quad(0, 0, k);
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
    float fl[2][8];     // gelu of the first half (registers 0..7) of the tile of chunk c
    // The 32 activations of a slot (evaluation e: e < 16 -> hrest[e / 8][e % 8], else the first half of hacc) are
    // spread over its 32 / NE steps and software-pipelined over three half-steps, so that two independent
    // dependency chains are in flight behind every MFMA (a wave is alone on its SIMD and issues in order: a single
    // chain would leave its latencies exposed):
    //   behind the first MFMA of step s:      end of evaluation s - 1 (1 + e, rcp, x *)  |  start of evaluation s
    //   behind the second MFMA of step s:     polynomial and exp2 of evaluation s; one piece of the next slot's fetch
    // The last evaluation of a slot ends in the first step of the next one.
    constexpr int NE = 16 / KS > 0 ? 16 / KS : 1;  // evaluations per step
    constexpr int NS1 = KS, NS2 = 4 * CTH;
    static_assert(NS1 * NE == 16 && NS2 * NE == 16, "both phases must cover 16 evaluations");
    float px[NE], pe[NE];           // evaluation in its last part: argument, exp2 term
    float cx[NE], cx2[NE], cq[NE];  // evaluation in its first parts: argument, min(x^2, 81), polynomial so far
    // nothing of the block before may reach this one (its last slot evaluates what the zero weights of the padding
    // slot produce from its rows: finite only if those rows are)
#pragma unroll
    for (int q = 0; q < NE; ++q) px[q] = pe[q] = 0.f;
#pragma unroll
    for (int m = 0; m < 2; ++m) {
      hown[m][0] = u32x4{0, 0, 0, 0};
#pragma unroll
      for (int j = 0; j < 8; ++j) hrest[m][j] = fl[m][j] = 0.f;
    }

    for (int c = 0; c <= NC; ++c, ++gs) {
      // slot gs has landed (every wave waits for its own share, then all meet) and the other buffer is free.  The
      // first slot of a later block was waited for before the epilogue of the block before it, whose stores may
      // still be in flight here.
      if (c > 0 || gs == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      const int c_next = c < NC ? c + 1 : 0;
      const u32x4 *wb = wbuf + (gs & 1) * SU + lane;
      // this wave's fragments of the slot: W1 of hidden tile p; W2 of its channel half, hidden tile p ("own") first
      const u32x4 *w1f = wb + p * KS * 64;
      const u32x4 *w2own = wb + (NF1 + p * CTH * 4 + 2 * p) * 64, *w2par = wb + (NF1 + p * CTH * 4 + 2 * (1 - p)) * 64;

      // One slot = 2 phases of KS resp. 4 * CTH steps; a step = one weight fragment (read from LDS AHEAD steps
      // early) and two MFMAs with the vector work of the activations behind each:
      //   phase 1   h^T tile p of hidden chunk c += W1 fragment . u^T (both row halves);
      //             gelu of the second half of the tile of chunk c-1 -> the tile is complete, goes to the partner
      //   phase 2   y^T += W2 fragment(ct, k4) of hidden chunk c-1 . gelu(h)^T (own tile, then the partner's);
      //             gelu of the first half of the tile of chunk c
      constexpr int RING = 6, AHEAD = 5;
      f32x16 hacc[2];
#pragma unroll
      for (int r = 0; r < 16; ++r) hacc[0][r] = hacc[1][r] = b1s[(c < NC ? 64 * c : 0) + 32 * p + rowmap(r, g)];
      // vector work behind the first MFMA of step S (0 .. NS1 + NS2 - 1 over both phases)
      auto behind_first = [&](auto S_) {
        constexpr int S = decltype(S_)::value;
        static_for<NE>([&](auto q_) {
          constexpr int q = decltype(q_)::value, e = S * NE + q, ep = (e + 32 - NE) % 32, m = (ep % 16) / 8, j = ep % 8;
          const float done = px[q] * __builtin_amdgcn_rcpf(1.f + pe[q]);
          if constexpr (ep < 16) {
            hrest[m][j] = done;
            if constexpr (j == 7) hown[m][1] = pack8(hrest[m]);
          } else {
            fl[m][j] = done;
            if constexpr (j == 7) hown[m][0] = pack8(fl[m]);
          }
          if constexpr (e < 16) cx[q] = hrest[e / 8][e % 8];
          else cx[q] = hacc[(e - 16) / 8][e % 8];
          cx2[q] = fminf(cx[q] * cx[q], 81.f);
          cq[q] = fmaf(-3.51902394e-04f * -2.f * kLog2e, cx2[q], 3.70080200e-02f * -2.f * kLog2e);
        });
      };
      auto behind_second = [&]() {
#pragma unroll
        for (int q = 0; q < NE; ++q) {
          const float t2 = fmaf(cq[q], cx2[q], 7.97505275e-01f * -2.f * kLog2e);
          px[q] = cx[q];
          pe[q] = __builtin_amdgcn_exp2f(cx[q] * t2);
        }
      };
      {
        // fragment of step S of the slot: W1 (tile p, k-step S) in phase 1, then W2 with (k4' = t / CTH, ct = t % CTH),
        // k4' < 2: own tile, kk = k4' % 2
        auto frag = [&](auto S_) {
          constexpr int S = decltype(S_)::value;
          if constexpr (S < NS1) {
            return w1f[S * 64];
          } else {
            constexpr int t = S - NS1, k4 = t / CTH, ct = t % CTH;
            return (k4 < 2 ? w2own : w2par)[(ct * 4 + (k4 & 1)) * 64];
          }
        };
        u32x4 fr[RING];  // one ring over both phases: the first fragments of phase 2 are on their way before phase 1 ends
        static_for<AHEAD>([&](auto q) { fr[decltype(q)::value] = frag(q); });
        static_for<NS1 + NS2>([&](auto S_) {
          constexpr int S = decltype(S_)::value;
          if constexpr (S == NS1 + 2 * CTH - 2) {  // two steps before the partner's tile (written in step NS1) is needed
            __syncthreads();
#pragma unroll
            for (int m = 0; m < 2; ++m)
#pragma unroll
              for (int k = 0; k < 2; ++k) hpar[m][k] = xch[(((wave ^ 1) * 2 + m) * 2 + k) * 64 + lane];
          }
          if constexpr (S + AHEAD < NS1 + NS2) fr[(S + AHEAD) % RING] = frag(std::integral_constant<int, S + AHEAD>{});
          const u32x4 a = fr[S % RING];
          if constexpr (S < NS1) {
            hacc[0] = mma(a, ub[0][S], hacc[0]);
            __builtin_amdgcn_sched_barrier(0);  // keeps the issue order as written
            behind_first(S_);
            __builtin_amdgcn_sched_barrier(0);
            hacc[1] = mma(a, ub[1][S], hacc[1]);
            __builtin_amdgcn_sched_barrier(0);
            behind_second();
            // the other buffer was last read in phase 2 of the slot before this one
            if constexpr (S % 4 == 3 && S / 4 < NDMA / 4) fetch_quad(gs + 1, c_next, S / 4);
            __builtin_amdgcn_sched_barrier(0);
          } else {
            constexpr int t = S - NS1, k4 = t / CTH, ct = t % CTH, kk = k4 & 1;
            // own tile: hown[m][0] (first half of chunk c-1) is read in steps 0 .. CTH-1 and rewritten (chunk c) from
            // step 8 / NE on; hown[m][1] is complete after the first half-step of step 0 and read from step CTH on
            yacc[0][ct] = mma(a, k4 < 2 ? hown[0][kk] : hpar[0][kk], yacc[0][ct]);
            __builtin_amdgcn_sched_barrier(0);
            behind_first(S_);
            __builtin_amdgcn_sched_barrier(0);
            yacc[1][ct] = mma(a, k4 < 2 ? hown[1][kk] : hpar[1][kk], yacc[1][ct]);
            __builtin_amdgcn_sched_barrier(0);
            behind_second();
            if constexpr (t == 0) {
              // the tile of chunk c-1 is complete: hand it to the partner (who reads it after the barrier above;
              // the one at the start of the next slot separates that read from the next write)
#pragma unroll
              for (int m = 0; m < 2; ++m)
#pragma unroll
                for (int k = 0; k < 2; ++k) xch[((wave * 2 + m) * 2 + k) * 64 + lane] = hown[m][k];
            }
            __builtin_amdgcn_sched_barrier(0);
          }
        });
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
          for (int j = 0; j < 8; ++j) hrest[m][j] = hacc[m][8 + j];
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
        rsd[rr] = load_streaming(reinterpret_cast<const rowv *>(residual + r * C + i * CPH));
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
      if (ok) store_streaming(reinterpret_cast<rowv *>(y + r * C + i * CPH), ob);
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
        if (ok) store_streaming(reinterpret_cast<rowv *>(ln_out + r * C + i * CPH), lb);
      }
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing may still be landing in LDS when the workgroup ends
}

// ---------------------------------------------------------------------------------------------------------------
// The same MLP for C = 512 (and, for comparison, 256): every wave owns 32 rows of the block outright.
//
// One workgroup of 4 waves per CU, one wave per SIMD; a block is 128 rows.  A wave keeps its rows' inputs (B operands,
// C/4 registers) and all C output channels of y^T (C/2 accumulation registers) for the whole block and shares nothing
// but the weight stream with the other waves: no tile exchange, one barrier per slot.  The price is that a weight
// fragment read from LDS feeds one MFMA only (32 B per cycle and SIMD, half of what LDS delivers).
//
// Weights stream through LDS in slots of HS hidden units (HS = 16384 / C: 64 KB of W1 and W2 fragments per slot, two
// buffers).  The MFMAs of the two products alternate, so that no accumulator is used twice in a row and the vector
// work of the activation finds an MFMA to hide behind everywhere; the products therefore run two slots apart:
//   slot c:   h(c)^T = W1[chunk c] . u^T + b1           (first MFMA of every pair)
//             g(c-1) = gelu(h(c-1)), rounded to bf16: B operands of the second product (vector work, in two or three
//             parts behind consecutive MFMAs)
//             y^T   += W2[:, chunk c-2] . g(c-2)^T      (second MFMA of every pair)
// Slot c of the packed weights holds the fragments in the order they are consumed: pair P = 0..31 -> W1 fragment
// (tile P % NT, k-step P / NT) of chunk c, then W2 fragment (ct = P % CT, tile and k-half from P / CT) of chunk c-2.
// ---------------------------------------------------------------------------------------------------------------
namespace rows {

template <int C>
struct Cfg {
  static constexpr int KS = C / 16, CT = C / 32;
  static constexpr int HS = 16384 / C;  // hidden units per slot
  static constexpr int NT = HS / 32;    // hidden tiles per slot
  static constexpr int NP = 32;         // MFMA pairs per slot
  static constexpr int SU = 2 * NP * 64;  // 16-byte units per slot
  static_assert(NT * KS == NP && CT * NT * 2 == NP, "both products take 32 MFMAs per slot");
};

__global__ __launch_bounds__(256) void pack_kernel(WeightView w1, WeightView w2, u32x4 *__restrict__ blob, int C, int F) {
  const int KS = C / 16, CT = C / 32, HS = 16384 / C, NT = HS / 32, NCH = F / HS;
  (void)KS;
  const int64_t total = (int64_t)(NCH + 2) * 4096;
  for (int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x; u < total; u += (int64_t)gridDim.x * 256) {
    const int c = (int)(u >> 12), r = (int)(u & 4095), frag = r >> 6, lane = r & 63, i = lane & 31, g = lane >> 5;
    const int P = frag >> 1;
    uint32_t e[4] = {0, 0, 0, 0};
    if ((frag & 1) == 0) {
      if (c < NCH) {
        const int n = P % NT, ks = P / NT;
        weight_bits8(w1, HS * c + 32 * n + i, 16 * ks + 8 * g, e);
      }
    } else if (c >= 2) {
      const int ct = P % CT, nk = P / CT, n = nk >> 1, kk = nk & 1;
      const int64_t row2 = 32 * ct + i, col2 = HS * (c - 2) + 32 * n;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        e[j] = (uint32_t)weight_bits(w2, row2, col2 + kperm(kk, g, 2 * j)) |
               ((uint32_t)weight_bits(w2, row2, col2 + kperm(kk, g, 2 * j + 1)) << 16);
    }
    blob[u] = u32x4{e[0], e[1], e[2], e[3]};
  }
}

// acc += A . B with the accumulator in ordinary vector registers.  The compiler places every MFMA accumulator of a
// kernel with more than 256 registers in the accumulation half of the register file; the 256 registers of y^T fill
// that half, so the h^T tile is kept out of it by issuing its MFMAs this way.  The compiler does not see an MFMA here:
// the caller keeps vector reads and writes of acc well away from it (an MFMA on another accumulator in between).
__device__ __forceinline__ void mma_in_vgprs(u32x4 a, u32x4 b, f32x16 &acc) {
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b));
}

// LayerNorm of a wave's 32 rows held as B operands (lane (i, g): channels 16 ks + 8 g .. + 7 of row i for every k-step,
// i.e. half a row; lane ^ 32 holds the other half), in place: the rows a producer left un-normalised become the
// operands of the first product.  The sums of x and x^2 come from the packed pairs themselves (v_dot2c_f32_bf16: two
// exact bf16 products and a float32 accumulation per instruction, four chains each), the variance as
// E[x^2] - mean^2 in float32 -- exact enough for a residual stream, whose mean is of the order of its spread; gams /
// bets: weight and bias in LDS.
template <int C>
__device__ __forceinline__ void normalize_operand_rows(u32x4 (&ub)[C / 16], const float *gams, const float *bets, float eps,
                                                       int g) {
  constexpr int KS = C / 16;
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  const bf16x2 ones = {(__bf16)1.f, (__bf16)1.f};
  float s[4] = {0.f, 0.f, 0.f, 0.f}, q[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const uint32_t word = ub[ks][w];  // through a scalar: a bit cast straight off the vector element reads element 0
      const bf16x2 pr = __builtin_bit_cast(bf16x2, word);
      s[w] = __builtin_amdgcn_fdot2_f32_bf16(pr, ones, s[w], false);
      q[w] = __builtin_amdgcn_fdot2_f32_bf16(pr, pr, q[w], false);
    }
  const float mean = half_sum((s[0] + s[1]) + (s[2] + s[3])) * (1.f / C);
  const float ex2 = half_sum((q[0] + q[1]) + (q[2] + q[3])) * (1.f / C);
  const float rstd = rsqrtf(fmaxf(fmaf(-mean, mean, ex2), 0.f) + eps), shift = -mean * rstd;
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const f32x4 ga = *reinterpret_cast<const f32x4 *>(gams + 16 * ks + 8 * g), gb = *reinterpret_cast<const f32x4 *>(gams + 16 * ks + 8 * g + 4);
    const f32x4 ba = *reinterpret_cast<const f32x4 *>(bets + 16 * ks + 8 * g), bb = *reinterpret_cast<const f32x4 *>(bets + 16 * ks + 8 * g + 4);
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float g0 = w < 2 ? ga[2 * w] : gb[2 * w - 4], g1 = w < 2 ? ga[2 * w + 1] : gb[2 * w - 3];
      const float c0 = w < 2 ? ba[2 * w] : bb[2 * w - 4], c1 = w < 2 ? ba[2 * w + 1] : bb[2 * w - 3];
      const float v0 = __uint_as_float(ub[ks][w] << 16), v1 = __uint_as_float(ub[ks][w] & 0xffff0000u);
      ub[ks][w] = pack2(fmaf(fmaf(v0, rstd, shift), g0, c0), fmaf(fmaf(v1, rstd, shift), g1, c1));
    }
  }
}

// Epilogue of the row-owning kernels: a wave's y^T (channel 32 ct + rowmap(r, g) of row i, C channels x 32 rows) to
// row-major bf16 rows, + residual, LayerNorm, full-row stores.  The rows pass through `stg`, the wave's own STG bytes
// of LDS, RPR = STG / (2 C) rows at a time; after_staging() is called once the last round is staged (the accumulators
// are free from then on).  gams / bets: LayerNorm weight and bias in LDS.
template <int C, bool HAS_RES, bool HAS_LN, int STG = 16384, class AfterStaging>
__device__ __forceinline__ void finish_rows(const f32x16 (&yacc)[C / 32], uint32_t *stg, int i, int g, int64_t row0,
                                            int64_t M, const uint16_t *__restrict__ residual, uint16_t *__restrict__ y,
                                            uint16_t *__restrict__ ln_out, const float *gams, const float *bets,
                                            float ln_eps, AfterStaging &&after_staging, int64_t ld = C) {
  constexpr int CT = C / 32;
  constexpr int G4 = C / 4;             // 8-byte granules (4 channels) per staged row
  constexpr int RPR = STG / (2 * C);  // rows staged per round
  constexpr int NROUND = 32 / RPR;
  // lane indices taken afresh, so that nothing derived from them for the epilogue is kept across the slot loop
  int il = i, gl = g;
  asm volatile("" : "+v"(il), "+v"(gl));
  const int hl = gl;  // each half of the wave finishes one row per step
  typedef uint32_t rowv __attribute__((ext_vector_type(4)));
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  constexpr int NV = C / 256;  // 16-byte pieces per lane and row: piece v = channels 256 v + 8 il .. + 7
  static_assert(C % 256 == 0, "half a wave covers 256 consecutive channels per access");
  // y^T -> bf16 once: yp[ct][q] = channels 32 ct + 8 q + 4 g .. + 3 of row i; the accumulators are free after this
  u32x2 yp[CT][4];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      yp[ct][q][0] = pack2(yacc[ct][4 * q + 0], yacc[ct][4 * q + 1]);
      yp[ct][q][1] = pack2(yacc[ct][4 * q + 2], yacc[ct][4 * q + 3]);
    }
  constexpr int NIT = RPR / 2;             // steps per round: two rows each
  constexpr int PF = NIT < 4 ? NIT : 4;    // residual rows are fetched this many steps ahead
#pragma unroll
  for (int rd = 0; rd < NROUND; ++rd) {
    rowv rsd[NIT][NV];
    auto load_residual = [&](auto rr_) {
      constexpr int rr = decltype(rr_)::value;
      if constexpr (HAS_RES) {
        int64_t r = row0 + rd * RPR + 2 * rr + hl;
        if (r >= M) r = M > 0 ? M - 1 : 0;  // M = 0: a wave without rows (nothing is stored)
#pragma unroll
        for (int v = 0; v < NV; ++v) rsd[rr][v] = load_streaming(reinterpret_cast<const rowv *>(residual + r * ld + 256 * v + 8 * il));
      }
    };
    static_for<PF>(load_residual);
    // staged rows: granule gr (4 channels) of row rw sits at gr ^ ((2 rw) % G4)
    if (NROUND == 1 || (il / RPR) == rd) {
      const int rw = il % RPR;
#pragma unroll
      for (int ct = 0; ct < CT; ++ct)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int gr = (8 * ct + 2 * q + gl) ^ ((2 * rw) & (G4 - 1));
          *reinterpret_cast<u32x2 *>(stg + rw * (C / 2) + gr * 2) = yp[ct][q];
        }
    }
    // the wave's LDS operations complete in order: its reads below see the writes above.  Once the last round is
    // staged the rows of this workgroup's next block can travel (past the end: this block again)
    if (rd == NROUND - 1) after_staging();
    // two rows per step: lanes 0-31 one row, lanes 32-63 the next
    static_for<NIT>([&](auto rr_) {
      constexpr int rr = decltype(rr_)::value;
      if constexpr (rr + PF < NIT) load_residual(std::integral_constant<int, rr + PF>{});
      const int rw = 2 * rr + hl;
      const int64_t r = row0 + rd * RPR + rw;
      const bool ok = r < M;
      float val[8 * NV];
#pragma unroll
      for (int v = 0; v < NV; ++v) {
        // granules 64 v + 2 il, + 1 of row rw; the swizzle flips an even number, so the pair stays adjacent
        const rowv sv = *reinterpret_cast<const rowv *>(stg + rw * (C / 2) + (((64 * v + 2 * il) ^ ((2 * rw) & (G4 - 1))) << 1));
        rowv ob;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          float t0 = __uint_as_float(sv[w] << 16), t1 = __uint_as_float(sv[w] & 0xffff0000u);
          if constexpr (HAS_RES) {  // the MLP output is a bf16 tensor; the sum is rounded again
            t0 += __uint_as_float(rsd[rr][v][w] << 16);
            t1 += __uint_as_float(rsd[rr][v][w] & 0xffff0000u);
          }
          ob[w] = pack2(t0, t1);
          val[8 * v + 2 * w] = __uint_as_float(ob[w] << 16);
          val[8 * v + 2 * w + 1] = __uint_as_float(ob[w] & 0xffff0000u);
        }
        if (ok) store_streaming(reinterpret_cast<rowv *>(y + r * ld + 256 * v + 8 * il), ob);
      }
      if constexpr (HAS_LN) {
        float s1 = 0.f;
#pragma unroll
        for (int k = 0; k < 8 * NV; ++k) s1 += val[k];
        const float mean = half_wave_sum(s1) * (1.f / C);
        float s2 = 0.f;
#pragma unroll
        for (int k = 0; k < 8 * NV; ++k) {
          const float dl = val[k] - mean;
          s2 = fmaf(dl, dl, s2);
        }
        const float rstd = rsqrtf(half_wave_sum(s2) * (1.f / C) + ln_eps);
        const float shift = -mean * rstd;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
          const f32x4 ga = *reinterpret_cast<const f32x4 *>(gams + 256 * v + 8 * il), gb = *reinterpret_cast<const f32x4 *>(gams + 256 * v + 8 * il + 4);
          const f32x4 ba = *reinterpret_cast<const f32x4 *>(bets + 256 * v + 8 * il), bb = *reinterpret_cast<const f32x4 *>(bets + 256 * v + 8 * il + 4);
          rowv lb;
#pragma unroll
          for (int w = 0; w < 4; ++w) {
            const float g0 = w < 2 ? ga[2 * w] : gb[2 * w - 4], g1 = w < 2 ? ga[2 * w + 1] : gb[2 * w - 3];
            const float c0 = w < 2 ? ba[2 * w] : bb[2 * w - 4], c1 = w < 2 ? ba[2 * w + 1] : bb[2 * w - 3];
            lb[w] = pack2(fmaf(fmaf(val[8 * v + 2 * w], rstd, shift), g0, c0), fmaf(fmaf(val[8 * v + 2 * w + 1], rstd, shift), g1, c1));
          }
          if (ok) store_streaming(reinterpret_cast<rowv *>(ln_out + r * ld + 256 * v + 8 * il), lb);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  }
}

// in_gamma != nullptr: the rows of u are un-normalised; the kernel applies LayerNorm(in_gamma, in_beta, in_eps) to them
// as it turns them into operands (the block's ln_mlp1[0], transolver.py:303, without a trip through memory).
template <int C, int TAIL>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void mlp_rows_kernel(
    const u32x4 *__restrict__ blob, const float *__restrict__ b1, const float *__restrict__ b2,
    const uint16_t *__restrict__ u, uint16_t *__restrict__ y, const uint16_t *__restrict__ residual,
    const float *__restrict__ ln_gamma, const float *__restrict__ ln_beta, float ln_eps, uint16_t *__restrict__ ln_out,
    int64_t M, int F, int64_t nblocks, const float *__restrict__ in_gamma, const float *__restrict__ in_beta,
    float in_eps) {
  using K = Cfg<C>;
  constexpr bool HAS_RES = TAIL == 1 || TAIL == 2, HAS_LN = TAIL == 1 || TAIL == 3;
  constexpr int KS = K::KS, CT = K::CT, HS = K::HS, NT = K::NT, NP = K::NP, SU = K::SU;
  constexpr int WU = SU / 4;    // units of a slot fetched by each wave (16 KB: four groups of four loads)
  extern __shared__ u32x4 smem[];
  u32x4 *wbuf = smem;  // 2 * SU
  float *b1s = reinterpret_cast<float *>(wbuf + 2 * SU);
  float *b2s = b1s + F;
  float *gams = b2s + C, *bets = gams + C;  // LayerNorm weight and bias
  float *igams = bets + C, *ibets = igams + C;  // weight and bias of the LayerNorm applied to the input rows
  const int tid = threadIdx.x, lane = tid & 63, i = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: addresses derived from it stay scalar
  const int NCH = F / HS;

  for (int k = tid; k < F; k += 256) b1s[k] = b1[k];
  for (int k = tid; k < C; k += 256) {
    b2s[k] = b2[k];
    gams[k] = HAS_LN ? ln_gamma[k] : 1.f;
    bets[k] = HAS_LN ? ln_beta[k] : 0.f;
    igams[k] = in_gamma ? in_gamma[k] : 1.f;
    ibets[k] = in_gamma ? in_beta[k] : 0.f;
  }
  __syncthreads();  // the biases are read before the first barrier of the slot loop

  // 4 KB group k of this wave's share of slot c into buffer gs & 1
  auto fetch_group = [&](int64_t gs, int c, int k) {
    const u32x4 *src = blob + (int64_t)c * SU + wave * WU + k * 256;
    const unsigned dst = (unsigned)(uintptr_t)(wbuf + (gs & 1) * SU + wave * WU + k * 256);
    load_4k_to_lds(src, lane * 16, dst);
  };
  // lane (i, g) holds row i of the wave's 32, channels 16 ks + 8 g .. + 7
  auto load_rows = [&](int64_t mb, u32x4(&ub)[KS]) {
    int64_t r = mb * kRowsPerBlock + wave * 32 + i;
    if (r >= M) r = M - 1;
    const uint16_t *src = u + r * C + 8 * g;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) ub[ks] = *reinterpret_cast<const u32x4 *>(src + 16 * ks);
  };

  int64_t gs = 0;  // slots processed so far by this workgroup (buffer parity)
  if ((int64_t)blockIdx.x < nblocks) {
#pragma unroll
    for (int k = 0; k < 4; ++k) fetch_group(0, 0, k);
  }
  u32x4 ub[KS];
  if ((int64_t)blockIdx.x < nblocks) load_rows(blockIdx.x, ub);
  for (int64_t mb = blockIdx.x; mb < nblocks; mb += gridDim.x) {
    const int64_t row0 = mb * kRowsPerBlock + wave * 32;
    if (in_gamma) normalize_operand_rows<C>(ub, igams, ibets, in_eps, g);
    f32x16 yacc[CT];  // channel 32 ct + rowmap(r, g) of row i
    f32x16 hacc[NT];  // hidden unit 32 n + rowmap(r, g) of the slot's chunk, row i
    // the output bias is where the sum starts; nothing of the block before may reach this one (the padding slots
    // multiply what the rows produce by zero weights, which is zero only for finite rows)
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
      for (int r = 0; r < 16; ++r) yacc[ct][r] = b2s[32 * ct + rowmap(r, g)];
#pragma unroll
    for (int n = 0; n < NT; ++n)
#pragma unroll
      for (int r = 0; r < 16; ++r) hacc[n][r] = 0.f;
    // gelu(h) of chunk c-2 as B operands [tile][k half].  The operands of chunk c-1 replace them one by one as soon
    // as the last MFMA that reads the old one is issued: operand q = 2 n + kk is read by pairs q CT .. (q+1) CT - 1 and
    // complete (eight evaluations, packed two by two into gnew) with evaluation 8 q + 7.
    u32x4 gprev[NT][2], gnew = u32x4{0, 0, 0, 0};
#pragma unroll
    for (int n = 0; n < NT; ++n) gprev[n][0] = gprev[n][1] = u32x4{0, 0, 0, 0};

    for (int c = 0; c < NCH + 2; ++c, ++gs) {
      // slot gs has landed (every wave waits for its own share, then all meet) and the other buffer is free.  The
      // first slot of a later block was waited for before the epilogue of the block before it, whose stores may
      // still be in flight here.
      if (c > 0 || gs == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      const int c_next = c < NCH + 1 ? c + 1 : 0;
      const u32x4 *wb = wbuf + (gs & 1) * SU + lane;
      float hprev[NT][16];  // h(c-1), to be activated in this slot
#pragma unroll
      for (int n = 0; n < NT; ++n)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          hprev[n][r] = hacc[n][r];
          hacc[n][r] = b1s[(c < NCH ? HS * c : 0) + 32 * n + rowmap(r, g)];
        }
      // evaluation e = 0 .. 16 NT - 1 of the slot is register e % 16 of tile e / 16; eight results in a row make one
      // B operand.  NT = 2: one evaluation per pair, its end behind the first MFMA of the next pair; NT = 1: one
      // evaluation per two pairs.
      float ex = 0.f, ex2 = 0.f, eq = 0.f, ee = 0.f;  // evaluation in flight: argument, min(x^2, 81), polynomial, exp2 term
      float feven = 0.f;                              // result of the even evaluation of a pair of results
      auto begin1 = [&](auto e_) {
        constexpr int e = decltype(e_)::value;
        ex = hprev[e / 16][e % 16];
        ex2 = fminf(ex * ex, 81.f);
        eq = fmaf(-3.51902394e-04f * -2.f * kLog2e, ex2, 3.70080200e-02f * -2.f * kLog2e);
      };
      auto begin2 = [&]() {
        const float t2 = fmaf(eq, ex2, 7.97505275e-01f * -2.f * kLog2e);
        ee = __builtin_amdgcn_exp2f(ex * t2);
      };
      // end of evaluation e with argument x and exp2 term t
      auto finish = [&](auto e_, float x, float t) {
        constexpr int e = decltype(e_)::value, j = e % 8;
        const float v = x * __builtin_amdgcn_rcpf(1.f + t);
        if constexpr (j % 2 == 0) feven = v;
        else gnew[j / 2] = pack2(feven, v);
      };
      // operand q of chunk c-1 replaces the one of chunk c-2
      auto publish = [&](auto q_) {
        constexpr int q = decltype(q_)::value;
        gprev[q / 2][q % 2] = gnew;
      };

      constexpr int RING = 8, AHEAD = 6;  // in fragments; a pair consumes two
      u32x4 fr[RING];
      static_for<AHEAD>([&](auto q) { fr[decltype(q)::value] = wb[decltype(q)::value * 64]; });
      static_for<NP>([&](auto P_) {
        constexpr int P = decltype(P_)::value;
        constexpr int n1 = P % NT, ks1 = P / NT;
        constexpr int ct = P % CT, nk = P / CT, n2 = nk >> 1, kk = nk & 1;
        if constexpr (2 * P + AHEAD < 2 * NP) fr[(2 * P + AHEAD) % RING] = wb[(2 * P + AHEAD) * 64];
        if constexpr (P == 0) asm volatile("s_nop 7" ::: "memory");  // hacc was just written by vector instructions
        mma_in_vgprs(fr[(2 * P) % RING], ub[ks1], hacc[n1]);
        __builtin_amdgcn_sched_barrier(0);  // keeps the issue order as written
        // Evaluation e ends behind the first MFMA of pair PF(e) = e EPV + EPV (EPV = pairs per evaluation), operand q
        // is complete at PF(8 q + 7) = (q + 1) CT and last read by the second MFMA of pair (q + 1) CT - 1: it is
        // published behind the second MFMA of pair (q + 1) CT (operand 2 NT - 1: of the last pair, where its last
        // evaluation ends too).
        constexpr int EPV = 2 / NT;
        if constexpr (EPV == 1) {
          // the end of the evaluation before and the start of this one: two independent chains
          const float done_x = ex, done_e = ee;
          begin1(P_);
          if constexpr (P > 0) finish(std::integral_constant<int, P - 1>{}, done_x, done_e);
        } else {
          if constexpr (P % 2 == 0) {
            const float done_x = ex, done_e = ee;
            begin1(std::integral_constant<int, P / 2>{});
            if constexpr (P > 0) finish(std::integral_constant<int, P / 2 - 1>{}, done_x, done_e);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (2 * P + 1 + AHEAD < 2 * NP) fr[(2 * P + 1 + AHEAD) % RING] = wb[(2 * P + 1 + AHEAD) * 64];
        yacc[ct] = mma(fr[(2 * P + 1) % RING], gprev[n2][kk], yacc[ct]);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (EPV == 1 || P % 2 == 0) begin2();
        if constexpr (P > 0 && P % CT == 0) publish(std::integral_constant<int, P / CT - 1>{});
        if constexpr (P == NP - 1) {
          finish(std::integral_constant<int, 16 * NT - 1>{}, ex, ee);
          publish(std::integral_constant<int, 2 * NT - 1>{});
        }
        // the other buffer was last read in the slot before this one
        if constexpr (P % 8 == 3) fetch_group(gs + 1, c_next, P / 8);
        __builtin_amdgcn_sched_barrier(0);
      });
    }

    // ---- epilogue: the buffer of the last slot is idle once every wave is past its last MFMA; each wave stages
    // ---- its own rows in its own quarter of it, RPR rows at a time ----
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's share of the next block's first slot has landed
    __syncthreads();
    uint32_t *stg = reinterpret_cast<uint32_t *>(wbuf + ((gs - 1) & 1) * SU + wave * WU);  // this wave's 16 KB
    // once the last rows are staged the rows of this workgroup's next block can travel (past the end: this block again)
    finish_rows<C, HAS_RES, HAS_LN>(yacc, stg, i, g, row0, M, residual, y, ln_out, gams, bets, ln_eps,
                                    [&]() { load_rows(mb + gridDim.x < nblocks ? mb + gridDim.x : mb, ub); });
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing may still be landing in LDS when the workgroup ends
}

// ---------------------------------------------------------------------------------------------------------------
// mlp_rows2_kernel: the row-owning MLP for C = 256 with two waves per SIMD.  Workgroup = 8 waves, a block = 256 rows, a
// wave owns 32 rows: inputs as B operands (64 registers), y^T for all 256 channels (128 registers), everything else
// small enough for 256 registers per wave, so that the second wave of a SIMD covers the first one's vector work and
// LDS waits.  Weights stream in slots of 32 hidden units (32 KB: 16 W1 fragments of chunk c, then 16 W2 fragments of
// chunk c-1 ordered k-half major), two buffers, one barrier per slot; per slot a wave runs
//   phase 1   h(c)^T = W1[chunk c] . u^T + b1                       16 MFMAs on one accumulator
//   phase 2   y^T += W2[:, chunk c-1] . g(c-1)^T                    16 MFMAs (k half 0 for all channel tiles, then 1)
//             with g(c) = gelu(h(c)) evaluated behind them, one value per MFMA, straight from the accumulator of
//             phase 1; the first B operand of g(c) replaces that of g(c-1) once its last reader is issued.
// The epilogue stages through 8 KB per wave of a separate 64 KB region.
// ---------------------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void pack2_kernel(WeightView w1, WeightView w2, u32x4 *__restrict__ blob, int C, int F) {
  const int KS = C / 16, CT = C / 32, NCH = F / 32, SU = (KS + 2 * CT) * 64;
  const int64_t total = (int64_t)(NCH + 1) * SU;
  for (int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x; u < total; u += (int64_t)gridDim.x * 256) {
    const int c = (int)(u / SU), r = (int)(u - (int64_t)c * SU), frag = r >> 6, lane = r & 63, i = lane & 31, g = lane >> 5;
    uint32_t e[4] = {0, 0, 0, 0};
    if (frag < KS) {
      if (c < NCH) {
        weight_bits8(w1, 32 * c + i, 16 * frag + 8 * g, e);
      }
    } else if (c > 0) {
      const int t = frag - KS, kk = t / CT, ct = t % CT;
      const int64_t row2 = 32 * ct + i, col2 = 32 * (c - 1);
#pragma unroll
      for (int j = 0; j < 4; ++j)
        e[j] = (uint32_t)weight_bits(w2, row2, col2 + kperm(kk, g, 2 * j)) |
               ((uint32_t)weight_bits(w2, row2, col2 + kperm(kk, g, 2 * j + 1)) << 16);
    }
    blob[u] = u32x4{e[0], e[1], e[2], e[3]};
  }
}

// WAVES = 8: one workgroup per CU (two waves per SIMD from the same workgroup), epilogue staged in a region of its
// own.  WAVES = 4: two workgroups per CU, each with one wave per SIMD and its own weight stream; the epilogue of one
// (bound by the CU's store rate) then overlaps with the matrix work of the other; it stages through the idle weight
// buffer.
template <int C, int TAIL, int WAVES>
__global__ __launch_bounds__(64 * WAVES, 8 / WAVES) void mlp_rows2_kernel(
    const u32x4 *__restrict__ blob, const float *__restrict__ b1, const float *__restrict__ b2,
    const uint16_t *__restrict__ u, uint16_t *__restrict__ y, const uint16_t *__restrict__ residual,
    const float *__restrict__ ln_gamma, const float *__restrict__ ln_beta, float ln_eps, uint16_t *__restrict__ ln_out,
    int64_t M, int F, int64_t nblocks, const float *__restrict__ in_gamma, const float *__restrict__ in_beta,
    float in_eps) {
  constexpr bool HAS_RES = TAIL == 1 || TAIL == 2, HAS_LN = TAIL == 1 || TAIL == 3;
  constexpr int KS = C / 16, CT = C / 32, NF = KS + 2 * CT, SU = NF * 64;
  constexpr int WU = SU / WAVES;   // units of a slot fetched by each wave
  constexpr int NGRP = WU / 256;   // groups of four loads per wave and slot
  static_assert(WU % 256 == 0, "whole groups of four loads per wave and slot");
  constexpr int STG = 8192;        // bytes of epilogue staging per wave
  constexpr int kRows = 32 * WAVES;  // rows per block
  constexpr bool OWN_STAGE = WAVES == 8;
  extern __shared__ u32x4 smem[];
  u32x4 *wbuf = smem;                                             // 2 * SU
  uint32_t *stage = reinterpret_cast<uint32_t *>(wbuf + 2 * SU);  // OWN_STAGE: 8 waves x STG bytes
  float *b1s = reinterpret_cast<float *>(stage + (OWN_STAGE ? 8 * STG / 4 : 0));
  float *b2s = b1s + F;
  float *gams = b2s + C, *bets = gams + C;
  float *igams = bets + C, *ibets = igams + C;  // weight and bias of the LayerNorm applied to the input rows
  const int tid = threadIdx.x, lane = tid & 63, i = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: addresses derived from it stay scalar
  const int NCH = F / 32;
  for (int k = tid; k < F; k += 64 * WAVES) b1s[k] = b1[k];
  for (int k = tid; k < C; k += 64 * WAVES) {
    b2s[k] = b2[k];
    gams[k] = HAS_LN ? ln_gamma[k] : 1.f;
    bets[k] = HAS_LN ? ln_beta[k] : 0.f;
    igams[k] = in_gamma ? in_gamma[k] : 1.f;
    ibets[k] = in_gamma ? in_beta[k] : 0.f;
  }
  __syncthreads();
  auto fetch = [&](int64_t gs, int c) {  // this wave's share of slot c into buffer gs & 1
#pragma unroll
    for (int k = 0; k < NGRP; ++k) {
      const u32x4 *src = blob + (int64_t)c * SU + wave * WU + k * 256;
      const unsigned dst = (unsigned)(uintptr_t)(wbuf + (gs & 1) * SU + wave * WU + k * 256);
      load_4k_to_lds(src, lane * 16, dst);
    }
  };
  auto load_rows = [&](int64_t mb, u32x4(&ub)[KS]) {
    int64_t r = mb * kRows + wave * 32 + i;
    if (r >= M) r = M - 1;
    const uint16_t *src = u + r * C + 8 * g;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) ub[ks] = *reinterpret_cast<const u32x4 *>(src + 16 * ks);
  };
  int64_t gs = 0;
  if ((int64_t)blockIdx.x < nblocks) fetch(0, 0);
  u32x4 ub[KS];
  if ((int64_t)blockIdx.x < nblocks) load_rows(blockIdx.x, ub);
  for (int64_t mb = blockIdx.x; mb < nblocks; mb += gridDim.x) {
    const int64_t row0 = mb * kRows + wave * 32;
    if (in_gamma) normalize_operand_rows<C>(ub, igams, ibets, in_eps, g);
    f32x16 yacc[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
      for (int r = 0; r < 16; ++r) yacc[ct][r] = b2s[32 * ct + rowmap(r, g)];
    // gelu(h) of the chunk before as the two B operands of phase 2; nothing of the block before may reach this one.
    // The 16 activations of a chunk are spread over the 32 MFMAs that follow its first product, one per two MFMAs:
    // the first eight (k half 0) behind phase 2 of the same slot, straight from the accumulator, the other eight
    // (copied to hrest at the end of the slot) behind phase 1 of the next one.
    u32x4 gop[2] = {u32x4{0, 0, 0, 0}, u32x4{0, 0, 0, 0}}, gnew = u32x4{0, 0, 0, 0};
    float hrest[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) hrest[j] = 0.f;
    float ex = 0.f, ee = 0.f, feven = 0.f;  // evaluation in flight: argument and exp2 term; even result of a pair
    auto begin = [&](float x) {
      ex = x;
      const float x2 = fminf(x * x, 81.f);
      float q = fmaf(-3.51902394e-04f * -2.f * kLog2e, x2, 3.70080200e-02f * -2.f * kLog2e);
      q = fmaf(q, x2, 7.97505275e-01f * -2.f * kLog2e);
      ee = __builtin_amdgcn_exp2f(x * q);
    };
    auto finish = [&](auto j_) {  // result j (0 .. 7) of the operand being formed
      constexpr int j = decltype(j_)::value;
      const float v = ex * __builtin_amdgcn_rcpf(1.f + ee);
      if constexpr (j % 2 == 0) feven = v;
      else gnew[j / 2] = pack2(feven, v);
    };
    for (int c = 0; c <= NCH; ++c, ++gs) {
      // slot gs has landed (every wave waits for its own share, then all meet) and the other buffer is free.  The
      // first slot of a later block was waited for before the epilogue of the block before it.
      if (c > 0 || gs == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      const u32x4 *wb = wbuf + (gs & 1) * SU + lane;
      f32x16 hacc;
#pragma unroll
      for (int r = 0; r < 16; ++r) hacc[r] = b1s[(c < NCH ? 32 * c : 0) + rowmap(r, g)];
      constexpr int RING = 3, AHEAD = 2;
      u32x4 fr[RING];
      static_for<AHEAD>([&](auto q) { fr[decltype(q)::value] = wb[decltype(q)::value * 64]; });
      static_for<KS>([&](auto S_) {
        constexpr int S = decltype(S_)::value;
        if constexpr (S + AHEAD < NF) fr[(S + AHEAD) % RING] = wb[(S + AHEAD) * 64];
        hacc = mma(fr[S % RING], ub[S], hacc);
        __builtin_amdgcn_sched_barrier(0);
        // second half of the activations of the chunk before: value S / 2 starts behind even steps, ends behind odd ones
        if constexpr (S % 2 == 0) begin(hrest[S / 2]);
        else finish(std::integral_constant<int, S / 2>{});
        if constexpr (S == 1) fetch(gs + 1, c < NCH ? c + 1 : 0);  // the other buffer was last read in the slot before
        __builtin_amdgcn_sched_barrier(0);
      });
      static_assert(KS == 16 && 2 * CT == 16, "eight activations per phase");
      gop[1] = gnew;  // k half 1 of the chunk before: its last reader was the last step of the slot before
      static_for<2 * CT>([&](auto t_) {
        constexpr int t = decltype(t_)::value, S = KS + t, kk = t / CT, ct = t % CT;
        if constexpr (S + AHEAD < NF) fr[(S + AHEAD) % RING] = wb[(S + AHEAD) * 64];
        yacc[ct] = mma(fr[S % RING], gop[kk], yacc[ct]);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (t % 2 == 0) begin(hacc[t / 2]);
        else finish(std::integral_constant<int, t / 2>{});
        __builtin_amdgcn_sched_barrier(0);
      });
      gop[0] = gnew;  // k half 0 of this chunk; that of the chunk before was last read by step CT - 1
#pragma unroll
      for (int j = 0; j < 8; ++j) hrest[j] = hacc[8 + j];
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's share of the next block's first slot has landed
    uint32_t *stg = stage + wave * (STG / 4);
    if constexpr (!OWN_STAGE) {  // the buffer of the last slot is idle once every wave is past its last MFMA
      __syncthreads();
      stg = reinterpret_cast<uint32_t *>(wbuf + ((gs - 1) & 1) * SU) + wave * (STG / 4);
    }
    finish_rows<C, HAS_RES, HAS_LN, STG>(yacc, stg, i, g, row0, M, residual, y, ln_out, gams, bets,
                                         ln_eps, [&]() { load_rows(mb + gridDim.x < nblocks ? mb + gridDim.x : mb, ub); });
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing may still be landing in LDS when the workgroup ends
}

// ---------------------------------------------------------------------------------------------------------------
// premlp_rows_kernel: the model's preprocess MLP, y = W2 . gelu(W1 . u + b1) + b2 [-> LayerNorm(y)], for rows with a
// handful of input features (c_in <= 16: coordinates, normals, fields) and 256 output channels per launch
// (transolver.py:518-525, and the first block's ln_1 at :300).  The hidden layer never reaches memory.
// Workgroup = 8 waves, two per SIMD, a block = 256 rows; a wave owns 32 rows:
//   u^T as ONE B operand (k = the c_in inputs, zero beyond), W1 whole in LDS as F / 32 A fragments, so a hidden chunk of
//   32 units costs one MFMA: h(c)^T = W1[chunk c] . u^T + b1;
//   y^T (256 channels x 32 rows, 128 registers) += W2[:, chunk c] . gelu(h(c))^T: 16 MFMAs per chunk, W2 streaming
//   through LDS in slots of 16 fragments (16 KB), two buffers, one barrier per slot.
// Software pipeline over the chunks, per iteration c: the first product of chunk c + 1 (its result is read an
// iteration later), the 16 MFMAs of the second product of chunk c - 1, and behind each of them one of the 16
// activations of chunk c (erf-accurate GELU, two evaluations in flight), which become the two B operands of the next
// iteration.  The activations (16 per 17 MFMAs) make the loop vector-bound; it still runs several times faster than
// two GEMM launches with the hidden layer in memory between them.
// blob (premlp_pack_kernel): W1 fragments [F / 32][lane]: W1[32 n + i][8 g + j] (zero beyond c_in); then per column
// block of 256 outputs the slots [F / 32][t = kk 8 + ct][lane]: W2[col0 + 32 ct + i][32 c + kperm(kk, g, j)].
// ---------------------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void premlp_pack_kernel(const uint16_t *__restrict__ w1, const uint16_t *__restrict__ w2,
                                                          u32x4 *__restrict__ blob, int c_in, int F, int C) {
  const int NCH = F / 32;
  const int64_t n1 = (int64_t)NCH * 64, total = n1 + (int64_t)(C / 256) * NCH * 16 * 64;
  for (int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x; u < total; u += (int64_t)gridDim.x * 256) {
    const int lane = (int)(u & 63), i = lane & 31, g = lane >> 5;
    uint16_t e[8];
    if (u < n1) {
      const int n = (int)(u >> 6);
#pragma unroll
      for (int j = 0; j < 8; ++j) e[j] = 8 * g + j < c_in ? w1[(int64_t)(32 * n + i) * c_in + 8 * g + j] : (uint16_t)0;
    } else {
      int64_t q = (u - n1) >> 6;
      const int t = (int)(q & 15);
      q >>= 4;
      const int c = (int)(q % NCH), blk = (int)(q / NCH), kk = t >> 3, ct = t & 7;
      const uint16_t *src = w2 + (int64_t)(256 * blk + 32 * ct + i) * F + 32 * c;
#pragma unroll
      for (int j = 0; j < 8; ++j) e[j] = src[kperm(kk, g, j)];
    }
    u32x4 v;
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = (uint32_t)e[2 * j] | ((uint32_t)e[2 * j + 1] << 16);
    blob[u] = v;
  }
}

// two direct global -> LDS loads of 64 x 16 bytes each (2 KB), as load_4k_to_lds
__device__ __forceinline__ void load_2k_to_lds(const void *sbase, unsigned lane16, unsigned lds) {
  asm volatile(
      "s_mov_b32 m0, %2\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %1, %0\n\t"
      "global_load_lds_dwordx4 %1, %0 offset:1024" ::"s"(sbase),
      "v"(lane16), "s"(lds)
      : "memory");
}

template <bool HAS_LN>
__global__ __launch_bounds__(512, 1) void premlp_rows_kernel(
    const u32x4 *__restrict__ blob, const float *__restrict__ b1, const float *__restrict__ b2,
    const uint16_t *__restrict__ u, int c_in, uint16_t *__restrict__ y, int64_t ld, const float *__restrict__ ln_gamma,
    const float *__restrict__ ln_beta, float ln_eps, uint16_t *__restrict__ ln_out, int64_t M, int F, int col_block,
    int64_t nblocks) {
  constexpr int C = 256, CT = 8, NF = 2 * CT, SU = NF * 64;  // a slot: 16 fragments
  constexpr int WU = SU / 8;                                  // units of a slot fetched by each wave (2 KB)
  constexpr int STG = 8192, kRows = 256;
  extern __shared__ u32x4 smem[];
  const int NCH = F / 32;
  u32x4 *w1s = smem;                    // NCH * 64
  u32x4 *wbuf = w1s + NCH * 64;         // 2 * SU
  uint32_t *stage = reinterpret_cast<uint32_t *>(wbuf + 2 * SU);  // 8 waves x STG bytes
  float *b1s = reinterpret_cast<float *>(stage + 8 * STG / 4);
  float *b2s = b1s + F;
  float *gams = b2s + C, *bets = gams + C;
  const int tid = threadIdx.x, lane = tid & 63, i = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const u32x4 *w2blob = blob + (int64_t)NCH * 64 + (int64_t)col_block * NCH * SU;
  for (int k = tid; k < NCH * 64; k += 512) w1s[k] = blob[k];
  for (int k = tid; k < F; k += 512) b1s[k] = b1[k];
  for (int k = tid; k < C; k += 512) {
    b2s[k] = b2[256 * col_block + k];
    gams[k] = HAS_LN ? ln_gamma[k] : 1.f;
    bets[k] = HAS_LN ? ln_beta[k] : 0.f;
  }
  auto fetch = [&](int64_t gs, int c) {  // this wave's share of slot c into buffer gs & 1
    const u32x4 *src = w2blob + (int64_t)c * SU + wave * WU;
    const unsigned dst = (unsigned)(uintptr_t)(wbuf + (gs & 1) * SU + wave * WU);
    load_2k_to_lds(src, lane * 16, dst);
  };
  // the wave's 32 rows as one B operand: lane (i, g) holds inputs 8 g .. 8 g + 7 of row i (zero beyond c_in)
  auto load_rows = [&](int64_t mb) {
    int64_t r = mb * kRows + wave * 32 + i;
    if (r >= M) r = M - 1;
    const uint16_t *src = u + r * c_in + 8 * g;
    uint16_t e[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) e[j] = 8 * g + j < c_in ? src[j] : (uint16_t)0;
    u32x4 v;
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = (uint32_t)e[2 * j] | ((uint32_t)e[2 * j + 1] << 16);
    return v;
  };
  int64_t gs = 0;
  if ((int64_t)blockIdx.x < nblocks) fetch(0, 0);
  __syncthreads();  // W1 and the biases are in LDS
  for (int64_t mb = blockIdx.x; mb < nblocks; mb += gridDim.x) {
    const int64_t row0 = mb * kRows + wave * 32;
    const u32x4 ub = load_rows(mb);
    f32x16 yacc[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
      for (int r = 0; r < 16; ++r) yacc[ct][r] = b2s[32 * ct + rowmap(r, g)];
    // h of the chunk being activated; the operands of the chunk before (zero before the first: its slot adds nothing)
    f32x16 hcur;
#pragma unroll
    for (int r = 0; r < 16; ++r) hcur[r] = b1s[rowmap(r, g)];
    hcur = mma(w1s[lane], ub, hcur);
    u32x4 gop[2] = {u32x4{0, 0, 0, 0}, u32x4{0, 0, 0, 0}};
    for (int c = 0; c <= NCH; ++c, ++gs) {
      // slot gs has landed (every wave waits for its own share, then all meet) and the other buffer is free.  The
      // first slot of a later block was waited for before the epilogue of the block before it.
      if (c > 0 || gs == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      // iteration c + 1 reads chunk c; the last iteration fetches the first slot of the next block (chunk 0, twice:
      // iteration 0 multiplies it by the zero operands)
      fetch(gs + 1, c < NCH ? c : 0);
      const u32x4 *wb = wbuf + (gs & 1) * SU + lane;
      // first product of chunk c + 1 (clamped past the end: computed, never used)
      const int cn = c + 1 < NCH ? c + 1 : NCH - 1;
      f32x16 hnext;
#pragma unroll
      for (int r = 0; r < 16; ++r) hnext[r] = b1s[32 * cn + rowmap(r, g)];
      hnext = mma(w1s[cn * 64 + lane], ub, hnext);
      u32x4 gnew[2];
      float ex = 0.f, ee = 0.f, feven = 0.f;  // evaluation in flight: argument and exp2 term; even result of a pair
      constexpr int RING = 3, AHEAD = 2;
      u32x4 fr[RING];
      static_for<AHEAD>([&](auto q) { fr[decltype(q)::value] = wb[decltype(q)::value * 64]; });
      __builtin_amdgcn_sched_barrier(0);
      static_for<NF>([&](auto t_) {
        constexpr int t = decltype(t_)::value, kk = t / CT, ct = t % CT;
        if constexpr (t + AHEAD < NF) fr[(t + AHEAD) % RING] = wb[(t + AHEAD) * 64];
        yacc[ct] = mma(fr[t % RING], gop[kk], yacc[ct]);
        __builtin_amdgcn_sched_barrier(0);
        // the end of activation t - 1 and the start of activation t: two independent chains behind the MFMA
        const float dx = ex, de = ee;
        {
          const float x = hcur[t];
          ex = x;
          const float x2 = fminf(x * x, 81.f);
          float q = fmaf(-3.51902394e-04f * -2.f * kLog2e, x2, 3.70080200e-02f * -2.f * kLog2e);
          q = fmaf(q, x2, 7.97505275e-01f * -2.f * kLog2e);
          ee = __builtin_amdgcn_exp2f(x * q);
        }
        if constexpr (t > 0) {
          constexpr int e = t - 1, j = e % 8;
          const float v = dx * __builtin_amdgcn_rcpf(1.f + de);
          if constexpr (j % 2 == 0) feven = v;
          else gnew[e / 8][j / 2] = pack2(feven, v);
        }
        __builtin_amdgcn_sched_barrier(0);
      });
      gnew[1][3] = pack2(feven, ex * __builtin_amdgcn_rcpf(1.f + ee));
      gop[0] = gnew[0];
      gop[1] = gnew[1];
      hcur = hnext;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's share of the next block's first slot has landed
    uint32_t *stg = stage + wave * (STG / 4);
    finish_rows<C, false, HAS_LN, STG>(yacc, stg, i, g, row0, M, nullptr, y, ln_out, gams, bets, ln_eps, [] {}, ld);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing may still be landing in LDS when the workgroup ends
}

// ---------------------------------------------------------------------------------------------------------------
// linear_rows_kernel: y = W x + b [+ residual] [-> LayerNorm(y)] for bf16 rows with C inputs and C outputs (the
// layer's out_linear with the block's residual and the following LayerNorm, transolver.py:296-300), on the skeleton
// of mlp_rows_kernel: a wave owns 32 rows (inputs as B operands, all C outputs of y^T in accumulation registers), W
// streams through LDS in slots of 64 fragments in consumption order (fragment j of slot c: output tile j % CT,
// k-step c (64 / CT) + j / CT), one barrier per slot, the epilogue above.
// ---------------------------------------------------------------------------------------------------------------
// head_order = 0: the reduction index of k-step ks runs over input channels 16 ks + 8 g + j (rows read in natural
// layout); 1: over 32 (ks / 2) + kperm(ks % 2, g, j) (rows read as the packed operand tiles the slice kernels write)
__global__ __launch_bounds__(256) void linear_pack_kernel(WeightView w, u32x4 *__restrict__ blob, int C, int head_order) {
  const int CT = C / 32, KPS = 64 / CT;
  const int64_t total = (int64_t)C * C / 8;
  for (int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x; u < total; u += (int64_t)gridDim.x * 256) {
    const int c = (int)(u >> 12), j = (int)(u & 4095) >> 6, lane = (int)(u & 63), i = lane & 31, g = lane >> 5;
    const int ct = j % CT, ks = c * KPS + j / CT;
    const int64_t row = 32 * ct + i;
    uint32_t e[4];
    if (!head_order) {
      weight_bits8(w, row, 16 * ks + 8 * g, e);
    } else {
#pragma unroll
      for (int q = 0; q < 4; ++q)
        e[q] = (uint32_t)weight_bits(w, row, 32 * (ks >> 1) + kperm(ks & 1, g, 2 * q)) |
               ((uint32_t)weight_bits(w, row, 32 * (ks >> 1) + kperm(ks & 1, g, 2 * q + 1)) << 16);
    }
    blob[u] = u32x4{e[0], e[1], e[2], e[3]};
  }
}

// PACKED_IN: the rows arrive as packed operand tiles, x = [tile][head][2][lane] of 16 bytes with tile = b tpb + t
// covering points 32 t .. 32 t + 31 of batch b (N points per batch, tpb tiles); a wave then owns one tile and a block
// four consecutive ones.  Otherwise x is (M, C) row-major and a block 128 consecutive rows (N, tpb unused).
template <int C, int TAIL, bool PACKED_IN>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void linear_rows_kernel(
    const u32x4 *__restrict__ blob, const float *__restrict__ bias, const uint16_t *__restrict__ x,
    uint16_t *__restrict__ y, const uint16_t *__restrict__ residual, const float *__restrict__ ln_gamma,
    const float *__restrict__ ln_beta, float ln_eps, uint16_t *__restrict__ ln_out, int64_t M, int64_t nblocks,
    int64_t N, int tpb) {
  constexpr bool HAS_RES = TAIL == 1 || TAIL == 2, HAS_LN = TAIL == 1 || TAIL == 3;
  constexpr int KS = C / 16, CT = C / 32, SU = 4096, WU = SU / 4;
  constexpr int NSLOT = CT * KS / 64, KPS = 64 / CT;
  static_assert(64 % CT == 0 && CT * KS % 64 == 0, "whole k-steps per slot");
  extern __shared__ u32x4 smem[];
  u32x4 *wbuf = smem;  // 2 * SU
  float *bs = reinterpret_cast<float *>(wbuf + 2 * SU);
  float *gams = bs + C, *bets = gams + C;
  const int tid = threadIdx.x, lane = tid & 63, i = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: addresses derived from it stay scalar
  for (int k = tid; k < C; k += 256) {
    bs[k] = bias ? bias[k] : 0.f;
    gams[k] = HAS_LN ? ln_gamma[k] : 1.f;
    bets[k] = HAS_LN ? ln_beta[k] : 0.f;
  }
  __syncthreads();
  auto fetch_group = [&](int64_t gs, int c, int k) {
    const u32x4 *src = blob + (int64_t)c * SU + wave * WU + k * 256;
    const unsigned dst = (unsigned)(uintptr_t)(wbuf + (gs & 1) * SU + wave * WU + k * 256);
    load_4k_to_lds(src, lane * 16, dst);
  };
  const int64_t ntiles = PACKED_IN ? M : 0;  // PACKED_IN: M counts tiles
  auto load_rows = [&](int64_t mb, u32x4(&ub)[KS]) {
    if constexpr (PACKED_IN) {
      int64_t gt = mb * 4 + wave;
      if (gt >= ntiles) gt = ntiles - 1;
      const u32x4 *src = reinterpret_cast<const u32x4 *>(x) + gt * (KS * 64) + lane;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) ub[ks] = load_streaming(src + ks * 64);
    } else {
      int64_t r = mb * kRowsPerBlock + wave * 32 + i;
      if (r >= M) r = M - 1;
      const uint16_t *src = x + r * C + 8 * g;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) ub[ks] = *reinterpret_cast<const u32x4 *>(src + 16 * ks);
    }
  };
  int64_t gs = 0;
  if ((int64_t)blockIdx.x < nblocks) {
#pragma unroll
    for (int k = 0; k < 4; ++k) fetch_group(0, 0, k);
  }
  u32x4 ub[KS];
  if ((int64_t)blockIdx.x < nblocks) load_rows(blockIdx.x, ub);
  for (int64_t mb = blockIdx.x; mb < nblocks; mb += gridDim.x) {
    // first row of this wave and the end of its valid rows
    int64_t row0 = mb * kRowsPerBlock + wave * 32, row_end = M;
    if constexpr (PACKED_IN) {
      const int64_t gt = mb * 4 + wave, bb = gt / tpb, t = gt - bb * tpb;
      row0 = bb * N + t * 32;
      row_end = gt < ntiles ? (bb + 1) * N : 0;  // tiles past the end own no rows
      if (gt >= ntiles) row0 = 0;
    }
    f32x16 yacc[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
      for (int r = 0; r < 16; ++r) yacc[ct][r] = bs[32 * ct + rowmap(r, g)];
    static_for<NSLOT>([&](auto c_) {
      constexpr int c = decltype(c_)::value;
      // slot gs has landed and the other buffer is free (the first slot of a later block was waited for before the
      // epilogue of the block before it, whose stores may still be in flight here)
      if (c > 0 || gs == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      const u32x4 *wb = wbuf + (gs & 1) * SU + lane;
      constexpr int RING = 8, AHEAD = 6;
      u32x4 fr[RING];
      static_for<AHEAD>([&](auto q) { fr[decltype(q)::value] = wb[decltype(q)::value * 64]; });
      static_for<64>([&](auto j_) {
        constexpr int j = decltype(j_)::value, ct = j % CT, ks = c * KPS + j / CT;
        if constexpr (j + AHEAD < 64) fr[(j + AHEAD) % RING] = wb[(j + AHEAD) * 64];
        yacc[ct] = mma(fr[j % RING], ub[ks], yacc[ct]);
        if constexpr (j % 16 == 7) fetch_group(gs + 1, (c + 1) % NSLOT, j / 16);
        __builtin_amdgcn_sched_barrier(0);
      });
      ++gs;
    });
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's share of the next block's first slot has landed
    __syncthreads();
    uint32_t *stg = reinterpret_cast<uint32_t *>(wbuf + ((gs - 1) & 1) * SU + wave * WU);  // this wave's 16 KB
    finish_rows<C, HAS_RES, HAS_LN>(yacc, stg, i, g, row0, row_end, residual, y, ln_out, gams, bets, ln_eps,
                                    [&]() { load_rows(mb + gridDim.x < nblocks ? mb + gridDim.x : mb, ub); });
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing may still be landing in LDS when the workgroup ends
}

// ---------------------------------------------------------------------------------------------------------------
// project_rows_kernel: the layer's two input projections (PA.py:501-514 for the irregular mesh), written as the packed
// operand tiles the slice kernels read.  Workgroup = 8 waves (two per SIMD), a block = 8 tiles of 32 points; a wave
// owns one tile (tile = b tpb + t), keeps its rows as MFMA operands (C/4 registers) and runs two products over them:
//   x_mid^T = W_x . x^T + b_x    weights as A, rows as B: lanes <-> points, registers <-> channels; the two packed
//                                halves of a head are B operands (columns = points, k = the head's channels, kperm order)
//   fx_mid  = x . W_fx^T + b_fx  rows as A, weights as B: lanes <-> channels, registers <-> points; the two packed
//                                halves of a head are A operands (rows = channels, k = points, kperm order)
// Output tiles are the outer loop: a slot of the weight stream (64 fragments, 64 KB) holds all C/16 k-steps of
// HPS = 1024 / C heads, interleaved so that the HPS accumulators take turns; when the slot is done the heads leave as
// 2 HPS stores of 1 KB per wave: out[((tile H + head) 2 + half) 64 + lane].  Only HPS accumulators are live, which is
// what lets two waves share a SIMD, and the stores are spread evenly over the kernel.
// blob: W_x then W_fx, each H / HPS slots in that order (project_pack_kernel).
// ---------------------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void project_pack_kernel(WeightView w, u32x4 *__restrict__ blob, int C) {
  const int KS = C / 16, HPS = 64 / KS;  // heads per slot
  const int64_t total = (int64_t)C * C / 8;
  for (int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x; u < total; u += (int64_t)gridDim.x * 256) {
    const int c = (int)(u >> 12), j = (int)(u & 4095) >> 6, lane = (int)(u & 63), i = lane & 31, g = lane >> 5;
    const int ct = HPS * c + j % HPS, ks = j / HPS;
    uint32_t e[4];
    weight_bits8(w, 32 * ct + i, 16 * ks + 8 * g, e);
    blob[u] = u32x4{e[0], e[1], e[2], e[3]};
  }
}

template <int C>
__global__ __launch_bounds__(512) void project_rows_kernel(
    const u32x4 *__restrict__ blob, const float *__restrict__ bias_x, const float *__restrict__ bias_fx,
    const uint16_t *__restrict__ x, u32x4 *__restrict__ xm_pack, u32x4 *__restrict__ fx_pack, int64_t N, int tpb,
    int64_t ntiles, int64_t nblocks) {
  constexpr int KS = C / 16, CT = C / 32, SU = 4096, WU = SU / 8;
  constexpr int HPS = 64 / KS;       // heads per slot (2 at C = 512, 4 at C = 256)
  constexpr int NSLOT = CT / HPS;    // slots per product
  static_assert(KS * HPS == 64 && CT % HPS == 0, "a slot holds all k-steps of HPS heads");
  extern __shared__ u32x4 smem[];
  u32x4 *wbuf = smem;  // 2 * SU
  float *bxs = reinterpret_cast<float *>(wbuf + 2 * SU);
  float *bfs = bxs + C;
  const int tid = threadIdx.x, lane = tid & 63, i = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: addresses derived from it stay scalar
  for (int k = tid; k < C; k += 512) {
    bxs[k] = bias_x ? bias_x[k] : 0.f;
    bfs[k] = bias_fx ? bias_fx[k] : 0.f;
  }
  __syncthreads();
  // 4 KB group k (0, 1) of this wave's eighth of slot c (0 .. 2 NSLOT - 1 over both products) into buffer gs & 1
  auto fetch_group = [&](int64_t gs, int c, int k) {
    const u32x4 *src = blob + (int64_t)c * SU + wave * WU + k * 256;
    const unsigned dst = (unsigned)(uintptr_t)(wbuf + (gs & 1) * SU + wave * WU + k * 256);
    load_4k_to_lds(src, lane * 16, dst);
  };
  // lane (i, g) holds point i of the wave's tile, channels 16 ks + 8 g .. + 7; points past the batch's end repeat
  // its last one (the slice kernels give them zero weight)
  auto load_rows = [&](int64_t mb, u32x4(&ub)[KS]) {
    int64_t gt = mb * 8 + wave;
    if (gt >= ntiles) gt = ntiles - 1;
    const int64_t bb = gt / tpb, t = gt - bb * tpb;
    int64_t n = t * 32 + i;
    if (n >= N) n = N - 1;
    const uint16_t *src = x + (bb * N + n) * C + 8 * g;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) ub[ks] = *reinterpret_cast<const u32x4 *>(src + 16 * ks);
  };
  int64_t gs = 0;
  if ((int64_t)blockIdx.x < nblocks) {
    fetch_group(0, 0, 0);
    fetch_group(0, 0, 1);
  }
  u32x4 ub[KS];
  for (int64_t mb = blockIdx.x; mb < nblocks; mb += gridDim.x) {
    const int64_t gt = mb * 8 + wave;
    const bool live = gt < ntiles;
    load_rows(mb, ub);
    for (int c = 0; c < 2 * NSLOT; ++c, ++gs) {
      const bool second = c >= NSLOT;          // the fx product
      const int ct0 = HPS * (c - (second ? NSLOT : 0));  // heads ct0 .. ct0 + HPS - 1
      // Slot gs has landed (every wave waits for its own share, then all meet) and the other buffer is free.  The
      // share was requested before the 2 HPS stores of the slot before: those may still be in flight.
      if (c == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      else if constexpr (HPS == 2) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
      else asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
      __syncthreads();
      const u32x4 *wb = wbuf + (gs & 1) * SU + lane;
      f32x16 acc[HPS];
#pragma unroll
      for (int q = 0; q < HPS; ++q)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[q][r] = second ? bfs[32 * (ct0 + q) + i] : bxs[32 * (ct0 + q) + rowmap(r, g)];
      constexpr int RING = 6, AHEAD = 4;
      u32x4 fr[RING];
      static_for<AHEAD>([&](auto q) { fr[decltype(q)::value] = wb[decltype(q)::value * 64]; });
      const int c_next = c + 1 < 2 * NSLOT ? c + 1 : 0;
      if (!second) {
        static_for<64>([&](auto j_) {
          constexpr int j = decltype(j_)::value;
          if constexpr (j + AHEAD < 64) fr[(j + AHEAD) % RING] = wb[(j + AHEAD) * 64];
          acc[j % HPS] = mma(fr[j % RING], ub[j / HPS], acc[j % HPS]);
          if constexpr (j == 1 || j == 9) fetch_group(gs + 1, c_next, j / 8);
          __builtin_amdgcn_sched_barrier(0);
        });
      } else {
        static_for<64>([&](auto j_) {
          constexpr int j = decltype(j_)::value;
          if constexpr (j + AHEAD < 64) fr[(j + AHEAD) % RING] = wb[(j + AHEAD) * 64];
          acc[j % HPS] = mma(ub[j / HPS], fr[j % RING], acc[j % HPS]);
          if constexpr (j == 1 || j == 9) fetch_group(gs + 1, c_next, j / 8);
          __builtin_amdgcn_sched_barrier(0);
        });
      }
      // exactly 2 HPS stores per slot and wave (see the wait above): tiles past the end rewrite the last one's
      u32x4 *dst = (second ? fx_pack : xm_pack) + ((live ? gt : ntiles - 1) * CT + ct0) * (2 * 64) + lane;
#pragma unroll
      for (int q = 0; q < HPS; ++q) {
        store_streaming(dst + (2 * q) * 64, pack_half<0>(acc[q]));
        store_streaming(dst + (2 * q + 1) * 64, pack_half<1>(acc[q]));
      }
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing may still be landing in LDS when the workgroup ends
}

// ---------------------------------------------------------------------------------------------------------------
// conv_project_rows_kernel: the two input projections of the structured-grid layers (k x k Conv2d / k x k x k Conv3d,
// stride 1, zero padding k / 2; PA.py:721-742, :857-867) as an implicit GEMM, written as the packed operand tiles the
// slice kernels read.  The skeleton is project_rows_kernel's: workgroup = 8 waves (two per SIMD), a block = 8 tiles of
// 32 points, a wave owns one tile.  The reduction runs over taps x channels in steps of one tap and 256 channels: for
// such a step the wave holds the rows of its points' neighbours at that tap as MFMA operands (64 registers; rows
// outside the grid are read from a row of zeros) and multiplies them with the step's weights for 256 outputs of one
// projection, whose 8 accumulators stay live over all steps: first x_mid^T = W_x . x^T (weights as A), then
// fx_mid = x . W_fx^T (weights as B), at 512 channels each in two passes of 256 outputs.  A register of the rows is
// reloaded for the next step right behind the last MFMA that read it, so the neighbour loads ride under a whole step
// of MFMAs.  Weights stream through LDS in slots of 64 fragments: slot (pass steps + step) 2 + hk holds k-steps
// 8 hk .. 8 hk + 7 of that step for the pass's 8 output tiles (fragment j: output tile j % 8, k-step j / 8).
// blob: the slots in that order, then 512 bytes of zeros (conv_pack_kernel).
// ---------------------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void conv_pack_kernel(WeightView wx, WeightView wfx, u32x4 *__restrict__ blob, int C,
                                                        int taps, int tap_major) {
  const int NCH = C / 256, steps = taps * NCH;  // reduction steps per pass; passes: 2 projections x NCH output halves
  const int64_t total = (int64_t)2 * NCH * steps * 2 * 4096;
  for (int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x; u < total + 32; u += (int64_t)gridDim.x * 256) {
    if (u >= total) {
      blob[u] = u32x4{0, 0, 0, 0};
      continue;
    }
    const int slot = (int)(u >> 12), j = (int)(u & 4095) >> 6, lane = (int)(u & 63), i = lane & 31, g = lane >> 5;
    const int pass = slot / (steps * 2), r = slot - pass * (steps * 2), step = r >> 1, hk = r & 1;
    const int proj = pass / NCH, oh = pass - proj * NCH, tap = step / NCH, ch = step - tap * NCH;
    const int ct = j % 8, ks = hk * 8 + j / 8;
    const WeightView w = proj ? wfx : wx;
    const int64_t row = 32 * (8 * oh + ct) + i;
    const int c0 = 256 * ch + 16 * ks + 8 * g;
    uint32_t e[4];
    if (tap_major) {
      weight_bits8(w, row, (int64_t)tap * C + c0, e);
    } else {
#pragma unroll
      for (int q = 0; q < 4; ++q)
        e[q] = (uint32_t)weight_bits(w, row, (int64_t)(c0 + 2 * q) * taps + tap) |
               ((uint32_t)weight_bits(w, row, (int64_t)(c0 + 2 * q + 1) * taps + tap) << 16);
    }
    blob[u] = u32x4{e[0], e[1], e[2], e[3]};
  }
}

template <int C>
__global__ __launch_bounds__(512) void conv_project_rows_kernel(
    const u32x4 *__restrict__ blob, const float *__restrict__ bias_x, const float *__restrict__ bias_fx,
    const uint16_t *__restrict__ x, u32x4 *__restrict__ xm_pack, u32x4 *__restrict__ fx_pack, int64_t N, int tpb,
    int64_t ntiles, int64_t nblocks, int gh, int gw, int gd, int ksz) {
  constexpr int KS = 16, CTB = 8, SU = 4096, WU = SU / 8;  // k-steps and output tiles of a step, slot and wave share
  constexpr int NCH = C / 256;   // 256-channel chunks of the input = output halves of a projection
  constexpr int CT = C / 32;     // output tiles of a projection
  static_assert(C % 256 == 0, "steps of 256 channels");
  extern __shared__ u32x4 smem[];
  u32x4 *wbuf = smem;  // 2 * SU
  float *bxs = reinterpret_cast<float *>(wbuf + 2 * SU);
  float *bfs = bxs + C;
  const int tid = threadIdx.x, lane = tid & 63, i = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: addresses derived from it stay scalar
  for (int k = tid; k < C; k += 512) {
    bxs[k] = bias_x ? bias_x[k] : 0.f;
    bfs[k] = bias_fx ? bias_fx[k] : 0.f;
  }
  __syncthreads();
  const int gdd = gd > 0 ? gd : 1, ksd = gd > 0 ? ksz : 1, pad = ksz / 2;
  const int taps = ksz * ksz * ksd, steps = taps * NCH;
  const int nslots = 2 * NCH * steps * 2;  // per block
  const uint16_t *zero_row = reinterpret_cast<const uint16_t *>(blob + (int64_t)nslots * SU) + 8 * g;
  auto fetch_group = [&](int64_t gs, int c, int k) {
    const u32x4 *src = blob + (int64_t)c * SU + wave * WU + k * 256;
    const unsigned dst = (unsigned)(uintptr_t)(wbuf + (gs & 1) * SU + wave * WU + k * 256);
    load_4k_to_lds(src, lane * 16, dst);
  };
  // this lane's point of the wave's tile in block mb: batch base and grid coordinates
  const uint16_t *xb = x;
  int ci = 0, cj = 0, cl = 0;
  auto locate = [&](int64_t mb) {
    int64_t gt = mb * 8 + wave;
    if (gt >= ntiles) gt = ntiles - 1;
    const int64_t bb = gt / tpb, t = gt - bb * tpb;
    int64_t n = t * 32 + i;
    if (n >= N) n = N - 1;  // points past the batch's end repeat its last one (the slice kernels give them zero weight)
    xb = x + bb * N * C + 8 * g;
    int nn = (int)n;
    cl = nn % gdd;
    nn /= gdd;
    ci = nn / gw;
    cj = nn - ci * gw;
  };
  // where this lane's operand rows of reduction step `step` start (its 16-byte piece of k-step 0 of the step's 256
  // channels of the neighbour at the step's tap), or the row of zeros outside the grid
  auto step_row = [&](int step) -> const uint16_t * {
    const int tap = step / NCH, ch = step - tap * NCH;
    const int uv = tap / ksd, zz = tap - uv * ksd, u = uv / ksz, v = uv - u * ksz;
    const int ii = ci + u - pad, jj = cj + v - pad, ll = cl + (gd > 0 ? zz - pad : 0);
    const bool ok = ii >= 0 && ii < gh && jj >= 0 && jj < gw && ll >= 0 && ll < gdd;
    return ok ? xb + (((int64_t)ii * gw + jj) * gdd + ll) * C + 256 * ch : zero_row;
  };
  int64_t gs = 0;
  u32x4 ub[KS];
  if ((int64_t)blockIdx.x < nblocks) {
    fetch_group(0, 0, 0);
    fetch_group(0, 0, 1);
    locate(blockIdx.x);
    const uint16_t *r0 = step_row(0);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) ub[ks] = *reinterpret_cast<const u32x4 *>(r0 + 16 * ks);
  }
  for (int64_t mb = blockIdx.x; mb < nblocks; mb += gridDim.x) {
    const int64_t gt = mb * 8 + wave;
    const int64_t gto = gt < ntiles ? gt : ntiles - 1;  // tiles past the end rewrite the last one's results
    static_for<2 * NCH>([&](auto p_) {
      constexpr int p = decltype(p_)::value;
      constexpr int proj = p / NCH;  // 0: x_mid^T (weights as A), 1: fx_mid (weights as B)
      constexpr int oh = p % NCH;    // which 256 outputs
      f32x16 acc[CTB];
#pragma unroll
      for (int ct = 0; ct < CTB; ++ct)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          acc[ct][r] = proj ? bfs[32 * (CTB * oh + ct) + i] : bxs[32 * (CTB * oh + ct) + rowmap(r, g)];
      for (int step = 0; step < steps; ++step) {
        // the rows the registers are refilled with while this step is multiplied: the next step's, the first step's
        // again for the next pass, the first step of the wave's tile in the workgroup's next block after the last pass
        const uint16_t *nxt;
        if (step + 1 < steps) {
          nxt = step_row(step + 1);
        } else {
          if (p == 2 * NCH - 1) locate(mb + gridDim.x < nblocks ? mb + gridDim.x : mb);
          nxt = step_row(0);
        }
        static_for<2>([&](auto hk_) {
          constexpr int hk = decltype(hk_)::value;
          const int c = (p * steps + step) * 2 + hk;
          // Slot gs has landed (every wave waits for its own share, then all meet) and the other buffer is free.  Its
          // share was requested before the 7 row reloads that closed the slot before (and, at a pass's start, before
          // the 2 x 8 stores of the pass before): those may still be in flight.
          if (gs == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
          else if (step == 0 && hk == 0) asm volatile("s_waitcnt vmcnt(23)" ::: "memory");
          else asm volatile("s_waitcnt vmcnt(7)" ::: "memory");
          __syncthreads();
          const u32x4 *wb = wbuf + (gs & 1) * SU + lane;
          constexpr int RING = 6, AHEAD = 4;
          u32x4 fr[RING];
          static_for<AHEAD>([&](auto q) { fr[decltype(q)::value] = wb[decltype(q)::value * 64]; });
          const int c_next = c + 1 < nslots ? c + 1 : 0;
          static_for<64>([&](auto j_) {
            constexpr int j = decltype(j_)::value, ct = j % CTB, ks = hk * 8 + j / CTB;
            if constexpr (j + AHEAD < 64) fr[(j + AHEAD) % RING] = wb[(j + AHEAD) * 64];
            if constexpr (proj == 0) acc[ct] = mma(fr[j % RING], ub[ks], acc[ct]);
            else acc[ct] = mma(ub[ks], fr[j % RING], acc[ct]);
            if constexpr (j == 1 || j == 9) fetch_group(gs + 1, c_next, j / 8);
            if constexpr (ct == CTB - 1) ub[ks] = *reinterpret_cast<const u32x4 *>(nxt + 16 * ks);
            __builtin_amdgcn_sched_barrier(0);
          });
          ++gs;
        });
      }
      u32x4 *dst = (proj ? fx_pack : xm_pack) + (gto * CT + CTB * oh) * (2 * 64) + lane;
#pragma unroll
      for (int ct = 0; ct < CTB; ++ct) {
        store_streaming(dst + (2 * ct) * 64, pack_half<0>(acc[ct]));
        store_streaming(dst + (2 * ct + 1) * 64, pack_half<1>(acc[ct]));
      }
    });
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing may still be landing in LDS when the workgroup ends
}

}  // namespace rows

// ---------------------------------------------------------------------------------------------------------------
// C = 512 runs the row-owning kernel with one wave per SIMD, C = 256 the one with two, C = 128 the paired kernel
static bool use_rows_kernel(int64_t C) { return C == 512; }
static bool use_rows2_kernel(int64_t C) { return C == 256; }

// dynamic LDS of the kernel that serves (C, F): two weight buffers, staging / exchange areas, biases and LayerNorm vectors
static size_t lds_need(int64_t C, int64_t F) {
  if (use_rows_kernel(C)) return (size_t)2 * 4096 * 16 + (size_t)(F + 5 * C) * 4;
  if (use_rows2_kernel(C)) return (size_t)2 * (C / 16 + 2 * (C / 32)) * 64 * 16 + 8 * 8192 + (size_t)(F + 5 * C) * 4;
  return (size_t)(2 * slot_units((int)C) + 4 * 4 * 64) * 16 + (size_t)(F + C) * 4;
}

bool supported(int dtype, int64_t rows, int64_t C, int64_t F) {
  if (dtype != PA_BF16 || rows <= 0 || F < 64 || F % 64 != 0 || F > 8192) return false;
  if (C != 128 && C != 256 && C != 512) return false;
  return lds_need(C, F) <= (size_t)kMaxLdsBytes;
}

int64_t blob_bytes(int64_t C, int64_t F) {
  if (use_rows_kernel(C)) return (F / (16384 / C) + 2) * (int64_t)4096 * 16;
  if (use_rows2_kernel(C)) return (F / 32 + 1) * (int64_t)(C / 16 + 2 * (C / 32)) * 64 * 16;
  return (F / 64 + 1) * (int64_t)slot_units((int)C) * 16;
}


// w1_scale / w2_scale: nullptr for bf16 weights; else w1 / w2 are fp8-e4m3 bytes with one scale per output row
int pack(int64_t C, int64_t F, const void *w1, const float *w1_scale, const void *w2, const float *w2_scale, void *blob,
         hipStream_t st) {
  const WeightView v1{w1, w1_scale, C}, v2{w2, w2_scale, F};
  const bool by_rows = use_rows_kernel(C), by_rows2 = use_rows2_kernel(C);
  const int64_t total = by_rows    ? (F / (16384 / C) + 2) * (int64_t)4096
                        : by_rows2 ? (F / 32 + 1) * (int64_t)(C / 16 + 2 * (C / 32)) * 64
                                   : (F / 64 + 1) * (int64_t)slot_units((int)C);
  const int grid = (int)((total + 255) / 256 < 1024 ? (total + 255) / 256 : 1024);
  if (by_rows2)
    hipLaunchKernelGGL(rows::pack2_kernel, dim3(grid), dim3(256), 0, st, v1, v2, static_cast<u32x4 *>(blob), (int)C, (int)F);
  else if (by_rows)
    hipLaunchKernelGGL(rows::pack_kernel, dim3(grid), dim3(256), 0, st, v1, v2, static_cast<u32x4 *>(blob), (int)C, (int)F);
  else
    hipLaunchKernelGGL(pack_kernel, dim3(grid), dim3(256), 0, st, v1, v2, static_cast<u32x4 *>(blob), (int)C, (int)F);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? PA_OK : (int)e;
}

template <int C, int TAIL>
static int launch_rows(int64_t rows, int F, const void *blob, const float *b1, const float *b2, const void *u, void *y,
                       const pa_block_tail *tail, const InputLn &in, int num_cu, hipStream_t st) {
  const size_t lds = lds_need(C, F);
  if (lds > kMaxLdsBytes) return PA_ERR_UNSUPPORTED;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(rows::mlp_rows_kernel<C, TAIL>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return (int)e;
  const int64_t nblocks = (rows + kRowsPerBlock - 1) / kRowsPerBlock;
  const int64_t grid = nblocks < num_cu ? nblocks : num_cu;
  hipLaunchKernelGGL((rows::mlp_rows_kernel<C, TAIL>), dim3((unsigned)grid), dim3(256), lds, st,
                     static_cast<const u32x4 *>(blob), b1, b2, static_cast<const uint16_t *>(u),
                     static_cast<uint16_t *>(y), tail ? static_cast<const uint16_t *>(tail->residual) : nullptr,
                     tail ? tail->ln_gamma : nullptr, tail ? tail->ln_beta : nullptr, tail ? tail->ln_eps : 0.f,
                     tail ? static_cast<uint16_t *>(tail->ln_out) : nullptr, rows, F, nblocks, in.gamma, in.beta, in.eps);
  e = hipGetLastError();
  return e == hipSuccess ? PA_OK : (int)e;
}

template <int C, int TAIL>
static int launch_rows2(int64_t rows, int F, const void *blob, const float *b1, const float *b2, const void *u, void *y,
                        const pa_block_tail *tail, const InputLn &in, int num_cu, hipStream_t st) {
  constexpr int WAVES = 8;  // one workgroup per CU; 4 (two per CU, own weight streams) measured 2 % slower
  const size_t lds = lds_need(C, F);  // sized for WAVES = 8 (own staging region)
  if (lds > kMaxLdsBytes) return PA_ERR_UNSUPPORTED;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(rows::mlp_rows2_kernel<C, TAIL, WAVES>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return (int)e;
  const int64_t nblocks = (rows + 32 * WAVES - 1) / (32 * WAVES);
  const int64_t resident = (int64_t)num_cu * (8 / WAVES);
  const int64_t grid = nblocks < resident ? nblocks : resident;
  hipLaunchKernelGGL((rows::mlp_rows2_kernel<C, TAIL, WAVES>), dim3((unsigned)grid), dim3(64 * WAVES), lds, st,
                     static_cast<const u32x4 *>(blob), b1, b2, static_cast<const uint16_t *>(u),
                     static_cast<uint16_t *>(y), tail ? static_cast<const uint16_t *>(tail->residual) : nullptr,
                     tail ? tail->ln_gamma : nullptr, tail ? tail->ln_beta : nullptr, tail ? tail->ln_eps : 0.f,
                     tail ? static_cast<uint16_t *>(tail->ln_out) : nullptr, rows, F, nblocks, in.gamma, in.beta, in.eps);
  e = hipGetLastError();
  return e == hipSuccess ? PA_OK : (int)e;
}

template <int C>
static int launch_rows2_c(int64_t rows, int F, const void *blob, const float *b1, const float *b2, const void *u, void *y,
                          const pa_block_tail *tail, const InputLn &in, int num_cu, hipStream_t st) {
  const bool res = tail && tail->residual, ln = tail && tail->ln_out;
  if (res && ln) return launch_rows2<C, 1>(rows, F, blob, b1, b2, u, y, tail, in, num_cu, st);
  if (res) return launch_rows2<C, 2>(rows, F, blob, b1, b2, u, y, tail, in, num_cu, st);
  if (ln) return launch_rows2<C, 3>(rows, F, blob, b1, b2, u, y, tail, in, num_cu, st);
  return launch_rows2<C, 0>(rows, F, blob, b1, b2, u, y, nullptr, in, num_cu, st);
}

template <int C>
static int launch_rows_c(int64_t rows, int F, const void *blob, const float *b1, const float *b2, const void *u, void *y,
                         const pa_block_tail *tail, const InputLn &in, int num_cu, hipStream_t st) {
  const bool res = tail && tail->residual, ln = tail && tail->ln_out;
  if (res && ln) return launch_rows<C, 1>(rows, F, blob, b1, b2, u, y, tail, in, num_cu, st);
  if (res) return launch_rows<C, 2>(rows, F, blob, b1, b2, u, y, tail, in, num_cu, st);
  if (ln) return launch_rows<C, 3>(rows, F, blob, b1, b2, u, y, tail, in, num_cu, st);
  return launch_rows<C, 0>(rows, F, blob, b1, b2, u, y, nullptr, in, num_cu, st);
}

template <int C, int TAIL>
static int launch(int64_t rows, int F, const void *blob, const float *b1, const float *b2, const void *u, void *y,
                  const pa_block_tail *tail, int num_cu, hipStream_t st) {
  const size_t lds = lds_need(C, F);
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

// ---- out_linear with the block's tail on the row-owning kernel --------------------------------------------------
bool linear_supported(int dtype, int64_t rows, int64_t C) {
  return dtype == PA_BF16 && rows > 0 && (C == 512 || C == 256);
}

int64_t linear_blob_bytes(int64_t C) { return C * C * 2; }

template <int C, int TAIL, bool PACKED_IN>
static int launch_linear(int64_t rows, const void *blob, const float *bias, const void *x, void *y,
                         const pa_block_tail *tail, int64_t N, int tpb, int num_cu, hipStream_t st) {
  const size_t lds = (size_t)2 * 4096 * 16 + (size_t)3 * C * 4;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(rows::linear_rows_kernel<C, TAIL, PACKED_IN>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return (int)e;
  // PACKED_IN: `rows` counts tiles of 32 points, four to a block
  const int64_t nblocks = PACKED_IN ? (rows + 3) / 4 : (rows + kRowsPerBlock - 1) / kRowsPerBlock;
  const int64_t grid = nblocks < num_cu ? nblocks : num_cu;
  hipLaunchKernelGGL((rows::linear_rows_kernel<C, TAIL, PACKED_IN>), dim3((unsigned)grid), dim3(256), lds, st,
                     static_cast<const u32x4 *>(blob), bias, static_cast<const uint16_t *>(x),
                     static_cast<uint16_t *>(y), tail ? static_cast<const uint16_t *>(tail->residual) : nullptr,
                     tail ? tail->ln_gamma : nullptr, tail ? tail->ln_beta : nullptr, tail ? tail->ln_eps : 0.f,
                     tail ? static_cast<uint16_t *>(tail->ln_out) : nullptr, rows, nblocks, N, tpb);
  e = hipGetLastError();
  return e == hipSuccess ? PA_OK : (int)e;
}

template <int C, bool PACKED_IN>
static int linear_c(int64_t rows, const void *blob, const float *bias, const void *x, void *y, const pa_block_tail *tail,
                    int64_t N, int tpb, int num_cu, hipStream_t st) {
  const bool res = tail && tail->residual, ln = tail && tail->ln_out;
  if (res && ln) return launch_linear<C, 1, PACKED_IN>(rows, blob, bias, x, y, tail, N, tpb, num_cu, st);
  if (res) return launch_linear<C, 2, PACKED_IN>(rows, blob, bias, x, y, tail, N, tpb, num_cu, st);
  if (ln) return launch_linear<C, 3, PACKED_IN>(rows, blob, bias, x, y, tail, N, tpb, num_cu, st);
  return launch_linear<C, 0, PACKED_IN>(rows, blob, bias, x, y, nullptr, N, tpb, num_cu, st);
}

template <bool PACKED_IN>
static int linear_any(int64_t rows, int64_t C, const void *w, const float *w_scale, const float *bias, const void *x,
                      void *y, const pa_block_tail *tail, void *blob, int64_t N, int tpb, int num_cu, hipStream_t st) {
  if (C != 512 && C != 256) return PA_ERR_UNSUPPORTED;
  const int64_t total = C * C / 8;
  hipLaunchKernelGGL(rows::linear_pack_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st,
                     WeightView{w, w_scale, C}, static_cast<u32x4 *>(blob), (int)C, PACKED_IN ? 1 : 0);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return (int)e;
  if (C == 512) return linear_c<512, PACKED_IN>(rows, blob, bias, x, y, tail, N, tpb, num_cu, st);
  return linear_c<256, PACKED_IN>(rows, blob, bias, x, y, tail, N, tpb, num_cu, st);
}

// y = W x + bias (+ tail) for (rows, C) row-major x; `blob` = linear_blob_bytes(C) bytes of scratch for the
// fragment-ordered weights.  w_scale: nullptr for a bf16 W, else W is fp8-e4m3 bytes with one scale per output row.
int linear(int64_t rows, int64_t C, const void *w, const float *w_scale, const float *bias, const void *x, void *y,
           const pa_block_tail *tail, void *blob, int num_cu, hipStream_t st) {
  return linear_any<false>(rows, C, w, w_scale, bias, x, y, tail, blob, 0, 1, num_cu, st);
}

// the same with x as packed operand tiles [B tpb][C / 32][2][64 lanes] of 16 bytes (tile b tpb + t = points
// 32 t .. 32 t + 31 of batch b, k order kperm within a head); y and the tail tensors stay (B, N, C) row-major
int linear_packed(int64_t B, int64_t N, int64_t C, const void *w, const float *w_scale, const float *bias,
                  const void *x_pack, void *y, const pa_block_tail *tail, void *blob, int num_cu, hipStream_t st) {
  const int64_t tpb = (N + 31) / 32;
  return linear_any<true>(B * tpb, C, w, w_scale, bias, x_pack, y, tail, blob, N, (int)tpb, num_cu, st);
}

// the layer's two input projections as packed operand tiles (x_mid: B operands, fx_mid: A operands); `blob` =
// 2 linear_blob_bytes(C) bytes of scratch.  s_x / s_fx: nullptr for bf16 weights, else per-row scales of e4m3 weights.
int project_packed(int64_t B, int64_t N, int64_t C, const void *w_x, const float *s_x, const float *b_x, const void *w_fx,
                   const float *s_fx, const float *b_fx, const void *x, void *xm_pack, void *fx_pack, void *blob,
                   int num_cu, hipStream_t st) {
  if (C != 512 && C != 256) return PA_ERR_UNSUPPORTED;
  const int64_t total = C * C / 8;
  u32x4 *bl = static_cast<u32x4 *>(blob);
  hipLaunchKernelGGL(rows::project_pack_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st,
                     WeightView{w_x, s_x, C}, bl, (int)C);
  hipLaunchKernelGGL(rows::project_pack_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st,
                     WeightView{w_fx, s_fx, C}, bl + total, (int)C);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return (int)e;
  const size_t lds = (size_t)2 * 4096 * 16 + (size_t)2 * C * 4;
  const void *kernel = C == 512 ? reinterpret_cast<const void *>(rows::project_rows_kernel<512>)
                                : reinterpret_cast<const void *>(rows::project_rows_kernel<256>);
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return (int)e;
  const int64_t tpb = (N + 31) / 32, ntiles = B * tpb, nblocks = (ntiles + 7) / 8;
  const int64_t grid = nblocks < num_cu ? nblocks : num_cu;
  if (C == 512)
    hipLaunchKernelGGL((rows::project_rows_kernel<512>), dim3((unsigned)grid), dim3(512), lds, st, bl, b_x, b_fx,
                       static_cast<const uint16_t *>(x), static_cast<u32x4 *>(xm_pack), static_cast<u32x4 *>(fx_pack),
                       N, (int)tpb, ntiles, nblocks);
  else
    hipLaunchKernelGGL((rows::project_rows_kernel<256>), dim3((unsigned)grid), dim3(512), lds, st, bl, b_x, b_fx,
                       static_cast<const uint16_t *>(x), static_cast<u32x4 *>(xm_pack), static_cast<u32x4 *>(fx_pack),
                       N, (int)tpb, ntiles, nblocks);
  e = hipGetLastError();
  return e == hipSuccess ? PA_OK : (int)e;
}

// the same for the grid convolutions of the structured layers (conv_project_rows_kernel); weights (H*32, C, k, ..) in
// torch's layout or tap-major (H*32, k, .., C); `blob` = conv_project_blob_bytes(C, taps) bytes of scratch
bool conv_project_supported(int dtype, int64_t B, int64_t N, int64_t C) {
  return dtype == PA_BF16 && (C == 256 || C == 512) && B > 0 && N > 0 && N * C * 2 < ((int64_t)1 << 40);
}

int64_t conv_project_blob_bytes(int64_t C, int64_t taps) { return 2 * taps * C * C * 2 + 512; }

int conv_project_packed(int64_t B, int64_t N, int64_t C, int64_t gh, int64_t gw, int64_t gd, int64_t k, int tap_major,
                        const void *w_x, const float *b_x, const void *w_fx, const float *b_fx, const void *x,
                        void *xm_pack, void *fx_pack, void *blob, int num_cu, hipStream_t st) {
  if ((C != 256 && C != 512) || k <= 0 || k % 2 == 0 || gh <= 0 || gw <= 0 || gd < 0) return PA_ERR_UNSUPPORTED;
  if (gh * gw * (gd > 0 ? gd : 1) != N) return PA_ERR_DIMS;
  const int64_t taps = k * k * (gd > 0 ? k : 1);
  const int64_t units = 2 * taps * C * C / 8 + 32;
  u32x4 *bl = static_cast<u32x4 *>(blob);
  const int64_t pgrid = (units + 255) / 256 < 2048 ? (units + 255) / 256 : 2048;
  hipLaunchKernelGGL(rows::conv_pack_kernel, dim3((unsigned)pgrid), dim3(256), 0, st,
                     WeightView{w_x, nullptr, taps * C}, WeightView{w_fx, nullptr, taps * C}, bl, (int)C, (int)taps,
                     tap_major);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return (int)e;
  const size_t lds = (size_t)2 * 4096 * 16 + (size_t)2 * C * 4;
  const void *kernel = C == 512 ? reinterpret_cast<const void *>(rows::conv_project_rows_kernel<512>)
                                : reinterpret_cast<const void *>(rows::conv_project_rows_kernel<256>);
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return (int)e;
  const int64_t tpb = (N + 31) / 32, ntiles = B * tpb, nblocks = (ntiles + 7) / 8;
  const int64_t grid = nblocks < num_cu ? nblocks : num_cu;
  if (C == 512)
    hipLaunchKernelGGL((rows::conv_project_rows_kernel<512>), dim3((unsigned)grid), dim3(512), lds, st, bl, b_x, b_fx,
                       static_cast<const uint16_t *>(x), static_cast<u32x4 *>(xm_pack), static_cast<u32x4 *>(fx_pack),
                       N, (int)tpb, ntiles, nblocks, (int)gh, (int)gw, (int)gd, (int)k);
  else
    hipLaunchKernelGGL((rows::conv_project_rows_kernel<256>), dim3((unsigned)grid), dim3(512), lds, st, bl, b_x, b_fx,
                       static_cast<const uint16_t *>(x), static_cast<u32x4 *>(xm_pack), static_cast<u32x4 *>(fx_pack),
                       N, (int)tpb, ntiles, nblocks, (int)gh, (int)gw, (int)gd, (int)k);
  e = hipGetLastError();
  return e == hipSuccess ? PA_OK : (int)e;
}

// ---- the preprocess MLP (few inputs -> F -> C) on premlp_rows_kernel ---------------------------------------------
static size_t premlp_lds(int64_t F) {
  return (size_t)((F / 32) * 64 + 2 * 16 * 64) * 16 + (size_t)8 * 8192 + (size_t)(F + 3 * 256) * 4;
}

bool premlp_supported(int dtype, int64_t rows, int64_t c_in, int64_t F, int64_t C) {
  if (dtype != PA_BF16 || rows <= 0 || c_in < 1 || c_in > 16 || F < 32 || F % 32 != 0 || F > 4096) return false;
  if (C != 256 && C != 512) return false;
  return premlp_lds(F) <= (size_t)kMaxLdsBytes;
}

int64_t premlp_blob_bytes(int64_t F, int64_t C) { return ((F / 32) * 64 + (C / 256) * (F / 32) * 16 * 64) * (int64_t)16; }

// y (rows, C) = W2 gelu(W1 u + b1) + b2 for u (rows, c_in); with ln_out (C = 256 only): ln_out = LayerNorm(y) too.
// C = 512 runs as two column blocks of 256 outputs (the hidden layer is evaluated once per block).
int premlp(int64_t rows, int64_t c_in, int64_t F, int64_t C, const void *w1, const float *b1, const void *w2,
           const float *b2, const void *u, void *y, const float *ln_gamma, const float *ln_beta, float ln_eps,
           void *ln_out, void *blob, int num_cu, hipStream_t st) {
  if (!premlp_supported(PA_BF16, rows, c_in, F, C)) return PA_ERR_UNSUPPORTED;
  if (ln_out && C != 256) return PA_ERR_UNSUPPORTED;
  const int64_t total = premlp_blob_bytes(F, C) / 16;
  hipLaunchKernelGGL(rows::premlp_pack_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st,
                     static_cast<const uint16_t *>(w1), static_cast<const uint16_t *>(w2), static_cast<u32x4 *>(blob),
                     (int)c_in, (int)F, (int)C);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return (int)e;
  const size_t lds = premlp_lds(F);
  const void *kernel = ln_out ? reinterpret_cast<const void *>(rows::premlp_rows_kernel<true>)
                              : reinterpret_cast<const void *>(rows::premlp_rows_kernel<false>);
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return (int)e;
  const int64_t nblocks = (rows + 255) / 256;
  const int64_t grid = nblocks < num_cu ? nblocks : num_cu;
  for (int blk = 0; blk < (int)(C / 256); ++blk) {
    uint16_t *yb = static_cast<uint16_t *>(y) + 256 * blk;
    if (ln_out)
      hipLaunchKernelGGL(rows::premlp_rows_kernel<true>, dim3((unsigned)grid), dim3(512), lds, st,
                         static_cast<const u32x4 *>(blob), b1, b2, static_cast<const uint16_t *>(u), (int)c_in, yb, C,
                         ln_gamma, ln_beta, ln_eps, static_cast<uint16_t *>(ln_out), rows, (int)F, blk, nblocks);
    else
      hipLaunchKernelGGL(rows::premlp_rows_kernel<false>, dim3((unsigned)grid), dim3(512), lds, st,
                         static_cast<const u32x4 *>(blob), b1, b2, static_cast<const uint16_t *>(u), (int)c_in, yb, C,
                         nullptr, nullptr, 0.f, nullptr, rows, (int)F, blk, nblocks);
    e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
  }
  return PA_OK;
}

// in.gamma != nullptr: LayerNorm(in) is applied to the rows of u on their way in (C = 256 and 512 only)
bool input_ln_supported(int dtype, int64_t rows, int64_t C, int64_t F) {
  return supported(dtype, rows, C, F) && (C == 256 || C == 512);
}

int forward(int64_t rows, int64_t C, int64_t F, const void *blob, const float *b1, const float *b2, const void *u,
            void *y, const pa_block_tail *tail, const InputLn &in, int num_cu, hipStream_t st) {
  if (C == 512) return launch_rows_c<512>(rows, (int)F, blob, b1, b2, u, y, tail, in, num_cu, st);
  if (C == 256) return launch_rows2_c<256>(rows, (int)F, blob, b1, b2, u, y, tail, in, num_cu, st);
  if (in.gamma) return PA_ERR_UNSUPPORTED;
  if (C == 128) return launch_c<128>(rows, (int)F, blob, b1, b2, u, y, tail, num_cu, st);
  return PA_ERR_UNSUPPORTED;
}

}  // namespace mlp
}  // namespace pa
