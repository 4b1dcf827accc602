// Float32 per-point kernels of a 128-wide block, on split-bf16 products (pa_split_ops.h):
//   deslice_linear_kernel  the layer's way back to the points (PA.py:467-499): out_x = w . out_token per head,
//                          y = out_x W_out^T + b_out, then the caller's residual and LayerNorm (TR.py:300-303)
//   mlp_kernel             the block's MLP (mlp_layers.py:139-173, TR.py:301-307): y = W2 gelu(W1 u + b1) + b2 with the
//                          same tail
// Shape class: C = 128 channels (8 heads of 16, 32 slices for the hand-back), F a multiple of 128.
//
// Workgroup = 4 waves, a wave owns a tile of 32 rows and keeps every intermediate transposed: lane (i, g) <-> row i,
// accumulator register r of column tile t <-> channel 32 t + rowmap(r, g).  A product Y^T = W X^T takes the weight as
// the A operand and the rows as the B operand; the result, cut into bf16 pieces, is the B operand of the next product
// provided that product's weight is packed with its reduction index in the order the registers hold the channels
// (kperm).  So deslice -> out_linear and Linear -> GELU -> Linear run without the rows leaving the registers, and the
// residual + LayerNorm tail is a sum over a lane's 64 registers and its partner lane.
//
// Weights are cut into pieces once (pack kernels) as units of 12 KB = one k-step (16 reduction indices) of 128 output
// rows: [tile 0..3][piece 0..2][lane], and reach LDS with global_load_lds.
#include "pa_host.h"
#include "pa_mfma_ops.h"
#include "pa_split_ops.h"

namespace pa {
namespace f32rows {

using mfma::f32x16;
using mfma::half_sum;
using mfma::kperm;
using mfma::mma;
using mfma::rowmap;
using mfma::u32x4;
using namespace split;

constexpr int kC = 128, kH = 8, kD = 16, kS = 32;
using split::kUnit;

// W (128, K) -> K / 16 units
__global__ __launch_bounds__(256) void pack_linear_kernel(const float *__restrict__ w, int K, int permuted,
                                                          u32x4 *__restrict__ blob) {
  pack_unit(w, K, 16 * blockIdx.x, permuted != 0, blob + (int64_t)blockIdx.x * kUnit, threadIdx.x);
}

// Mlp weights W1 (F, 128), W2 (128, F) -> per chunk of 128 hidden features 8 units of W1's rows (natural order) and
// 8 units of W2's columns (permuted: the hidden features arrive as accumulator registers)
__global__ __launch_bounds__(256) void pack_mlp_kernel(const float *__restrict__ w1, const float *__restrict__ w2, int F,
                                                       u32x4 *__restrict__ blob) {
  const int c = blockIdx.x >> 4, u = blockIdx.x & 15;
  u32x4 *unit = blob + (int64_t)blockIdx.x * kUnit;
  if (u < 8) pack_unit(w1 + (int64_t)c * 128 * kC, kC, 16 * u, false, unit, threadIdx.x);
  else pack_unit(w2 + c * 128, F, 16 * (u - 8), true, unit, threadIdx.x);
}

// acc[t] += unit's tile t (A operand) . rows (B operand bp): the six products, the four tiles taking turns
__device__ __forceinline__ void kstep(f32x16 (&acc)[4], const u32x4 *unit_lane, const u32x4 (&bp)[3]) {
  u32x4 fr[4][3];
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int p = 0; p < 3; ++p) fr[t][p] = unit_lane[(t * 3 + p) * 64];
  constexpr int pw[6] = {0, 1, 0, 1, 2, 0}, pa[6] = {0, 0, 1, 1, 0, 2};
#pragma unroll
  for (int q = 0; q < 6; ++q)
#pragma unroll
    for (int t = 0; t < 4; ++t) acc[t] = mma(fr[t][pw[q]], bp[pa[q]], acc[t]);
}

// registers 8 kk .. 8 kk + 7 of an accumulator tile as the B operand of the next product's k-step
__device__ __forceinline__ void split_half(const f32x16 &v, int kk, u32x4 (&pl)[3]) {
  float e[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) e[j] = kk ? v[8 + j] : v[j];
  split8(e, pl);
}

// The tail on a wave's transposed tile: y = yT (+ residual) leaves, then LayerNorm(y) if asked for.  A lane holds 64
// of its row's 128 channels (4 consecutive ones per register quad), its partner lane the others.  gb: gamma | beta.
struct Head {  // output head behind the LayerNorm: out (rows, O) = LayerNorm(y) W^T + b, O <= 4; w points into LDS
  const float *w, *b;
  float *out;
  int O;
};

__device__ __forceinline__ void finish_rows(f32x16 (&yT)[4], int64_t row, bool ok, int g, const float *residual, float *y,
                                            float *ln_out, const float *gb, float eps, bool want_ln = false,
                                            Head head = Head{nullptr, nullptr, nullptr, 0}) {
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int64_t at = row * kC + 32 * t + 8 * q + 4 * g;
      float4 v = {yT[t][4 * q], yT[t][4 * q + 1], yT[t][4 * q + 2], yT[t][4 * q + 3]};
      if (residual) {
        const float4 r = *reinterpret_cast<const float4 *>(residual + at);
        v.x += r.x, v.y += r.y, v.z += r.z, v.w += r.w;
      }
      if (ok) *reinterpret_cast<float4 *>(y + at) = v;
      yT[t][4 * q] = v.x, yT[t][4 * q + 1] = v.y, yT[t][4 * q + 2] = v.z, yT[t][4 * q + 3] = v.w;
    }
  if (!ln_out && !want_ln) return;
  float sum = 0.f;
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) sum += yT[t][r];
  const float mean = half_sum(sum) * (1.f / kC);
  float sq = 0.f;
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float d = yT[t][r] - mean;
      sq = fmaf(d, d, sq);
    }
  const float rstd = 1.f / sqrtf(half_sum(sq) * (1.f / kC) + eps);
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int c0 = 32 * t + 8 * q + 4 * g;
      const float4 ga = *reinterpret_cast<const float4 *>(gb + c0), be = *reinterpret_cast<const float4 *>(gb + kC + c0);
      float4 o;
      o.x = (yT[t][4 * q] - mean) * rstd * ga.x + be.x;
      o.y = (yT[t][4 * q + 1] - mean) * rstd * ga.y + be.y;
      o.z = (yT[t][4 * q + 2] - mean) * rstd * ga.z + be.z;
      o.w = (yT[t][4 * q + 3] - mean) * rstd * ga.w + be.w;
      if (ok && ln_out) *reinterpret_cast<float4 *>(ln_out + row * kC + c0) = o;
      yT[t][4 * q] = o.x, yT[t][4 * q + 1] = o.y, yT[t][4 * q + 2] = o.z, yT[t][4 * q + 3] = o.w;
    }
  for (int o = 0; o < head.O; ++o) {  // a lane sums its 64 channels, its partner lane the others
    float acc = 0.f;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const float4 wq = *reinterpret_cast<const float4 *>(head.w + o * kC + 32 * t + 8 * q + 4 * g);
        acc = fmaf(yT[t][4 * q], wq.x, acc), acc = fmaf(yT[t][4 * q + 1], wq.y, acc);
        acc = fmaf(yT[t][4 * q + 2], wq.z, acc), acc = fmaf(yT[t][4 * q + 3], wq.w, acc);
      }
    acc = half_sum(acc) + (head.b ? head.b[o] : 0.f);
    if (ok && g == 0) head.out[row * head.O + o] = acc;
  }
}

struct Tail {
  const float *residual, *gamma, *beta;
  float *ln_out;
  float eps;
};

__device__ __forceinline__ void stage_gamma_beta(float *gb, const Tail &tail, int tid) {
  if (tid < kC) {
    gb[tid] = tail.gamma ? tail.gamma[tid] : 1.f;
    gb[kC + tid] = tail.beta ? tail.beta[tid] : 0.f;
  }
}

// The batch's attended slice tokens (H, S, D float32, 16 KB) as the block-diagonal A operands of the hand-back:
// tokp[(pair 4 + kk) 3 + piece][lane], lane (i, g): row (hh, d) = (i / 16, i % 16), reduction index k = 16 kk + 8 g + j
// over (head of the pair, slice) -- out_token[2 pair + hh][k % 32][d] where k / 32 == hh, else 0.  The tokens are read
// once, coalesced (4 float4 per thread, fetched by the caller ahead of its other loads), put into `raw` (4096 floats
// of LDS scratch) and cut from there.  Ends with a barrier.
__device__ __forceinline__ void fetch_tokens(const float *tok, float4 (&t4)[4], int tid) {
#pragma unroll
  for (int q = 0; q < 4; ++q) t4[q] = reinterpret_cast<const float4 *>(tok)[tid + 256 * q];
}
__device__ __forceinline__ void build_token_operands(const float4 (&t4)[4], float *raw, u32x4 *tokp, int tid) {
#pragma unroll
  for (int q = 0; q < 4; ++q) reinterpret_cast<float4 *>(raw)[tid + 256 * q] = t4[q];
  __syncthreads();
  for (int item = tid; item < 16 * 64; item += 256) {
    const int pk = item >> 6, l = item & 63, li = l & 31, lg = l >> 5;
    const int pair = pk >> 2, kk = pk & 3, hh = li >> 4, d = li & 15;
    float e[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int k = 16 * kk + 8 * lg + j;
      e[j] = (k >> 5) == hh ? raw[((2 * pair + hh) * kS + (k & 31)) * kD + d] : 0.f;
    }
    u32x4 pl[3];
    split8(e, pl);
#pragma unroll
    for (int p = 0; p < 3; ++p) tokp[(pk * 3 + p) * 64 + l] = pl[p];
  }
  __syncthreads();
}

// acc[t][r] += v[32 t + rowmap(r, g)] for a vector v of 128 floats in LDS (4 consecutive channels per register quad)
__device__ __forceinline__ void add_channel_vector(f32x16 (&acc)[4], const float *v, int g) {
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float4 b = *reinterpret_cast<const float4 *>(v + 32 * t + 8 * q + 4 * g);
      acc[t][4 * q] += b.x, acc[t][4 * q + 1] += b.y, acc[t][4 * q + 2] += b.z, acc[t][4 * q + 3] += b.w;
    }
}

// ---------------------------------------------------------------------------------------------------------------
// deslice_linear_kernel.  A workgroup's four tiles belong to one batch.  LDS: W_out as 8 units (96 KB), the batch's
// attended slice tokens as A operands (48 KB), gamma | beta.
//   out_x^T (head pair P: 32 channels x 32 points) = T_P w_P^T, reduction index k = 0 .. 63 over (head of the pair,
//   slice): T_P[(hh, d)][k] = out_token[2 P + hh][k % 32][d] where k / 32 == hh, else 0;  w_P[point][k] is the point's
//   64 consecutive weights of the two heads.
// ---------------------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void deslice_linear_kernel(const u32x4 *__restrict__ blob,
                                                             const float *__restrict__ b_out,
                                                             const float *__restrict__ w,
                                                             const float *__restrict__ out_token, float *__restrict__ y,
                                                             Tail tail, int N, int bpb) {
  extern __shared__ u32x4 smem[];
  u32x4 *wout = smem;                   // 8 units
  u32x4 *tokp = smem + 8 * kUnit;       // [pair][kk][piece][lane]
  float *gb = reinterpret_cast<float *>(tokp + 16 * 192);
  const int tid = threadIdx.x, lane = tid & 63, i = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int b = blockIdx.x / bpb, gblk = blockIdx.x - b * bpb;
  const int n0 = (gblk * 4 + wave) * 32;
  const int n = min(n0 + i, N - 1);
  const bool ok = n0 + i < N;
  stage_gamma_beta(gb, tail, tid);
  float4 tok4[4];
  fetch_tokens(out_token + (int64_t)b * kH * kS * kD, tok4, tid);
  // this lane's half of its point's weights (two runs of 8 per head), and the output bias
  float wr[4][4][8];  // [head pair][kk][j]
  {
    const float *wrow = w + ((int64_t)b * N + n) * (kH * kS) + 8 * g;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
        const float4 *src = reinterpret_cast<const float4 *>(wrow + 64 * t + 16 * kk);
        const float4 lo = src[0], hi = src[1];
        wr[t][kk][0] = lo.x, wr[t][kk][1] = lo.y, wr[t][kk][2] = lo.z, wr[t][kk][3] = lo.w;
        wr[t][kk][4] = hi.x, wr[t][kk][5] = hi.y, wr[t][kk][6] = hi.z, wr[t][kk][7] = hi.w;
      }
  }
  f32x16 yT[4];
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) yT[t][r] = b_out ? b_out[32 * t + rowmap(r, g)] : 0.f;
  // the batch's tokens as block-diagonal A operands (W_out's slots are still empty: their first 16 KB are the scratch)
  build_token_operands(tok4, reinterpret_cast<float *>(smem), tokp, tid);
  // Every load above is complete (the builtin, so that the compiler knows it too) before W_out is requested: from here
  // on vmcnt counts this wave's 24 requests only, and the first product runs while they land.
  __builtin_amdgcn_s_waitcnt(0x0F70);
#pragma unroll
  for (int u = 0; u < 8; ++u)
    load_3k_to_lds(blob + u * kUnit + wave * 192, lane * 16, (unsigned)(uintptr_t)(wout + u * kUnit + wave * 192));
  __syncthreads();
  // out_x^T: the four head pairs take turns
  f32x16 ox[4];
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) ox[t][r] = 0.f;
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) {
    u32x4 bp[4][3];
#pragma unroll
    for (int t = 0; t < 4; ++t) split8(wr[t][kk], bp[t]);
    constexpr int pw[6] = {0, 1, 0, 1, 2, 0}, pa[6] = {0, 0, 1, 1, 0, 2};
#pragma unroll
    for (int q = 0; q < 6; ++q)
#pragma unroll
      for (int t = 0; t < 4; ++t)
        ox[t] = mma(tokp[((t * 4 + kk) * 3 + pw[q]) * 64 + lane], bp[t][pa[q]], ox[t]);
  }
  // y^T = W_out out_x^T + b_out; unit ks is needed at step ks: the 3 (7 - ks) younger requests may still be in flight
  static_for<8>([&](auto ks_) {
    constexpr int ks = decltype(ks_)::value;
    if constexpr (ks == 0) asm volatile("s_waitcnt vmcnt(21)" ::: "memory");
    if constexpr (ks == 1) asm volatile("s_waitcnt vmcnt(18)" ::: "memory");
    if constexpr (ks == 2) asm volatile("s_waitcnt vmcnt(15)" ::: "memory");
    if constexpr (ks == 3) asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
    if constexpr (ks == 4) asm volatile("s_waitcnt vmcnt(9)" ::: "memory");
    if constexpr (ks == 5) asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
    if constexpr (ks == 6) asm volatile("s_waitcnt vmcnt(3)" ::: "memory");
    if constexpr (ks == 7) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    u32x4 bp[3];
    split_half(ox[ks >> 1], ks & 1, bp);
    kstep(yT, wout + ks * kUnit + lane, bp);
  });
  finish_rows(yT, (int64_t)b * N + n, ok, g, tail.residual, y, tail.ln_out, gb, tail.eps);
}

// ---------------------------------------------------------------------------------------------------------------
// mlp_kernel.  LDS: a ring of 12 weight units (144 KB), gamma | beta.  Chunk c of 128 hidden features uses units
// 16 c .. 16 c + 7 (W1 rows) and 16 c + 8 .. 16 c + 15 (W2 columns); units are requested up to 12 ahead, 8 at a time
// after the product that frees their slots.
// ---------------------------------------------------------------------------------------------------------------
constexpr int kMlpRing = 12;

__global__ __launch_bounds__(256) void mlp_kernel(const u32x4 *__restrict__ blob, const float *__restrict__ b1,
                                                  const float *__restrict__ b2, const float *__restrict__ u,
                                                  float *__restrict__ y, Tail tail, int64_t M, int F) {
  extern __shared__ u32x4 smem[];
  float *gb = reinterpret_cast<float *>(smem + kMlpRing * kUnit);
  const int tid = threadIdx.x, lane = tid & 63, i = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int64_t row0 = ((int64_t)blockIdx.x * 4 + wave) * 32;
  const int64_t row = min(row0 + i, M - 1);
  const bool ok = row0 + i < M;
  const int total = (F / 128) * 16;
  int issued = 0;
  auto issue_upto = [&](int upto) {  // this wave's quarter (3 KB) of units issued .. upto - 1
    for (; issued < upto && issued < total; ++issued)
      load_3k_to_lds(blob + (int64_t)issued * kUnit + wave * 192, lane * 16,
                     (unsigned)(uintptr_t)(smem + (issued % kMlpRing) * kUnit + wave * 192));
  };
  // units below `upto` have landed for every wave: at most the 4 newest units (3 operations each) stay in flight
  auto wait_landed = [&](int upto) {
    if (issued - upto >= 4) asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  };
  stage_gamma_beta(gb, tail, tid);
  // the wave's rows: lane (i, g) holds channels 16 ks + 8 g .. + 7 of row i
  float xr[8][8];
  {
    const float *src = u + row * kC + 8 * g;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      const float4 lo = *reinterpret_cast<const float4 *>(src + 16 * ks), hi = *reinterpret_cast<const float4 *>(src + 16 * ks + 4);
      xr[ks][0] = lo.x, xr[ks][1] = lo.y, xr[ks][2] = lo.z, xr[ks][3] = lo.w;
      xr[ks][4] = hi.x, xr[ks][5] = hi.y, xr[ks][6] = hi.z, xr[ks][7] = hi.w;
    }
  }
  f32x16 yT[4], hT[4];
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      yT[t][r] = b2 ? b2[32 * t + rowmap(r, g)] : 0.f;
      hT[t][r] = b1 ? b1[32 * t + rowmap(r, g)] : 0.f;
    }
  // Every load above is complete (the builtin, so that the compiler knows it too) before the weights are requested:
  // in the first chunk vmcnt counts this wave's requests only, and the products start while they land.
  __builtin_amdgcn_s_waitcnt(0x0F70);
  issue_upto(kMlpRing);
  __syncthreads();
  // Step j (0 .. 15) of the first chunk needs unit j.  Units 0 .. 11 are requested up front, 12 .. 15 (and, with more
  // chunks, 16 .. 19) after the first product: with one chunk the younger requests that may stay in flight are units
  // j + 1 .. 11 during the first product and j + 1 .. 15 during the second.
  auto wait_first_chunk = [&](auto j_) {
    constexpr int j = decltype(j_)::value;
    if (total > kMlpRing + 4) {  // more chunks follow: wait once per product, for all but the 4 youngest units
      if constexpr (j == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      if constexpr (j == 8) asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
    } else {
      constexpr int younger = j < 8 ? 3 * (11 - j) : 3 * (15 - j);
      if constexpr (younger == 33) asm volatile("s_waitcnt vmcnt(33)" ::: "memory");
      if constexpr (younger == 30) asm volatile("s_waitcnt vmcnt(30)" ::: "memory");
      if constexpr (younger == 27) asm volatile("s_waitcnt vmcnt(27)" ::: "memory");
      if constexpr (younger == 24) asm volatile("s_waitcnt vmcnt(24)" ::: "memory");
      if constexpr (younger == 21) asm volatile("s_waitcnt vmcnt(21)" ::: "memory");
      if constexpr (younger == 18) asm volatile("s_waitcnt vmcnt(18)" ::: "memory");
      if constexpr (younger == 15) asm volatile("s_waitcnt vmcnt(15)" ::: "memory");
      if constexpr (younger == 12) asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
      if constexpr (younger == 9) asm volatile("s_waitcnt vmcnt(9)" ::: "memory");
      if constexpr (younger == 6) asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
      if constexpr (younger == 3) asm volatile("s_waitcnt vmcnt(3)" ::: "memory");
      if constexpr (younger == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    __syncthreads();
  };
  for (int c = 0; c < F / 128; ++c) {
    const int base = 16 * c;
    if (c > 0) {
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) hT[t][r] = b1 ? b1[128 * c + 32 * t + rowmap(r, g)] : 0.f;
      __builtin_amdgcn_s_waitcnt(0x0F70);
      wait_landed(base + 8);
    }
    static_for<8>([&](auto ks_) {
      constexpr int ks = decltype(ks_)::value;
      if (c == 0) wait_first_chunk(ks_);
      u32x4 bp[3];
      split8(xr[ks], bp);
      kstep(hT, smem + ((base + ks) % kMlpRing) * kUnit + lane, bp);
    });
    __syncthreads();  // the slots of W1's units are free
    issue_upto(base + 8 + kMlpRing);
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) hT[t][r] = gelu_erf(hT[t][r]);
    if (c > 0) wait_landed(base + 16);
    static_for<8>([&](auto ks_) {
      constexpr int ks = decltype(ks_)::value;
      if (c == 0) wait_first_chunk(std::integral_constant<int, 8 + ks>{});
      u32x4 bp[3];
      split_half(hT[ks >> 1], ks & 1, bp);
      kstep(yT, smem + ((base + 8 + ks) % kMlpRing) * kUnit + lane, bp);
    });
    __syncthreads();  // the slots of W2's units are free
    issue_upto(base + 16 + kMlpRing);
  }
  finish_rows(yT, row, ok, g, tail.residual, y, tail.ln_out, gb, tail.eps);
}

// ---------------------------------------------------------------------------------------------------------------
// block_tail_kernel: everything of a block that is local to a point, after the slice attention (TR.py:300-303):
//   out_x = w . out_token;  fx1 = out_x W_out^T + b_out + fx_in;  n = LayerNorm_2(fx1);
//   fx_out = W2 gelu(W1 n + b1) + b2 + fx1;  next_ln_out = LayerNorm_next(fx_out)
// = deslice_linear_kernel followed by mlp_kernel with the rows staying in registers in between (fx1 and its
// LayerNorm are never stored).  Weight stream: W_out (units 0 .. 7), then per chunk of 128 hidden features W1's rows
// and W2's columns (8 units each, both with the reduction index in register order); ring of 12 units whose last four
// slots first hold the batch's slice tokens as A operands.  LDS behind the ring: gamma | beta of both LayerNorms and
// the three biases.
// ---------------------------------------------------------------------------------------------------------------
struct BlockArgs {
  const float *b_out, *w, *out_token, *fx_in;
  const float *ln2_gamma, *ln2_beta;
  float ln2_eps;
  const float *b1, *b2;
  float *fx_out;
  Tail next;  // residual unused
  const float *head_w, *head_b;  // output head behind the next LayerNorm (O <= 4 outputs), or NULL
  float *head_out;
  int head_O;
};

__global__ __launch_bounds__(256) void pack_block_kernel(const float *__restrict__ w_out, const float *__restrict__ w1,
                                                         const float *__restrict__ w2, int F, u32x4 *__restrict__ blob) {
  u32x4 *unit = blob + (int64_t)blockIdx.x * kUnit;
  if (blockIdx.x < 8) {
    pack_unit(w_out, kC, 16 * blockIdx.x, true, unit, threadIdx.x);
    return;
  }
  const int q = blockIdx.x - 8, c = q >> 4, u = q & 15;
  if (u < 8) pack_unit(w1 + (int64_t)c * 128 * kC, kC, 16 * u, true, unit, threadIdx.x);
  else pack_unit(w2 + c * 128, F, 16 * (u - 8), true, unit, threadIdx.x);
}

__global__ __launch_bounds__(256) void block_tail_kernel(const u32x4 *__restrict__ blob, BlockArgs a, int N, int bpb, int F) {
  extern __shared__ u32x4 smem[];
  u32x4 *tokp = smem + 8 * kUnit;  // [pair][kk][piece][lane], in ring slots 8 .. 11 until the hand-back is done
  float *gb2 = reinterpret_cast<float *>(smem + kMlpRing * kUnit);  // gamma | beta of LayerNorm_2
  float *gbn = gb2 + 2 * kC;                                        // gamma | beta of the next LayerNorm
  float *bo = gbn + 2 * kC, *bb2 = bo + kC, *hw = bb2 + kC, *bb1 = hw + 4 * kC;  // b_out, b2, head weight, b1 (F)
  const int tid = threadIdx.x, lane = tid & 63, i = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int b = blockIdx.x / bpb, gblk = blockIdx.x - b * bpb;
  const int n0 = (gblk * 4 + wave) * 32;
  const int n = min(n0 + i, N - 1);
  const bool ok = n0 + i < N;
  const int64_t row = (int64_t)b * N + n;
  const int total = 8 + (F / 128) * 16;
  int issued = 0;
  auto issue_upto = [&](int upto) {
    for (; issued < upto && issued < total; ++issued)
      load_3k_to_lds(blob + (int64_t)issued * kUnit + wave * 192, lane * 16,
                     (unsigned)(uintptr_t)(smem + (issued % kMlpRing) * kUnit + wave * 192));
  };
  auto wait_landed = [&](int upto) {  // units below `upto` have landed for every wave (4 younger units may be in flight)
    if (issued - upto >= 4) asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  };
  // every global load of the prologue is issued before the first of them is used: one round trip to memory
  float sv[6] = {1.f, 0.f, 1.f, 0.f, 0.f, 0.f};
  if (tid < kC) {
    sv[0] = a.ln2_gamma[tid];
    sv[1] = a.ln2_beta[tid];
    if (a.next.gamma) sv[2] = a.next.gamma[tid];
    if (a.next.beta) sv[3] = a.next.beta[tid];
    if (a.b_out) sv[4] = a.b_out[tid];
    if (a.b2) sv[5] = a.b2[tid];
  }
  float4 tok4[4];
  fetch_tokens(a.out_token + (int64_t)b * kH * kS * kD, tok4, tid);
  // this lane's half of its point's weights and of its residual row
  float wr[4][4][8];
  {
    const float *wrow = a.w + row * (kH * kS) + 8 * g;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
        const float4 *src = reinterpret_cast<const float4 *>(wrow + 64 * t + 16 * kk);
        const float4 lo = src[0], hi = src[1];
        wr[t][kk][0] = lo.x, wr[t][kk][1] = lo.y, wr[t][kk][2] = lo.z, wr[t][kk][3] = lo.w;
        wr[t][kk][4] = hi.x, wr[t][kk][5] = hi.y, wr[t][kk][6] = hi.z, wr[t][kk][7] = hi.w;
      }
  }
  f32x16 fx1[4];  // first the residual, then fx1
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float4 r = *reinterpret_cast<const float4 *>(a.fx_in + row * kC + 32 * t + 8 * q + 4 * g);
      fx1[t][4 * q] = r.x, fx1[t][4 * q + 1] = r.y, fx1[t][4 * q + 2] = r.z, fx1[t][4 * q + 3] = r.w;
    }
  if (tid < kC) {
    gb2[tid] = sv[0], gb2[kC + tid] = sv[1];
    gbn[tid] = sv[2], gbn[kC + tid] = sv[3];
    bo[tid] = sv[4], bb2[tid] = sv[5];
  }
  for (int k = tid; k < F; k += 256) bb1[k] = a.b1 ? a.b1[k] : 0.f;
  for (int k = tid; k < a.head_O * kC; k += 256) hw[k] = a.head_w[k];
  // the batch's tokens as block-diagonal A operands (the ring's first slots are still empty: 16 KB of them are the
  // scratch)
  build_token_operands(tok4, reinterpret_cast<float *>(smem), tokp, tid);
  // every load above is complete (the builtin, so that the compiler knows it too) before the weights are requested
  __builtin_amdgcn_s_waitcnt(0x0F70);
  issue_upto(8);
  __syncthreads();
  // out_x^T: the four head pairs take turns
  f32x16 ox[4];
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) ox[t][r] = 0.f;
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) {
    u32x4 bp[4][3];
#pragma unroll
    for (int t = 0; t < 4; ++t) split8(wr[t][kk], bp[t]);
    constexpr int pw[6] = {0, 1, 0, 1, 2, 0}, pa[6] = {0, 0, 1, 1, 0, 2};
#pragma unroll
    for (int q = 0; q < 6; ++q)
#pragma unroll
      for (int t = 0; t < 4; ++t)
        ox[t] = mma(tokp[((t * 4 + kk) * 3 + pw[q]) * 64 + lane], bp[t][pa[q]], ox[t]);
  }
  __syncthreads();  // the tokens are used up: their slots join the ring
  issue_upto(kMlpRing);
  // fx1 = W_out out_x^T + b_out + fx_in
  add_channel_vector(fx1, bo, g);
  wait_landed(8);
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) {
    u32x4 bp[3];
    split_half(ox[ks >> 1], ks & 1, bp);
    kstep(fx1, smem + ks * kUnit + lane, bp);
  }
  __syncthreads();  // W_out's slots are free
  issue_upto(8 + kMlpRing);
  // n = LayerNorm_2(fx1), in registers
  f32x16 nT[4];
  {
    float sum = 0.f;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) sum += fx1[t][r];
    const float mean = half_sum(sum) * (1.f / kC);
    float sq = 0.f;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float d = fx1[t][r] - mean;
        sq = fmaf(d, d, sq);
      }
    const float rstd = 1.f / sqrtf(half_sum(sq) * (1.f / kC) + a.ln2_eps);
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int c0 = 32 * t + 8 * q + 4 * g;
        const float4 ga = *reinterpret_cast<const float4 *>(gb2 + c0), be = *reinterpret_cast<const float4 *>(gb2 + kC + c0);
        nT[t][4 * q] = (fx1[t][4 * q] - mean) * rstd * ga.x + be.x;
        nT[t][4 * q + 1] = (fx1[t][4 * q + 1] - mean) * rstd * ga.y + be.y;
        nT[t][4 * q + 2] = (fx1[t][4 * q + 2] - mean) * rstd * ga.z + be.z;
        nT[t][4 * q + 3] = (fx1[t][4 * q + 3] - mean) * rstd * ga.w + be.w;
      }
  }
  // the MLP; its second product accumulates on top of fx1 + b2
  add_channel_vector(fx1, bb2, g);
  for (int c = 0; c < F / 128; ++c) {
    const int base = 8 + 16 * c;
    f32x16 hT[4];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) hT[t][r] = 0.f;
    add_channel_vector(hT, bb1 + 128 * c, g);
    wait_landed(base + 8);
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      u32x4 bp[3];
      split_half(nT[ks >> 1], ks & 1, bp);
      kstep(hT, smem + ((base + ks) % kMlpRing) * kUnit + lane, bp);
    }
    __syncthreads();  // the slots of W1's units are free
    issue_upto(base + 8 + kMlpRing);
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) hT[t][r] = gelu_erf(hT[t][r]);
    wait_landed(base + 16);
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      u32x4 bp[3];
      split_half(hT[ks >> 1], ks & 1, bp);
      kstep(fx1, smem + ((base + 8 + ks) % kMlpRing) * kUnit + lane, bp);
    }
    __syncthreads();  // the slots of W2's units are free
    issue_upto(base + 16 + kMlpRing);
  }
  finish_rows(fx1, row, ok, g, nullptr, a.fx_out, a.next.ln_out, gbn, a.next.eps, a.head_O > 0,
              Head{hw, a.head_b, a.head_out, a.head_O});
}

// ---------------------------------------------------------------------------------------------------------------
// premlp_kernel: the model's preprocess Mlp (TR.py:519-525), Linear(c_in -> F) -> GELU -> Linear(F -> 128) with a few
// input features per point (coordinates and fields, c_in <= 8), and the first block's LayerNorm as the tail.  The first
// Linear is c_in multiply-adds per hidden feature on the vector units (its weights sit in LDS, every lane of a half
// wave reads the same feature's row); the second is mlp_kernel's second product over W2's units, 8 per chunk of 128
// hidden features.
// ---------------------------------------------------------------------------------------------------------------
constexpr int kPreMaxIn = 8;

__global__ __launch_bounds__(256) void pack_premlp_kernel(const float *__restrict__ w2, int F, u32x4 *__restrict__ blob) {
  const int c = blockIdx.x >> 3, u = blockIdx.x & 7;
  pack_unit(w2 + c * 128, F, 16 * u, true, blob + (int64_t)blockIdx.x * kUnit, threadIdx.x);
}

template <int C_IN>
__global__ __launch_bounds__(256) void premlp_kernel(const u32x4 *__restrict__ blob, const float *__restrict__ w1,
                                                     const float *__restrict__ b1, const float *__restrict__ b2,
                                                     const float *__restrict__ u, float *__restrict__ y, Tail tail,
                                                     int64_t M, int F) {
  extern __shared__ u32x4 smem[];
  float *gb = reinterpret_cast<float *>(smem + kMlpRing * kUnit);
  float *w1s = gb + 2 * kC;  // [input feature 0 .. C_IN - 1 | bias][hidden feature]: (C_IN + 1) * F floats
  const int tid = threadIdx.x, lane = tid & 63, i = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int64_t row0 = ((int64_t)blockIdx.x * 4 + wave) * 32;
  const int64_t row = min(row0 + i, M - 1);
  const bool ok = row0 + i < M;
  const int total = (F / 128) * 8;
  int issued = 0;
  auto issue_upto = [&](int upto) {
    for (; issued < upto && issued < total; ++issued)
      load_3k_to_lds(blob + (int64_t)issued * kUnit + wave * 192, lane * 16,
                     (unsigned)(uintptr_t)(smem + (issued % kMlpRing) * kUnit + wave * 192));
  };
  stage_gamma_beta(gb, tail, tid);
  for (int k = tid; k < F * (C_IN + 1); k += 256) {
    const int j = k / F, f = k - j * F;
    w1s[k] = j < C_IN ? w1[f * C_IN + j] : (b1 ? b1[f] : 0.f);
  }
  float xin[C_IN];
#pragma unroll
  for (int j = 0; j < C_IN; ++j) xin[j] = u[row * C_IN + j];
  f32x16 yT[4];
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) yT[t][r] = b2 ? b2[32 * t + rowmap(r, g)] : 0.f;
  __builtin_amdgcn_s_waitcnt(0x0F70);  // the loads above are complete before the weights are requested
  issue_upto(kMlpRing);
  __syncthreads();
  for (int c = 0; c < F / 128; ++c) {
    f32x16 hT[4];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int q = 0; q < 4; ++q) {  // the quad's 4 consecutive hidden features
        const float *wf = w1s + 128 * c + 32 * t + 8 * q + 4 * g;
        float4 a = *reinterpret_cast<const float4 *>(wf + C_IN * F);
#pragma unroll
        for (int j = 0; j < C_IN; ++j) {
          const float4 wj = *reinterpret_cast<const float4 *>(wf + j * F);
          a.x = fmaf(xin[j], wj.x, a.x), a.y = fmaf(xin[j], wj.y, a.y);
          a.z = fmaf(xin[j], wj.z, a.z), a.w = fmaf(xin[j], wj.w, a.w);
        }
        hT[t][4 * q] = gelu_erf(a.x), hT[t][4 * q + 1] = gelu_erf(a.y);
        hT[t][4 * q + 2] = gelu_erf(a.z), hT[t][4 * q + 3] = gelu_erf(a.w);
      }
    // units 8 c .. 8 c + 7 have landed for every wave: at most the 4 youngest units stay in flight
    if (issued - (8 * c + 8) >= 4) asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      u32x4 bp[3];
      split_half(hT[ks >> 1], ks & 1, bp);
      kstep(yT, smem + ((8 * c + ks) % kMlpRing) * kUnit + lane, bp);
    }
    __syncthreads();  // the slots of this chunk's units are free
    issue_upto(8 * c + 8 + kMlpRing);
  }
  finish_rows(yT, row, ok, g, tail.residual, y, tail.ln_out, gb, tail.eps);
}

static Tail make_tail(const pa_block_tail *t) {
  Tail r{};
  if (!t) return r;
  r.residual = static_cast<const float *>(t->residual);
  r.ln_out = static_cast<float *>(t->ln_out);
  r.gamma = t->ln_gamma;
  r.beta = t->ln_beta;
  r.eps = t->ln_eps;
  return r;
}

bool backend_supported(int dtype, const pa_shape &s) {
  return dtype == PA_F32 && s.C == kC && s.H == kH && s.D == kD && s.S == kS;
}

int64_t backend_blob_bytes() { return 8 * (int64_t)kUnit * 16; }

int backend(const pa_shape &s, const pa_params &p, const void *w, const float *out_token, void *y,
            const pa_block_tail *tail, void *blob, bool blob_ready, hipStream_t st) {
  if (!backend_supported(PA_F32, s)) return PA_ERR_UNSUPPORTED;
  int rc = PA_OK;
  if (!blob_ready) {
    hipLaunchKernelGGL(pack_linear_kernel, dim3(8), dim3(256), 0, st, static_cast<const float *>(p.out_linear_weight),
                       kC, 1, static_cast<u32x4 *>(blob));
    if ((rc = launch_status())) return rc;
  }
  const size_t lds = (size_t)(8 * kUnit + 16 * 192) * 16 + 2 * kC * 4;
  if ((rc = allow_dynamic_lds(deslice_linear_kernel, lds))) return rc;
  const int bpb = (int)(((s.N + 31) / 32 + 3) / 4);
  hipLaunchKernelGGL(deslice_linear_kernel, dim3((unsigned)(s.B * bpb)), dim3(256), lds, st,
                     static_cast<const u32x4 *>(blob), p.out_linear_bias, static_cast<const float *>(w), out_token,
                     static_cast<float *>(y), make_tail(tail), (int)s.N, bpb);
  return launch_status();
}

bool mlp_supported(int dtype, int64_t M, int64_t C, int64_t F) {
  return dtype == PA_F32 && M > 0 && C == kC && F >= 128 && F % 128 == 0 && F <= 8192;
}

int64_t mlp_blob_bytes(int64_t F) { return (F / 128) * 16 * (int64_t)kUnit * 16; }

int mlp_pack(int64_t F, const void *w1, const void *w2, void *blob, hipStream_t st) {
  hipLaunchKernelGGL(pack_mlp_kernel, dim3((unsigned)((F / 128) * 16)), dim3(256), 0, st, static_cast<const float *>(w1),
                     static_cast<const float *>(w2), (int)F, static_cast<u32x4 *>(blob));
  return launch_status();
}

int mlp_forward(int64_t M, int64_t F, const void *blob, const float *b1, const float *b2, const void *u, void *y,
                const pa_block_tail *tail, hipStream_t st) {
  const size_t lds = (size_t)kMlpRing * kUnit * 16 + 2 * kC * 4;
  int rc = allow_dynamic_lds(mlp_kernel, lds);
  if (rc) return rc;
  const int64_t blocks = ((M + 31) / 32 + 3) / 4;
  hipLaunchKernelGGL(mlp_kernel, dim3((unsigned)blocks), dim3(256), lds, st, static_cast<const u32x4 *>(blob), b1, b2,
                     static_cast<const float *>(u), static_cast<float *>(y), make_tail(tail), M, (int)F);
  return launch_status();
}

static size_t block_lds(int64_t F) { return (size_t)kMlpRing * kUnit * 16 + (size_t)(4 * kC + 2 * kC + 4 * kC + F) * 4; }

// F up to 1024 (mlp_ratio 8): what the interface documents and the parity tests cover
bool block_supported(int dtype, const pa_shape &s, int64_t F) {
  return backend_supported(dtype, s) && F >= 128 && F % 128 == 0 && F <= 1024 && block_lds(F) <= 160 * 1024;
}

int64_t block_blob_bytes(int64_t F) { return (8 + (F / 128) * 16) * (int64_t)kUnit * 16; }

int block_tail(const pa_shape &s, const pa_params &p, const pa_block_mlp &m, const void *w, const float *out_token,
               const void *fx_in, void *fx_out, const pa_block_tail *next, const pa_block_head *head, void *blob,
               bool blob_ready, hipStream_t st) {
  if (!block_supported(PA_F32, s, m.F)) return PA_ERR_UNSUPPORTED;
  int rc = PA_OK;
  if (!blob_ready) {
    hipLaunchKernelGGL(pack_block_kernel, dim3((unsigned)(8 + (m.F / 128) * 16)), dim3(256), 0, st,
                       static_cast<const float *>(p.out_linear_weight), static_cast<const float *>(m.w1),
                       static_cast<const float *>(m.w2), (int)m.F, static_cast<u32x4 *>(blob));
    if ((rc = launch_status())) return rc;
  }
  const size_t lds = block_lds(m.F);
  if ((rc = allow_dynamic_lds(block_tail_kernel, lds))) return rc;
  BlockArgs a{};
  a.b_out = p.out_linear_bias;
  a.w = static_cast<const float *>(w);
  a.out_token = out_token;
  a.fx_in = static_cast<const float *>(fx_in);
  a.ln2_gamma = m.ln_gamma;
  a.ln2_beta = m.ln_beta;
  a.ln2_eps = m.ln_eps;
  a.b1 = m.b1;
  a.b2 = m.b2;
  a.fx_out = static_cast<float *>(fx_out);
  a.next = make_tail(next);
  if (head) {
    a.head_w = static_cast<const float *>(head->weight);
    a.head_b = head->bias;
    a.head_out = static_cast<float *>(head->out);
    a.head_O = (int)head->O;
  }
  const int bpb = (int)(((s.N + 31) / 32 + 3) / 4);
  hipLaunchKernelGGL(block_tail_kernel, dim3((unsigned)(s.B * bpb)), dim3(256), lds, st,
                     static_cast<const u32x4 *>(blob), a, (int)s.N, bpb, (int)m.F);
  return launch_status();
}

static size_t premlp_lds(int64_t c_in, int64_t F) {
  return (size_t)kMlpRing * kUnit * 16 + 2 * kC * 4 + (size_t)F * (c_in + 1) * 4;
}

bool premlp_supported(int dtype, int64_t M, int64_t c_in, int64_t F, int64_t C) {
  return dtype == PA_F32 && M > 0 && C == kC && c_in >= 1 && c_in <= kPreMaxIn && F >= 128 && F % 128 == 0 &&
         premlp_lds(c_in, F) <= 160 * 1024;
}

int64_t premlp_blob_bytes(int64_t F) { return (F / 128) * 8 * (int64_t)kUnit * 16; }

int premlp_forward(int64_t M, int64_t c_in, int64_t F, const void *w1, const float *b1, const void *w2, const float *b2,
                   const void *u, void *y, const pa_block_tail *tail, void *blob, hipStream_t st) {
  hipLaunchKernelGGL(pack_premlp_kernel, dim3((unsigned)((F / 128) * 8)), dim3(256), 0, st,
                     static_cast<const float *>(w2), (int)F, static_cast<u32x4 *>(blob));
  int rc = launch_status();
  if (rc) return rc;
  const size_t lds = premlp_lds(c_in, F);
  const int64_t blocks = ((M + 31) / 32 + 3) / 4;
  auto launch = [&](auto kernel) {
    int rc2 = allow_dynamic_lds(kernel, lds);
    if (rc2) return rc2;
    hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(256), lds, st, static_cast<const u32x4 *>(blob),
                       static_cast<const float *>(w1), b1, b2, static_cast<const float *>(u), static_cast<float *>(y),
                       make_tail(tail), M, (int)F);
    return launch_status();
  };
  switch (c_in) {
    case 1: return launch(premlp_kernel<1>);
    case 2: return launch(premlp_kernel<2>);
    case 3: return launch(premlp_kernel<3>);
    case 4: return launch(premlp_kernel<4>);
    case 5: return launch(premlp_kernel<5>);
    case 6: return launch(premlp_kernel<6>);
    case 7: return launch(premlp_kernel<7>);
    case 8: return launch(premlp_kernel<8>);
    default: return PA_ERR_UNSUPPORTED;
  }
}

}  // namespace f32rows
}  // namespace pa
