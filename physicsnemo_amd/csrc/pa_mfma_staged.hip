// Staged bf16 MFMA forward for layers the fused kernels do not hold in registers (C = 512, i.e. 16 heads): the same
// arithmetic as the fused path, split at the natural-layout projections.
//   rows_linear_kernel          x -> x_mid (natural layout) and fx_mid (packed operand layout)          [pa_gemm.hip]
//   slice_softmax_pack_kernel   x_mid -> slice logits, temperature softmax -> packed slice weights       [this file]
//   slice_reduce_kernel         first pass of the slice-token sums                                       [pa_mfma.hip]
//   slice_attention_kernel      second pass, normalisation, slice attention                              [pa_mfma.hip]
//   deslice_natural_kernel      attended tokens back to the points -> out_x (natural layout)             [pa_mfma_bwd.hip]
//   rows_linear_kernel          out_linear                                                               [pa_gemm.hip]
#include "pa_common.h"
#include "pa_host.h"
#include "pa_mfma_ops.h"

namespace pa {
namespace mfma {

// ------------------------------------------------------------------------------------------------
// slice_softmax_pack_kernel: grid (G, B, head groups), one wave per head of the group; wave h walks the batch's
// 32-point tiles g, g + G, ...
//   logits^T (S x 32 pts) = W_slice (A, LDS, k = d in natural order) . x_mid^T (B = the points' rows, 16-byte loads)
//   softmax over s in the base-2 domain: in-lane over the accumulator registers plus one exchange with lane ^ 32
//   -> w_pack (the layout kernel (a) of the fused path writes); rows beyond N get zero weight.
// ------------------------------------------------------------------------------------------------
template <int S>
__global__ __launch_bounds__(512) void slice_softmax_pack_kernel(const uint16_t *__restrict__ x_mid,
                                                                 const float *__restrict__ w_slice,
                                                                 const float *__restrict__ b_slice,
                                                                 const float *__restrict__ temperature,
                                                                 u32x4 *__restrict__ w_pack, int64_t N, int tpb, int H) {
  constexpr int ST = (S + 31) / 32, NCH = S / 16;
  __shared__ u32x4 wsl[ST * 2 * 64];
  __shared__ float bsl[ST * 32];
  const int tid = threadIdx.x, lane = tid & 63, i = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int h = blockIdx.z * (blockDim.x >> 6) + wave;
  const int b = blockIdx.y;
  const int HD = H * 32;
  for (int u = tid; u < ST * 2 * 64; u += blockDim.x) {
    const int ul = u & 63, ui = ul & 31, ug = ul >> 5, f = u >> 6, st = f >> 1, kk = f & 1;
    const int s = 32 * st + ui;
    bf16x8 e;
#pragma unroll
    for (int j = 0; j < 8; ++j) e[j] = (__bf16)(s < S ? w_slice[s * 32 + 16 * kk + 8 * ug + j] : 0.f);
    wsl[u] = __builtin_bit_cast(u32x4, e);
  }
  for (int s = tid; s < ST * 32; s += blockDim.x) bsl[s] = s < S ? b_slice[s] : -1e30f;  // slices beyond S: weight 0
  __syncthreads();
  const float sc = kLog2e / clamp_temperature(temperature[h]);

  for (int t = blockIdx.x; t < tpb; t += gridDim.x) {
    const int64_t n = (int64_t)t * 32 + i;
    const bool valid = n < N;
    const uint16_t *row = x_mid + ((int64_t)b * N + (valid ? n : N - 1)) * HD + h * 32 + 8 * g;
    const u32x4 xm0 = *reinterpret_cast<const u32x4 *>(row), xm1 = *reinterpret_cast<const u32x4 *>(row + 16);
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
    u32x4 *wdst = w_pack + ((((int64_t)b * tpb + t) * H + h) * NCH) * 64 + lane;
#pragma unroll
    for (int cq = 0; cq < NCH; ++cq)
      wdst[cq * 64] = (cq & 1) ? pack_half<1>(lg[cq >> 1], inv) : pack_half<0>(lg[cq >> 1], inv);
  }
}

// ------------------------------------------------------------------------------------------------
// slice_softmax_pack_plus_kernel: the Transolver++ form (PA.py:166-170, :530-537, gumbel_softmax.py:49-57).  Same
// layout: wave = head, lanes <-> the tile's points, accumulator registers <-> slices.  Per point and head
//   hidden^T = W1 . x_mid^T + b1  (the first Linear of proj_temperature: a second MFMA pair on the same B operands)
//   temp     = max(temperature[h] + gelu(b2 + sum_s w2[s] gelu(hidden[s])), 0.01)        in-lane + one half exchange
//   w        = softmax_s((logits[s] - log(-log(u[s] + 1e-8) + 1e-8)) / temp)             u: the caller's U[0,1) samples
// `uniform` (B, N, H, S) bf16 in natural layout: a lane reads its slices (runs of four) with 8-byte loads.
// ------------------------------------------------------------------------------------------------
template <int S>
__global__ __launch_bounds__(512) void slice_softmax_pack_plus_kernel(
    const uint16_t *__restrict__ x_mid, const uint16_t *__restrict__ uniform, const float *__restrict__ w_slice,
    const float *__restrict__ b_slice, const float *__restrict__ temperature, const float *__restrict__ pt_w1,
    const float *__restrict__ pt_b1, const float *__restrict__ pt_w2, const float *__restrict__ pt_b2,
    u32x4 *__restrict__ w_pack, int64_t N, int tpb, int H) {
  constexpr int ST = (S + 31) / 32, NCH = S / 16;
  constexpr float kLn2 = 0.6931471805599453f;
  __shared__ u32x4 wsl[ST * 2 * 64];
  __shared__ u32x4 w1l[ST * 2 * 64];
  __shared__ float bsl[ST * 32], b1l[ST * 32], w2l[ST * 32];
  const int tid = threadIdx.x, lane = tid & 63, i = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int h = blockIdx.z * (blockDim.x >> 6) + wave;
  const int b = blockIdx.y;
  const int HD = H * 32, HS = H * S;
  for (int u = tid; u < ST * 2 * 64; u += blockDim.x) {
    const int ul = u & 63, ui = ul & 31, ug = ul >> 5, f = u >> 6, st = f >> 1, kk = f & 1;
    const int s = 32 * st + ui;
    bf16x8 e, e1;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      e[j] = (__bf16)(s < S ? w_slice[s * 32 + 16 * kk + 8 * ug + j] : 0.f);
      e1[j] = (__bf16)(s < S ? pt_w1[s * 32 + 16 * kk + 8 * ug + j] : 0.f);
    }
    wsl[u] = __builtin_bit_cast(u32x4, e);
    w1l[u] = __builtin_bit_cast(u32x4, e1);
  }
  for (int s = tid; s < ST * 32; s += blockDim.x) {
    bsl[s] = s < S ? b_slice[s] : -1e30f;  // slices beyond S: weight 0
    b1l[s] = s < S ? pt_b1[s] : 0.f;
    w2l[s] = s < S ? pt_w2[s] : 0.f;
  }
  __syncthreads();
  const float temp_h = temperature[h], b2 = pt_b2[0];

  for (int t = blockIdx.x; t < tpb; t += gridDim.x) {
    const int64_t n = (int64_t)t * 32 + i;
    const bool valid = n < N;
    const int64_t m = (int64_t)b * N + (valid ? n : N - 1);
    const uint16_t *row = x_mid + m * HD + h * 32 + 8 * g;
    const u32x4 xm0 = *reinterpret_cast<const u32x4 *>(row), xm1 = *reinterpret_cast<const u32x4 *>(row + 16);
    // the point's temperature
    float a2 = 0.f;
#pragma unroll 1
    for (int st = 0; st < ST; ++st) {  // not unrolled: the tile's registers are free again before the logits are formed
      f32x16 hd;
#pragma unroll
      for (int r = 0; r < 16; ++r) hd[r] = b1l[32 * st + rowmap(r, g)];
      hd = mma(w1l[(st * 2 + 0) * 64 + lane], xm0, hd);
      hd = mma(w1l[(st * 2 + 1) * 64 + lane], xm1, hd);
#pragma unroll
      for (int r = 0; r < 16; ++r) a2 = fmaf(w2l[32 * st + rowmap(r, g)], gelu_logistic(hd[r]), a2);
    }
    a2 = half_sum(a2) + b2;
    const float temp = bf16_bits_to_f32(f32_to_bf16_bits(fmaxf(temp_h + gelu_logistic(a2), 0.01f)));
    const float sc = kLog2e * __builtin_amdgcn_rcpf(temp);
    // logits + Gumbel noise
    const uint16_t *urow = uniform + m * HS + h * S;
    f32x16 lg[ST];
#pragma unroll
    for (int st = 0; st < ST; ++st) {
#pragma unroll
      for (int r = 0; r < 16; ++r) lg[st][r] = bsl[32 * st + rowmap(r, g)];
      lg[st] = mma(wsl[(st * 2 + 0) * 64 + lane], xm0, lg[st]);
      lg[st] = mma(wsl[(st * 2 + 1) * 64 + lane], xm1, lg[st]);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int s0 = 32 * st + 8 * q + 4 * g;  // slices rowmap(4 q .. 4 q + 3, g)
        if (s0 < S) {
          const uint2 raw = *reinterpret_cast<const uint2 *>(urow + s0);
          const float uu[4] = {__uint_as_float(raw.x << 16), __uint_as_float(raw.x & 0xffff0000u),
                               __uint_as_float(raw.y << 16), __uint_as_float(raw.y & 0xffff0000u)};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float inner = fmaf(-kLn2, __builtin_amdgcn_logf(uu[j] + 1e-8f), 1e-8f);  // -ln(u + eps) + eps
            lg[st][4 * q + j] = fmaf(-kLn2, __builtin_amdgcn_logf(inner), lg[st][4 * q + j]);
          }
        }
      }
    }
    float mx = -INFINITY;
#pragma unroll
    for (int st = 0; st < ST; ++st)
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, lg[st][r]);
    mx = half_max(mx);
    const float off = mx * sc;
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
    u32x4 *wdst = w_pack + ((((int64_t)b * tpb + t) * H + h) * NCH) * 64 + lane;
#pragma unroll
    for (int cq = 0; cq < NCH; ++cq)
      wdst[cq * 64] = (cq & 1) ? pack_half<1>(lg[cq >> 1], inv) : pack_half<0>(lg[cq >> 1], inv);
  }
}

// ------------------------------------------------------------------------------------------------
// slice_softmax_reduce_kernel: slice weights and the first pass of the slice-token sums in one kernel.
// grid (G, B, head groups), one wave per head of the group; wave h walks the batch's 32-point tiles g, g + G, ...
// and keeps the sums of its (batch, head) in registers:
//   w^T (32 s x 32 pts, lane <-> slice) = chunk . SEL          (an exact MFMA transpose, as in slice_reduce_kernel)
//   norm[s] += sum over the tile's points;   tok^T (32 d x 32 s) += fx_chunk (A: rows d, k = points) . bf16(w^T)
// One partial per workgroup row: partials[g][b][h][s][0..D-1] = sum_n w fx, [..][D] = sum_n w.
// ------------------------------------------------------------------------------------------------
// PACKED_X: x_mid is [tile][head][2][lane] (the B operands themselves) instead of (B, N, H*32) rows.
template <int S, bool PACKED_X>
__global__ __launch_bounds__(512) void slice_softmax_reduce_kernel(const uint16_t *__restrict__ x_mid,
                                                                   const u32x4 *__restrict__ fx_pack,
                                                                   const float *__restrict__ w_slice,
                                                                   const float *__restrict__ b_slice,
                                                                   const float *__restrict__ temperature,
                                                                   float *__restrict__ partials, int64_t N, int tpb,
                                                                   int H) {
  constexpr int ST = (S + 31) / 32, NCH = S / 16, D1 = 33;
  __shared__ u32x4 wsl[ST * 2 * 64];
  __shared__ float bsl[ST * 32];
  const int tid = threadIdx.x, lane = tid & 63, i = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int h = blockIdx.z * (blockDim.x >> 6) + wave;
  const int b = blockIdx.y;
  const int HD = H * 32;
  stage_slice_projection<S, PACKED_X>(w_slice, b_slice, wsl, bsl);
  __syncthreads();
  const float sc = kLog2e / clamp_temperature(temperature[h]);
  u32x4 sel[2];
#pragma unroll
  for (int par = 0; par < 2; ++par) {
    bf16x8 s8;
#pragma unroll
    for (int j = 0; j < 8; ++j) s8[j] = (__bf16)((i == kperm(par, g, j)) ? 1.f : 0.f);
    sel[par] = __builtin_bit_cast(u32x4, s8);
  }
  f32x16 tok[ST];
  float nrm[ST];
#pragma unroll
  for (int st = 0; st < ST; ++st) {
    nrm[st] = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) tok[st][r] = 0.f;
  }
  for (int t = blockIdx.x; t < tpb; t += gridDim.x) {
    const int64_t n = (int64_t)t * 32 + i;
    const bool valid = n < N;
    u32x4 xm0, xm1;
    if constexpr (PACKED_X) {
      const u32x4 *xsrc = reinterpret_cast<const u32x4 *>(x_mid) + ((((int64_t)b * tpb + t) * H + h) * 2) * 64 + lane;
      xm0 = load_streaming(xsrc);
      xm1 = load_streaming(xsrc + 64);
    } else {
      const uint16_t *row = x_mid + ((int64_t)b * N + (valid ? n : N - 1)) * HD + h * 32 + 8 * g;
      xm0 = *reinterpret_cast<const u32x4 *>(row);
      xm1 = *reinterpret_cast<const u32x4 *>(row + 16);
    }
    const u32x4 *fsrc = fx_pack + ((((int64_t)b * tpb + t) * H + h) * 2) * 64 + lane;
    const u32x4 f0 = load_streaming(fsrc), f1 = load_streaming(fsrc + 64);
    u32x4 chunk[NCH];
    slice_weights_of_tile<S>(wsl, bsl, xm0, xm1, sc, valid, lane, g, chunk);
#pragma unroll
    for (int st = 0; st < ST; ++st) {
      f32x16 tr;
#pragma unroll
      for (int r = 0; r < 16; ++r) tr[r] = 0.f;
      tr = mma(chunk[2 * st], sel[0], tr);
      if (2 * st + 1 < NCH) tr = mma(chunk[2 * st + 1 < NCH ? 2 * st + 1 : 0], sel[1], tr);
      float s16 = 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) s16 += tr[r];
      nrm[st] += s16;
      tok[st] = mma(f0, pack_half<0>(tr), tok[st]);
      tok[st] = mma(f1, pack_half<1>(tr), tok[st]);
    }
  }
  float *dst = partials + (((int64_t)blockIdx.x * gridDim.y + b) * H + h) * (S * D1);
#pragma unroll
  for (int st = 0; st < ST; ++st) {
    const int s = 32 * st + i;
    const float total = half_sum(nrm[st]);
    if (s < S) {
#pragma unroll
      for (int r = 0; r < 16; ++r) dst[s * D1 + rowmap(r, g)] = tok[st][r];
      if (g == 0) dst[s * D1 + 32] = total;
    }
  }
}

// ------------------------------------------------------------------------------------------------
// deslice_recompute_kernel: the attended tokens back to the points, slice weights recomputed from x_mid.
// grid (G, B, head groups), one wave per head of the group;
//   out_x^T_h (32 d x 32 pts) = tok'^T_h (A: tokp fragments, registers) . w_h (B: the chunks)
// out_x may be x_mid itself: a wave reads the 64 bytes of its (point, head) before it writes them, and nobody else
// touches them.
// ------------------------------------------------------------------------------------------------
// PACKED_X: x_mid and out_x are [tile][head][2][lane] operand tiles (out_x: lanes <-> points, k = the head's channels in
// kperm order, what linear_rows_kernel reads as its rows).
template <int S, bool PACKED_X>
__global__ __launch_bounds__(512) void deslice_recompute_kernel(const uint16_t *x_mid, const u32x4 *__restrict__ tokp,
                                                                const float *__restrict__ w_slice,
                                                                const float *__restrict__ b_slice,
                                                                const float *__restrict__ temperature, uint16_t *out_x,
                                                                int64_t N, int tpb, int H) {
  constexpr int ST = (S + 31) / 32, NCH = S / 16;
  __shared__ u32x4 wsl[ST * 2 * 64];
  __shared__ float bsl[ST * 32];
  const int tid = threadIdx.x, lane = tid & 63, i = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int h = blockIdx.z * (blockDim.x >> 6) + wave;
  const int b = blockIdx.y;
  const int HD = H * 32;
  stage_slice_projection<S, PACKED_X>(w_slice, b_slice, wsl, bsl);
  __syncthreads();
  const float sc = kLog2e / clamp_temperature(temperature[h]);
  u32x4 tp[NCH];
#pragma unroll
  for (int cq = 0; cq < NCH; ++cq) tp[cq] = tokp[(((int64_t)b * H + h) * NCH + cq) * 64 + lane];
  for (int t = blockIdx.x; t < tpb; t += gridDim.x) {
    const int64_t n = (int64_t)t * 32 + i;
    const bool valid = n < N;
    const int64_t m = (int64_t)b * N + (valid ? n : N - 1);
    const int64_t pk = ((((int64_t)b * tpb + t) * H + h) * 2) * 64 + lane;
    u32x4 xm0, xm1;
    if constexpr (PACKED_X) {
      const u32x4 *xsrc = reinterpret_cast<const u32x4 *>(x_mid) + pk;
      xm0 = load_streaming(xsrc);
      xm1 = load_streaming(xsrc + 64);
    } else {
      const uint16_t *row = x_mid + m * HD + h * 32 + 8 * g;
      xm0 = *reinterpret_cast<const u32x4 *>(row);
      xm1 = *reinterpret_cast<const u32x4 *>(row + 16);
    }
    // un-normalised weights e_s (bf16); out = (sum_s e_s tok'_s) / (sum_s e_s), the denominator from an MFMA whose A
    // operand is all ones: every row of that product is the column sum of the same rounded values
    u32x4 chunk[NCH];
    slice_weights_of_tile<S, true>(wsl, bsl, xm0, xm1, sc, valid, lane, g, chunk);
    f32x16 ox, den;
#pragma unroll
    for (int r = 0; r < 16; ++r) ox[r] = den[r] = 0.f;
    const u32x4 ones = u32x4{0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u};
#pragma unroll
    for (int cq = 0; cq < NCH; ++cq) {
      ox = mma(tp[cq], chunk[cq], ox);
      den = mma(ones, chunk[cq], den);
    }
    const float inv = __builtin_amdgcn_rcpf(den[0]);
#pragma unroll
    for (int r = 0; r < 16; ++r) ox[r] *= inv;
    if constexpr (PACKED_X) {
      u32x4 *odst = reinterpret_cast<u32x4 *>(out_x) + pk;
      store_streaming(odst, pack_half<0>(ox));
      store_streaming(odst + 64, pack_half<1>(ox));
    } else {
      store_tile_natural(ox, out_x + m * HD + h * 32, g, valid);
    }
  }
}

// shapes of the staged path: what the fused kernels serve plus C = 512, large enough for the row kernels to pay off
bool staged_supported(int dtype, const pa_shape &s) {
  // grid convolutions as projections: the implicit-GEMM kernel writes the same two layouts (tap-major weights)
  if (s.conv_k != 0 && (s.conv_tap_major != 1 || s.C % 8 != 0)) return false;
  if (dtype != PA_BF16 || s.D != 32 || s.C != s.H * 32) return false;
  if (s.C != 128 && s.C != 256 && s.C != 512) return false;
  if (s.S != 16 && s.S != 32 && s.S != 64 && s.S != 128) return false;
  if ((s.N + 31) / 32 * s.B > ((int64_t)1 << 31) / 16 || s.B > 65535) return false;
  return s.B * s.N >= 4096;
}

int slice_softmax_pack(const pa_shape &s, const pa_params &p, const void *x_mid, void *w_pack, int num_cu,
                       hipStream_t st) {
  const int waves = (int)(s.H < 8 ? s.H : 8);
  if (s.H % waves != 0) return PA_ERR_UNSUPPORTED;
  const int groups = (int)(s.H / waves);
  int64_t gx = (2 * (int64_t)num_cu + s.B * groups - 1) / (s.B * groups);
  const int64_t tpb = tiles_per_batch(s);
  if (gx > tpb) gx = tpb;
  if (gx < 1) gx = 1;
  const dim3 grid((unsigned)gx, (unsigned)s.B, (unsigned)groups), block((unsigned)(waves * 64));
#define PA_LAUNCH_SSP(SS)                                                                                           \
  hipLaunchKernelGGL((slice_softmax_pack_kernel<SS>), grid, block, 0, st, static_cast<const uint16_t *>(x_mid),     \
                     p.in_project_slice_weight, p.in_project_slice_bias, p.temperature, static_cast<u32x4 *>(w_pack), \
                     s.N, (int)tpb, (int)s.H)
  switch (s.S) {
    case 16: PA_LAUNCH_SSP(16); break;
    case 32: PA_LAUNCH_SSP(32); break;
    case 64: PA_LAUNCH_SSP(64); break;
    case 128: PA_LAUNCH_SSP(128); break;
    default: return PA_ERR_UNSUPPORTED;
  }
#undef PA_LAUNCH_SSP
  return launch_status();
}

int slice_softmax_pack_plus(const pa_shape &s, const pa_params &p, const pa_plus_params &pp, const void *x_mid,
                            const void *uniform, void *w_pack, int num_cu, hipStream_t st) {
  const int waves = (int)(s.H < 8 ? s.H : 8);
  if (s.H % waves != 0) return PA_ERR_UNSUPPORTED;
  const int groups = (int)(s.H / waves);
  int64_t gx = (2 * (int64_t)num_cu + s.B * groups - 1) / (s.B * groups);
  const int64_t tpb = tiles_per_batch(s);
  if (gx > tpb) gx = tpb;
  if (gx < 1) gx = 1;
  const dim3 grid((unsigned)gx, (unsigned)s.B, (unsigned)groups), block((unsigned)(waves * 64));
#define PA_LAUNCH_SSPP(SS)                                                                                          \
  hipLaunchKernelGGL((slice_softmax_pack_plus_kernel<SS>), grid, block, 0, st, static_cast<const uint16_t *>(x_mid), \
                     static_cast<const uint16_t *>(uniform), p.in_project_slice_weight, p.in_project_slice_bias,     \
                     p.temperature, pp.proj_temperature_0_weight, pp.proj_temperature_0_bias,                        \
                     pp.proj_temperature_2_weight, pp.proj_temperature_2_bias, static_cast<u32x4 *>(w_pack), s.N,    \
                     (int)tpb, (int)s.H)
  switch (s.S) {
    case 16: PA_LAUNCH_SSPP(16); break;
    case 32: PA_LAUNCH_SSPP(32); break;
    case 64: PA_LAUNCH_SSPP(64); break;
    case 128: PA_LAUNCH_SSPP(128); break;
    default: return PA_ERR_UNSUPPORTED;
  }
#undef PA_LAUNCH_SSPP
  return launch_status();
}

// grid of the two recomputing kernels: waves = heads per workgroup; a workgroup of 8 waves fills a CU (two waves per
// SIMD at their register count), so one workgroup per CU: fewer partial sums to combine
static void recompute_grid(const pa_shape &s, int num_cu, dim3 *grid, dim3 *block) {
  const int waves = (int)(s.H < 8 ? s.H : 8);
  const int groups = (int)(s.H / waves);
  const int per_cu = waves >= 8 ? 1 : 2;
  int64_t gx = (per_cu * (int64_t)num_cu + s.B * groups - 1) / (s.B * groups);
  const int64_t tpb = tiles_per_batch(s);
  if (gx > tpb) gx = tpb;
  if (gx < 1) gx = 1;
  *grid = dim3((unsigned)gx, (unsigned)s.B, (unsigned)groups);
  *block = dim3((unsigned)(waves * 64));
}

int64_t softmax_reduce_groups(const pa_shape &s, int num_cu) {
  dim3 grid, block;
  recompute_grid(s, num_cu, &grid, &block);
  return grid.x;
}

int slice_softmax_reduce(const pa_shape &s, const pa_params &p, const void *x_mid, bool packed_x, const void *fx_pack,
                         float *partials, int num_cu, hipStream_t st) {
  if (s.H % (s.H < 8 ? s.H : 8) != 0) return PA_ERR_UNSUPPORTED;
  dim3 grid, block;
  recompute_grid(s, num_cu, &grid, &block);
  const int tpb = (int)tiles_per_batch(s);
#define PA_LAUNCH_SSR1(SS, PK)                                                                                         \
  hipLaunchKernelGGL((slice_softmax_reduce_kernel<SS, PK>), grid, block, 0, st, static_cast<const uint16_t *>(x_mid), \
                     static_cast<const u32x4 *>(fx_pack), p.in_project_slice_weight, p.in_project_slice_bias,          \
                     p.temperature, partials, s.N, tpb, (int)s.H)
#define PA_LAUNCH_SSR(SS) \
  if (packed_x) PA_LAUNCH_SSR1(SS, true); else PA_LAUNCH_SSR1(SS, false)
  switch (s.S) {
    case 16: PA_LAUNCH_SSR(16); break;
    case 32: PA_LAUNCH_SSR(32); break;
    case 64: PA_LAUNCH_SSR(64); break;
    case 128: PA_LAUNCH_SSR(128); break;
    default: return PA_ERR_UNSUPPORTED;
  }
#undef PA_LAUNCH_SSR
#undef PA_LAUNCH_SSR1
  return launch_status();
}

int deslice_recompute(const pa_shape &s, const pa_params &p, const void *x_mid, bool packed_x, const void *tokp,
                      void *out_x, int num_cu, hipStream_t st) {
  if (s.H % (s.H < 8 ? s.H : 8) != 0) return PA_ERR_UNSUPPORTED;
  dim3 grid, block;
  recompute_grid(s, num_cu, &grid, &block);
  const int tpb = (int)tiles_per_batch(s);
#define PA_LAUNCH_DR1(SS, PK)                                                                                      \
  hipLaunchKernelGGL((deslice_recompute_kernel<SS, PK>), grid, block, 0, st, static_cast<const uint16_t *>(x_mid), \
                     static_cast<const u32x4 *>(tokp), p.in_project_slice_weight, p.in_project_slice_bias,          \
                     p.temperature, static_cast<uint16_t *>(out_x), s.N, tpb, (int)s.H)
#define PA_LAUNCH_DR(SS) \
  if (packed_x) PA_LAUNCH_DR1(SS, true); else PA_LAUNCH_DR1(SS, false)
  switch (s.S) {
    case 16: PA_LAUNCH_DR(16); break;
    case 32: PA_LAUNCH_DR(32); break;
    case 64: PA_LAUNCH_DR(64); break;
    case 128: PA_LAUNCH_DR(128); break;
    default: return PA_ERR_UNSUPPORTED;
  }
#undef PA_LAUNCH_DR
#undef PA_LAUNCH_DR1
  return launch_status();
}

}  // namespace mfma
}  // namespace pa
