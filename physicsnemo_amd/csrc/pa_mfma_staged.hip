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

}  // namespace mfma
}  // namespace pa
