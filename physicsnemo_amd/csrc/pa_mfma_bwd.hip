// bf16 MFMA kernels of the backward pass (the shapes of the fused MFMA forward path).  They consume the packed
// slice weights the forward kernels leave behind (w_pack) and natural-layout (B, N, H*32) activations / gradients:
//
//   deslice_natural_kernel        out_x[n, h, :] = sum_s w[n, h, s] tok'[h, s, :]         (input of d W_out = dy^T out_x)
//   backward_tables_kernel        per-(b, h) MFMA operand fragments of tok', d num and W_slice
//   slice_softmax_backward_mfma   per point: d w = g tok'^T + fx_mid d num^T + d nrm, softmax backward, d z, d T,
//                                 d x_mid = d z W_slice, d fx_mid = w d num                       (formulas: pa_backward.hip)
//
// Register layouts: see pa_mfma_ops.h.  Every product is arranged so that the accumulator tile has lanes <-> points and
// registers <-> slices / channels (the layout of the forward kernel's logits), i.e. the packed slice weights, the
// recomputed logits and d w line up element by element and all per-point reductions over the slices are in-lane sums
// plus one exchange with lane ^ 32.
#include "pa_common.h"
#include "pa_host.h"
#include "pa_mfma_ops.h"

namespace pa {
namespace mfma {

// ------------------------------------------------------------------------------------------------
// deslice_natural_kernel: grid (G, B, head groups), one wave per head of the group; wave h walks the batch's tiles
// g, g + G, ...
//   out_x^T_h (32 d x 32 pts) = tok'^T_h (A: tokp fragments, registers) . w_h (B: w_pack chunks)
// ------------------------------------------------------------------------------------------------
template <int S>
__global__ __launch_bounds__(512) void deslice_natural_kernel(const u32x4 *__restrict__ w_pack,
                                                              const u32x4 *__restrict__ tokp,
                                                              uint16_t *__restrict__ out_x, int64_t N, int tpb, int H) {
  constexpr int NCH = S / 16;
  const int tid = threadIdx.x, lane = tid & 63, i = lane & 31, g = lane >> 5;
  const int h = blockIdx.z * (blockDim.x >> 6) + __builtin_amdgcn_readfirstlane(tid >> 6);
  const int b = blockIdx.y;
  u32x4 tp[NCH];
#pragma unroll
  for (int cq = 0; cq < NCH; ++cq) tp[cq] = tokp[(((int64_t)b * H + h) * NCH + cq) * 64 + lane];
  for (int t = blockIdx.x; t < tpb; t += gridDim.x) {
    const int64_t gt = (int64_t)b * tpb + t;
    const u32x4 *wsrc = w_pack + ((gt * H + h) * NCH) * 64 + lane;
    f32x16 ox;
#pragma unroll
    for (int r = 0; r < 16; ++r) ox[r] = 0.f;
#pragma unroll
    for (int cq = 0; cq < NCH; ++cq) ox = mma(tp[cq], load_streaming(wsrc + cq * 64), ox);
    const int64_t n = (int64_t)t * 32 + i;
    const bool ok = n < N;
    store_tile_natural(ox, out_x + ((int64_t)b * N + (ok ? n : 0)) * (H * 32) + h * 32, g, ok);
  }
}

// ------------------------------------------------------------------------------------------------
// Operand fragments of the backward kernel (16-byte units, one per lane; lane = 32g + i; j = 0..7):
//   shared   wsl[(st*2 + kk)]   = W_slice[32st + i][16kk + 8g + j]                 A of the logits (k = d, natural order)
//            wsT[cq]            = W_slice[16cq + rowmap(j, g)][i]                   A of d x_mid (k = slices, chained order)
//   per (b,h) tokA[(st*2 + kk)] = tok'[32st + i][16kk + 8g + j]                    A of d w, first half of k
//            dnA[(st*2 + kk)]   = d num[32st + i][16kk + 8g + j]                   A of d w, second half of k
//            dnT[cq]            = d num[16cq + rowmap(j, g)][i]                     A of d fx_mid
// Slices >= S read as zero.
// ------------------------------------------------------------------------------------------------
struct BwdTablePlan {
  int st2, nch;         // fragments per group
  int64_t shared_units, per_head_units;
};
__host__ __device__ inline BwdTablePlan bwd_table_plan(int S) {
  BwdTablePlan p;
  p.st2 = 2 * ((S + 31) / 32);
  p.nch = S / 16;
  p.shared_units = (int64_t)(p.st2 + p.nch) * 64;
  p.per_head_units = (int64_t)(2 * p.st2 + p.nch) * 64;
  return p;
}

__global__ __launch_bounds__(256) void backward_tables_kernel(const float *__restrict__ w_slice,
                                                              const float *__restrict__ out_token,
                                                              const float *__restrict__ d_num, u32x4 *__restrict__ tabs,
                                                              int BH, int S) {
  const BwdTablePlan tp = bwd_table_plan(S);
  const int64_t total = tp.shared_units + (int64_t)BH * tp.per_head_units;
  for (int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x; u < total; u += (int64_t)gridDim.x * 256) {
    const int lane = (int)(u & 63), i = lane & 31, g = lane >> 5;
    int64_t f = u >> 6;  // fragment index
    const float *src;    // (S, 32) table
    bool natural;        // true: [slice 32st + i][16kk + 8g + j]; false: [16cq + rowmap(j, g)][i]
    int idx;
    if (f < tp.st2 + tp.nch) {
      src = w_slice;
      natural = f < tp.st2;
      idx = (int)(natural ? f : f - tp.st2);
    } else {
      f -= tp.st2 + tp.nch;
      const int64_t bh = f / (2 * tp.st2 + tp.nch);
      const int r = (int)(f - bh * (2 * tp.st2 + tp.nch));
      if (r < tp.st2) {
        src = out_token + bh * S * 32;
        natural = true;
        idx = r;
      } else if (r < 2 * tp.st2) {
        src = d_num + bh * S * 32;
        natural = true;
        idx = r - tp.st2;
      } else {
        src = d_num + bh * S * 32;
        natural = false;
        idx = r - 2 * tp.st2;
      }
    }
    uint16_t e[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      int s, d;
      if (natural) {
        s = 32 * (idx >> 1) + i;
        d = 16 * (idx & 1) + 8 * g + j;
      } else {
        s = 16 * idx + rowmap(j, g);
        d = i;
      }
      e[j] = s < S ? to_bf16_bits(src[s * 32 + d]) : (uint16_t)0;
    }
    u32x4 v;
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = (uint32_t)e[2 * j] | ((uint32_t)e[2 * j + 1] << 16);
    tabs[u] = v;
  }
}

// ------------------------------------------------------------------------------------------------
// slice_softmax_backward_mfma_kernel: grid (G, B), H waves; wave h owns head h; its tok' / d num fragments stay in
// registers (S <= 64) or in LDS (S = 128, where the registers are needed for d w), the W_slice fragments are shared
// through LDS.  Per 32-point tile and head:
//   z^T  (S x pts) = W_slice . x_mid^T + b_slice                       B = x_mid rows, 16-byte natural loads
//   dw^T (S x pts) = tok' . g^T + d num . fx_mid^T + d nrm             B = g / fx_mid rows
//   w: unpacked from w_pack; dot = sum_s w dw / sum_s w; dz = (w / T) (dw - dot); dT -= sum dz z / T
//   d x_mid^T (32 x pts) = W_slice^T . dz^T (B = bf16(dz^T) straight from registers); d fx_mid^T = d num^T . w (B = w_pack)
// Rows beyond N have w = 0 in w_pack (the forward writes zeros), so they contribute nothing; their loads are clamped to
// the last valid row and their stores are masked.
// ------------------------------------------------------------------------------------------------
template <int S>
__global__ __launch_bounds__(S > 64 ? 256 : 512) void slice_softmax_backward_mfma_kernel(
    const uint16_t *__restrict__ x_mid, const uint16_t *__restrict__ fx_mid, const uint16_t *__restrict__ d_out_x,
    const u32x4 *__restrict__ w_pack, const u32x4 *__restrict__ tabs, const float *__restrict__ d_norm,
    const float *__restrict__ b_slice, const float *__restrict__ temperature, uint16_t *__restrict__ d_proj,
    uint16_t *__restrict__ d_z, float *__restrict__ dT_part, int64_t N, int tpb, int H) {
  constexpr int ST = (S + 31) / 32, NCH = S / 16, ST2 = 2 * ST;
  constexpr bool LDSTAB = S > 64;  // tok' / d num fragments of d w in LDS instead of registers
  __shared__ u32x4 wsh[(ST2 + NCH) * 64];
  __shared__ float bsl[ST * 32];
  __shared__ float dnl[8 * ST * 32];  // d nrm of every head of this batch (H <= 8)
  extern __shared__ u32x4 tabl[];     // LDSTAB: [H][2 * ST2][64]
  const BwdTablePlan tp = bwd_table_plan(S);
  const int tid = threadIdx.x, lane = tid & 63, i = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int h = blockIdx.z * (blockDim.x >> 6) + wave;  // grid.z walks groups of heads (S = 128: 4 waves per workgroup)
  const int b = blockIdx.y;
  const int HD = H * 32;
  const int64_t bh = (int64_t)b * H + h;

  for (int u = tid; u < (ST2 + NCH) * 64; u += blockDim.x) wsh[u] = tabs[u];
  for (int s = tid; s < ST * 32; s += blockDim.x) bsl[s] = s < S ? b_slice[s] : 0.f;
  u32x4 tokA[LDSTAB ? 1 : ST2], dnA[LDSTAB ? 1 : ST2], dnT[NCH];
  {
    const u32x4 *mine = tabs + tp.shared_units + bh * tp.per_head_units + lane;
    if constexpr (LDSTAB) {
      for (int f = 0; f < 2 * ST2; ++f) tabl[(wave * 2 * ST2 + f) * 64 + lane] = mine[f * 64];
    } else {
#pragma unroll
      for (int f = 0; f < ST2; ++f) {
        tokA[f] = mine[f * 64];
        dnA[f] = mine[(ST2 + f) * 64];
      }
    }
#pragma unroll
    for (int cq = 0; cq < NCH; ++cq) dnT[cq] = mine[(2 * ST2 + cq) * 64];
  }
  const u32x4 *mytab = tabl + (wave * 2 * ST2) * 64 + lane;  // LDSTAB: this head's tok' fragments, then its d num fragments
  for (int e = tid; e < H * ST * 32; e += blockDim.x) {
    const int hh = e / (ST * 32), sl = e - hh * ST * 32;
    dnl[e] = sl < S ? d_norm[((int64_t)b * H + hh) * S + sl] : 0.f;
  }
  const float inv_t = 1.f / clamp_temperature(temperature[h]);
  float tsum = 0.f;
  __syncthreads();

  for (int t = blockIdx.x; t < tpb; t += gridDim.x) {
    const int64_t n = (int64_t)t * 32 + i;
    const bool ok = n < N;
    const int64_t row = (int64_t)b * N + (ok ? n : N - 1);
    const int64_t base = row * HD + h * 32 + 8 * g;
    u32x4 xm[2], fm[2], gg[2], wq[NCH];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      xm[kk] = *reinterpret_cast<const u32x4 *>(x_mid + base + 16 * kk);
      fm[kk] = *reinterpret_cast<const u32x4 *>(fx_mid + base + 16 * kk);
      gg[kk] = *reinterpret_cast<const u32x4 *>(d_out_x + base + 16 * kk);
    }
    {
      const u32x4 *wsrc = w_pack + ((((int64_t)b * tpb + t) * H + h) * NCH) * 64 + lane;
#pragma unroll
      for (int cq = 0; cq < NCH; ++cq) wq[cq] = load_streaming(wsrc + cq * 64);
    }
    // w of this lane's (point, slices): chunk cq = 2st + half holds registers 8 half .. 8 half + 7 as bf16
    auto w_of = [&](int st, int r) {
      const int cq = 2 * st + (r >> 3), j = r & 7;
      if (cq >= NCH) return 0.f;
      const uint32_t pair = wq[cq][j >> 1];
      return __uint_as_float((j & 1) ? (pair & 0xffff0000u) : (pair << 16));
    };
    // per point: dot = sum_s w dw;  sum_s dz z = (sum_s w dw z - dot sum_s w z) / T: the logits of a slice tile are
    // consumed as soon as they exist, only d w stays live across the tiles
    f32x16 dw[ST];
    float dot = 0.f, a1 = 0.f, a2 = 0.f, wsum = 0.f;
#pragma unroll
    for (int st = 0; st < ST; ++st) {
      f32x16 z;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        z[r] = bsl[32 * st + rowmap(r, g)];
        dw[st][r] = dnl[(h * ST + st) * 32 + rowmap(r, g)];
      }
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        z = mma(wsh[(st * 2 + kk) * 64 + lane], xm[kk], z);
        if constexpr (LDSTAB) {
          dw[st] = mma(mytab[(st * 2 + kk) * 64], gg[kk], dw[st]);
          dw[st] = mma(mytab[(ST2 + st * 2 + kk) * 64], fm[kk], dw[st]);
        } else {
          dw[st] = mma(tokA[st * 2 + kk], gg[kk], dw[st]);
          dw[st] = mma(dnA[st * 2 + kk], fm[kk], dw[st]);
        }
      }
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float w = w_of(st, r);
        const float wd = w * dw[st][r];
        dot += wd;
        wsum += w;
        a1 = fmaf(wd, z[r], a1);
        a2 = fmaf(w, z[r], a2);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    // the bf16 weights of a point do not sum to one exactly: dividing by their sum keeps sum_s d z = 0, without which
    // the defect times the common offset of the logits leaks into d temperature and d bias
    wsum = half_sum(wsum);
    dot = wsum > 0.f ? half_sum(dot) / wsum : 0.f;
    tsum += (a1 - dot * a2) * inv_t;  // a1, a2 are this lane's halves; the halves add up in the final wave sum
    f32x16(&dz)[ST] = dw;  // d z replaces d w in place
#pragma unroll
    for (int st = 0; st < ST; ++st)
#pragma unroll
      for (int r = 0; r < 16; ++r) dz[st][r] = w_of(st, r) * inv_t * (dw[st][r] - dot);
    __builtin_amdgcn_sched_barrier(0);
    f32x16 dxm, dfm;
#pragma unroll
    for (int r = 0; r < 16; ++r) dxm[r] = dfm[r] = 0.f;
#pragma unroll
    for (int cq = 0; cq < NCH; ++cq) {
      const u32x4 dzp = (cq & 1) ? pack_half<1>(dz[cq >> 1]) : pack_half<0>(dz[cq >> 1]);
      dxm = mma(wsh[(ST2 + cq) * 64 + lane], dzp, dxm);
      dfm = mma(dnT[cq], wq[cq], dfm);
    }
    const int64_t orow = (int64_t)b * N + (ok ? n : 0);
    uint16_t *pr = d_proj + orow * 2 * HD + h * 32;
    store_tile_natural(dxm, pr, g, ok);
    store_tile_natural(dfm, pr + HD, g, ok);
#pragma unroll
    for (int st = 0; st < ST; ++st)
      store_tile_natural(dz[st], d_z + (orow * H + h) * S + 32 * st, g, ok, S - 32 * st >= 32 ? 32 : 16);
  }
  // d T of this (workgroup, head): every lane holds part of the sum over its points and slices
  tsum = wave_sum(tsum);
  if (lane == 0) dT_part[((int64_t)blockIdx.y * gridDim.x + blockIdx.x) * H + h] = -tsum * inv_t;  // heads: disjoint
}

// ================================================================================================
// host side
// ================================================================================================
bool backward_supported(const pa_shape &s) { return supported(PA_BF16, s); }

int64_t backward_groups(const pa_shape &s, int num_cu) {
  int64_t g = (2 * (int64_t)num_cu + s.B - 1) / s.B;
  const int64_t tpb = tiles_per_batch(s);
  if (g > tpb) g = tpb;
  return g < 1 ? 1 : g;
}

int64_t backward_tables_bytes(const pa_shape &s) {
  const BwdTablePlan tp = bwd_table_plan((int)s.S);
  return (tp.shared_units + s.B * s.H * tp.per_head_units) * 16;
}

int deslice_natural(const pa_shape &s, const void *w_pack, const void *tokp, void *out_x, int num_cu, hipStream_t st) {
  const int waves = (int)(s.H < 8 ? s.H : 8);
  if (s.H % waves != 0) return PA_ERR_UNSUPPORTED;
  const int groups = (int)(s.H / waves);
  int64_t gx = backward_groups(s, num_cu) / groups;
  if (gx < 1) gx = 1;
  const dim3 grid((unsigned)gx, (unsigned)s.B, (unsigned)groups), block((unsigned)(waves * 64));
  const u32x4 *wp = static_cast<const u32x4 *>(w_pack), *tp = static_cast<const u32x4 *>(tokp);
  uint16_t *ox = static_cast<uint16_t *>(out_x);
  const int tpb = (int)tiles_per_batch(s);
  switch (s.S) {
    case 16: hipLaunchKernelGGL((deslice_natural_kernel<16>), grid, block, 0, st, wp, tp, ox, s.N, tpb, (int)s.H); break;
    case 32: hipLaunchKernelGGL((deslice_natural_kernel<32>), grid, block, 0, st, wp, tp, ox, s.N, tpb, (int)s.H); break;
    case 64: hipLaunchKernelGGL((deslice_natural_kernel<64>), grid, block, 0, st, wp, tp, ox, s.N, tpb, (int)s.H); break;
    case 128: hipLaunchKernelGGL((deslice_natural_kernel<128>), grid, block, 0, st, wp, tp, ox, s.N, tpb, (int)s.H); break;
    default: return PA_ERR_UNSUPPORTED;
  }
  return launch_status();
}

int slice_softmax_backward(const pa_shape &s, const pa_params &p, const void *x_mid, const void *fx_mid,
                           const void *d_out_x, const void *w_pack, const float *out_token, const float *d_num,
                           const float *d_norm, void *tables, void *d_proj, void *d_z, float *dT_part, int num_cu,
                           hipStream_t st) {
  if (!backward_supported(s)) return PA_ERR_UNSUPPORTED;
  u32x4 *tabs = static_cast<u32x4 *>(tables);
  hipLaunchKernelGGL(backward_tables_kernel, dim3(64), dim3(256), 0, st, p.in_project_slice_weight, out_token, d_num, tabs,
                     (int)(s.B * s.H), (int)s.S);
  int rc = launch_status();
  if (rc) return rc;
  // S = 128: 4 waves (heads) per workgroup, one wave per SIMD, their tok' / d num fragments in (dynamic) LDS
  const int waves = (int)(s.S > 64 ? 4 : s.H);
  const int groups = (int)(s.H / waves);
  const dim3 grid((unsigned)backward_groups(s, num_cu), (unsigned)s.B, (unsigned)groups), block((unsigned)(waves * 64));
  const int tpb = (int)tiles_per_batch(s);
  const size_t lds = s.S > 64 ? (size_t)waves * 2 * 2 * ((s.S + 31) / 32) * 64 * 16 : 0;
  if ((rc = allow_dynamic_lds(slice_softmax_backward_mfma_kernel<128>, lds))) return rc;
#define PA_LAUNCH_BWD(SS)                                                                                              \
  hipLaunchKernelGGL((slice_softmax_backward_mfma_kernel<SS>), grid, block, lds, st, static_cast<const uint16_t *>(x_mid), \
                     static_cast<const uint16_t *>(fx_mid), static_cast<const uint16_t *>(d_out_x),                     \
                     static_cast<const u32x4 *>(w_pack), tabs, d_norm, p.in_project_slice_bias, p.temperature,          \
                     static_cast<uint16_t *>(d_proj), static_cast<uint16_t *>(d_z), dT_part, s.N, tpb, (int)s.H)
  switch (s.S) {
    case 16: PA_LAUNCH_BWD(16); break;
    case 32: PA_LAUNCH_BWD(32); break;
    case 64: PA_LAUNCH_BWD(64); break;
    case 128: PA_LAUNCH_BWD(128); break;
    default: return PA_ERR_UNSUPPORTED;
  }
#undef PA_LAUNCH_BWD
  return launch_status();
}

}  // namespace mfma
}  // namespace pa
