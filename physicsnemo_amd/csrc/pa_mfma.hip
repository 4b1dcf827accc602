// bf16 MFMA kernels for the irregular-mesh PhysicsAttention layer on gfx950 (D = 32, C = H*32 in {128, 256},
// S in {16, 32, 64, 128}).  v_mfma_f32_32x32x16_bf16 everywhere, fp32 accumulation.
//
// Work unit: a TILE of 32 consecutive points of one batch, owned by one wavefront.
//
// MFMA register layouts used below (lane = 32*g + i, i = lane % 32, g = lane / 32):
//   A operand (32 x 16): lane holds row i, k = 8g + j, j = 0..7.      B operand (16 x 32): column i, k = 8g + j.
//   C/D (32 x 32): lane holds column i; register r = 0..15 is row  rowmap(r, g) = 8*(r/4) + 4*g + r%4.
// A C/D tile converted to bf16 is therefore directly a pair of A (or B) operands of a following MFMA whose
// reduction index is the C/D ROW index, taken in the order
//   kperm(kk, g, j) = 16*kk + 8*(j/4) + 4*g + j%4          (kk = 0, 1 selects registers 8kk .. 8kk+7)
// provided the other operand is loaded with the same permutation.  All chained products below rely on this;
// no shuffles or LDS transposes are needed between the GEMMs of one kernel.
//
// Intermediates between kernels are stored in that register order ("packed"), 16 bytes per lane, 1 KiB per wave
// store, so every global access of the three big kernels is a full-width coalesced transaction:
//   w_pack [tile][h][cq][lane][8]  slice weights, chunk cq = 16 slices: element j <-> slice 16cq + 8(j/4) + 4g + j%4
//                                  of point i of the tile                       (B operand of the deslice product)
//   fx_pack[tile][h][kk][lane][8]  fx_mid, lane i <-> channel d = i of head h, element j <-> point kperm(kk, g, j)
//                                                                                (A operand of the aggregation)
#include "pa_common.h"
#include "pa_host.h"
#include "pa_mfma_ops.h"

namespace pa {
namespace mfma {

// ------------------------------------------------------------------------------------------------
// Packed parameter blob (built once per parameter set by pack_params_kernel).  Offsets in 16-byte units.
//   win [h][m][ks][lane]  m = 0: in_project_x, 1: in_project_fx; W_m[h*32 + i][16ks + 8g + j]
//   wsl [st][kk][lane]    in_project_slice[32st + i][kperm(kk, g, j)]   (0 beyond S)
//   wout[ct][h][kk][lane] out_linear[32ct + i][h*32 + kperm(kk, g, j)],  ct < C/32
//   then float vectors (offsets in floats from fvec): bias_fx[C]; bias_logit[H][ST*32] = the slice bias with the bias
//   of in_project_x folded in, b_slice[s] + sum_d W_slice[s][d] * b_x[h*32 + d] (-1e30 beyond S); bias_out[C];
//   tscale[H] = log2(e) / clamp(temperature)
// The projection kernel therefore forms x_mid and fx_mid WITHOUT their biases: the one of x_mid reaches the slice
// logits through bias_logit, the one of fx_mid is added to the slice tokens after the aggregation
// (sum_n w (fx + b) = sum_n w fx + b sum_n w).
// ------------------------------------------------------------------------------------------------
struct BlobPlan {
  int64_t win, wsl, wout, fvec, total_units;  // 16-byte units
  int f_bias_fx, f_bias_logit, f_bias_out, f_tscale, nfloat;  // float offsets from fvec
};

__host__ __device__ inline BlobPlan blob_plan(int C, int S) {
  const int H = C / 32, KS = C / 16, ST = (S + 31) / 32, CT = C / 32;
  BlobPlan p;
  p.win = 0;
  p.wsl = p.win + (int64_t)H * 2 * KS * 64;
  p.wout = p.wsl + (int64_t)ST * 2 * 64;
  p.fvec = p.wout + (int64_t)CT * H * 2 * 64;
  p.f_bias_fx = 0;
  p.f_bias_logit = C;
  p.f_bias_out = p.f_bias_logit + H * ST * 32;
  p.f_tscale = p.f_bias_out + C;
  p.nfloat = p.f_tscale + H;
  p.total_units = p.fvec + (p.nfloat + 3) / 4;
  return p;
}

// only_out: fill in the out_linear part alone (wout, bias_out), which is all kernel (d) reads; nothing else of p is touched
__global__ __launch_bounds__(256) void pack_params_kernel(pa_params p, u32x4 *__restrict__ blob, int C, int S, int only_out) {
  const int H = C / 32, KS = C / 16, ST = (S + 31) / 32;
  const BlobPlan bp = blob_plan(C, S);
  // the three large weights: bf16 bits, or fp8-e4m3 bytes with per-row scales when the parameter set carries scales
  const WeightView wx{p.in_project_x_weight, p.in_project_x_scale, C}, wfx{p.in_project_fx_weight, p.in_project_fx_scale, C},
      wo{p.out_linear_weight, p.out_linear_scale, C};
  const int64_t n_units = bp.fvec;
  for (int64_t u = (only_out ? bp.wout : 0) + (int64_t)blockIdx.x * 256 + threadIdx.x; u < n_units; u += (int64_t)gridDim.x * 256) {
    const int lane = (int)(u & 63), i = lane & 31, g = lane >> 5;
    uint32_t e[4];
    if (u < bp.wsl) {
      int64_t q = u >> 6;
      const int ks = (int)(q % KS);
      q /= KS;
      const int m = (int)(q & 1), h = (int)(q >> 1);
      weight_bits8(m ? wfx : wx, h * 32 + i, 16 * ks + 8 * g, e);
    } else if (u < bp.wout) {
      const int q = (int)((u - bp.wsl) >> 6);
      const int kk = q & 1, st = q >> 1;
      const int s = 32 * st + i;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint16_t lo = s < S ? to_bf16_bits(p.in_project_slice_weight[(int64_t)s * 32 + kperm(kk, g, 2 * j)]) : (uint16_t)0;
        const uint16_t hi = s < S ? to_bf16_bits(p.in_project_slice_weight[(int64_t)s * 32 + kperm(kk, g, 2 * j + 1)]) : (uint16_t)0;
        e[j] = (uint32_t)lo | ((uint32_t)hi << 16);
      }
    } else {
      int q = (int)((u - bp.wout) >> 6);
      const int kk = q & 1;
      q >>= 1;
      const int h = q % H, ct = q / H;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        e[j] = (uint32_t)weight_bits(wo, ct * 32 + i, h * 32 + kperm(kk, g, 2 * j)) |
               ((uint32_t)weight_bits(wo, ct * 32 + i, h * 32 + kperm(kk, g, 2 * j + 1)) << 16);
    }
    blob[u] = u32x4{e[0], e[1], e[2], e[3]};
  }
  float *fv = reinterpret_cast<float *>(blob + bp.fvec);
  for (int k = (only_out ? bp.f_bias_out : 0) + blockIdx.x * 256 + threadIdx.x; k < (only_out ? bp.f_tscale : bp.nfloat);
       k += gridDim.x * 256) {
    float v;
    if (k < bp.f_bias_logit) {
      v = p.in_project_fx_bias[k];
    } else if (k < bp.f_bias_out) {
      const int q = k - bp.f_bias_logit, h = q / (ST * 32), sidx = q - h * (ST * 32);
      if (sidx < S) {
        v = p.in_project_slice_bias[sidx];
        for (int d = 0; d < 32; ++d) v = fmaf(p.in_project_slice_weight[sidx * 32 + d], p.in_project_x_bias[h * 32 + d], v);
      } else {
        v = -1e30f;
      }
    } else if (k < bp.f_tscale) {
      v = p.out_linear_bias[k - bp.f_bias_out];
    } else {
      v = kLog2e / clamp_temperature(p.temperature[k - bp.f_tscale]);
    }
    fv[k] = v;
  }
}

// ------------------------------------------------------------------------------------------------
// Kernel (a): projections + slice logits + temperature softmax, weights-stationary; optionally fused with the
// first pass of the slice-token aggregation (FUSED).
//   x_mid^T (32 ch x 32 pts) = Wx_h . x^T          A = Wx_h frags (registers), B = x frags (LDS)
//   fx_mid  (32 pts x 32 d)  = x . Wfx_h^T         A = x frags (LDS),          B = Wfx_h frags (registers)
//   logits^T(32 s x 32 pts)  = Wslice . x_mid^T    A = Wslice frags (LDS), B = bf16(x_mid^T) straight from registers
//   softmax over s: in-lane over the accumulator registers plus one exchange with lane^32               -> w_pack
//   !FUSED: fx_mid -> fx_pack (kernel (b) aggregates later)
//    FUSED: w^T (lanes <-> slices, registers <-> points) = w_chunk . SEL  (an exact MFMA "transpose"),
//           tok^T_h (32 d x S) += bf16(fx_mid)^T . w^T, norm_h += sum_n w in per-head accumulators that stay in
//           registers for the whole kernel (a wave owns its head, so there is no cross-wave reduction) and leave
//           as one partial per workgroup: partials[g][b][h][s][0..D-1] = sum_n w fx_mid, [..][D] = sum_n w
//           (layout of the combine kernel).
// Both biases of the projections are applied elsewhere (see the parameter blob).
// Grid (G workgroups per batch, B); workgroup (g, b) walks the tile sets g, g+G, ... of batch b, H waves (two per
// SIMD for C = 256).  Wave h owns head h and keeps its Wx | Wfx fragments (2 * KS * 4 = 128 registers for C = 256)
// in registers for the whole kernel: after the prologue there is no weight traffic at all.
// The x rows of a SET of TS tiles are staged in LDS by direct global -> LDS loads (no registers, no LDS write
// instructions): one wave load moves 64 x 16 bytes = RPC rows to 1 KiB of contiguous LDS.  A tile is NCK = 32 / RPC
// such chunks, chunk c holding rows c, c + NCK, ...; chunks lie 65 units apart, so unit u of row r sits at
// (r % NCK) * 65 + (r / NCK) * UPR + u.  For C = 256 (NCK = 16) the 16 lanes of a 128-bit access (rows i..i+15, same
// unit) cover all 64 banks, and every fragment address is one base register plus an immediate offset.  One fragment
// read (1 KiB) feeds two MFMAs.  The set buffers are double buffered; the loads of the next set are issued one tile
// at a time at the start of a tile; one barrier per set.  The loop over sets is the only loop; its body has no
// branch around a global memory operation (slots past the last tile of the batch recompute it and re-store
// identical values; they add nothing to the aggregation).
// ------------------------------------------------------------------------------------------------

// One direct global -> LDS load of 64 x 16 bytes: lane l reads sbase + voff(l) and its data land at LDS byte address
// lds + 16 l.  sbase and lds are wave-uniform.  Asynchronous, counted by vmcnt like any load.
__device__ __forceinline__ void load_row_chunk_to_lds(const void *sbase, unsigned voff, unsigned lds) {
  asm volatile(
      "s_mov_b32 m0, %2\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %1, %0" ::"s"(sbase),
      "v"(voff), "s"(lds)
      : "memory");
}

// CLOCKED: the workgroup in the middle of the grid also reports how long it ran, in shader cycles (s_memtime) and in
// ticks of the 100 MHz wall clock: clock_out[0], clock_out[1].  Their ratio is the shader clock the chip held under
// this very kernel; everything else is the same code (two scalar reads at the start, one store at the end).
template <int C, int S, bool FUSED, bool CLOCKED>
__device__ __forceinline__ void project_softmax_body(const u32x4 *__restrict__ blob, const uint16_t *__restrict__ x,
                                                     u32x4 *__restrict__ fx_pack, u32x4 *__restrict__ w_pack,
                                                     float *__restrict__ partials, int64_t N, int tpb,
                                                     uint64_t *__restrict__ clock_out) {
  constexpr int H = C / 32, KS = C / 16, ST = (S + 31) / 32, NCH = S / 16, D1 = 33;
  constexpr int WAVES = H, NT = WAVES * 64;
  constexpr int TS = 4;                 // tiles per set
  constexpr int UPR = C / 8;            // 16-byte units per row
  constexpr int RPC = 64 / UPR;         // rows per chunk (one wave load)
  constexpr int NCK = 32 / RPC;         // chunks per tile
  constexpr int TILE_UNITS = NCK * 65;
  constexpr int SET_UNITS = TS * TILE_UNITS;
  constexpr int CPW = NCK / WAVES;      // chunks per wave and tile
  constexpr int STORES_PER_TILE = NCH + (FUSED ? 0 : 2);
  static_assert(NCK % WAVES == 0, "the chunks of a tile must split evenly over the waves");
  extern __shared__ u32x4 smem[];
  u32x4 *xs = smem;                     // 2 * SET_UNITS
  u32x4 *wsl = xs + 2 * SET_UNITS;      // ST * 2 * 64
  u32x4 *sel = wsl + ST * 2 * 64;       // 4 * 64: the 0/1 selection matrices of the MFMA transpose + two zero ones
  float *fvec = reinterpret_cast<float *>(sel + 4 * 64);
  const BlobPlan bp = blob_plan(C, S);
  const int tid = threadIdx.x, lane = tid & 63, i = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: addresses derived from it stay scalar
  const int h = wave;
  const int b = blockIdx.y;
  uint64_t cycles0 = 0, ticks0 = 0;
  if constexpr (CLOCKED) {
    cycles0 = __builtin_readcyclecounter();
    ticks0 = wall_clock64();
  }
  const float *bias_s = fvec + bp.f_bias_logit + h * (ST * 32), *tscale = fvec + bp.f_tscale;

  u32x4 wx[KS], wf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int64_t base = bp.win + ((int64_t)h * 2) * KS * 64;
    wx[ks] = blob[base + ks * 64 + lane];
    wf[ks] = blob[base + (KS + ks) * 64 + lane];
  }
  for (int u = tid; u < ST * 2 * 64; u += NT) wsl[u] = blob[bp.wsl + u];
  {
    const float *src = reinterpret_cast<const float *>(blob + bp.fvec);
    for (int k = tid; k < bp.nfloat; k += NT) fvec[k] = src[k];
  }
  // per-head accumulators of the aggregation: tokacc[st][r] = sum_n w[n, 32st + i] fx_mid[n, rowmap(r, g)],
  // nrmacc[st] = this half-wave's share of sum_n w[n, 32st + i]
  f32x16 tokacc[ST];
  float nrmacc[ST];
#pragma unroll
  for (int st = 0; st < ST; ++st) {
    nrmacc[st] = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) tokacc[st][r] = 0.f;
  }
  if constexpr (FUSED) {
    if (tid < 256) {  // the two 0/1 selection matrices of the MFMA transpose, then two all-zero ones
      const int par = (tid >> 6) & 1;
      bf16x8 s8;
#pragma unroll
      for (int j = 0; j < 8; ++j) s8[j] = (__bf16)((tid < 128 && i == kperm(par, g, j)) ? 1.f : 0.f);
      sel[tid] = __builtin_bit_cast(u32x4, s8);
    }
  }

  const int nsets = (tpb + TS - 1) / TS;  // per batch
  const int nloc = (nsets - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x;
  const uint16_t *xbatch = x + (int64_t)b * N * C;
  const int rows_last = (int)(N - (int64_t)(tpb - 1) * 32);  // rows of the batch's last tile
  // staging: this wave's CPW chunks of tile `tile` of the batch into slot t of buffer buf.  Lane l of chunk c fetches
  // unit l % UPR of row c + NCK * (l / UPR); rows beyond N re-read row 0 of the tile (their weights are zeroed later).
  const int srow = lane / UPR, sunit = lane % UPR;
  auto stage = [&](int tile, int buf, int t) {
    const int tl = tile < tpb ? tile : tpb - 1;
    const uint16_t *xbase = xbatch + (int64_t)tl * 32 * C;
    const int rows_ok = tl == tpb - 1 ? rows_last : 32;
#pragma unroll
    for (int k = 0; k < CPW; ++k) {
      const int c = wave * CPW + k;
      int row = c + NCK * srow;
      row = row < rows_ok ? row : 0;
      const unsigned lds = (unsigned)(uintptr_t)(xs + buf * SET_UNITS + t * TILE_UNITS + c * 65);
      load_row_chunk_to_lds(xbase, (unsigned)(row * C + sunit * 8) * 2u, lds);
    }
  };
#pragma unroll
  for (int t = 0; t < TS; ++t) stage((int)blockIdx.x * TS + t, 0, t);  // first set
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  // A tile is worked on in two halves.
  //   MFMA half:   aggregation products of the tile before (operands left by its vector half), then the two
  //                projections of this tile, their results packed to bf16 operands.  Every MFMA here is independent
  //                of vector work, so the matrix pipe is fed back to back; registers: accumulators + fragment ring.
  //   vector half: slice logits (4 short MFMAs), softmax over the slices of each point in the base-2 domain,
  //                w = exp2((l - max) * log2e / T) / sum, the store of w_pack, the MFMA "transpose" of the weights,
  //                slice norms, and the transposed weights packed as operands of the next MFMA half.
  struct Tile {  // left by the MFMA half
    u32x4 xb0, xb1;    // x_mid^T as B operands of the logits
    u32x4 fx0, fx1;    // fx_mid^T as A operands of the aggregation
    int64_t tile;      // global tile index (b * tpb + tile in batch)
    bool dup;          // a slot past the batch's last tile: recomputed, contributes nothing to the aggregation
    bool valid;        // this lane's point exists
  };
  struct Agg {  // left by the vector half: operands of the aggregation products
    u32x4 tp[ST][2];
    u32x4 fx0, fx1;
  };
  auto aggregate = [&](const Agg &ag) {
    if constexpr (FUSED) {
#pragma unroll
      for (int st = 0; st < ST; ++st) tokacc[st] = mma(ag.fx0, ag.tp[st][0], tokacc[st]);
#pragma unroll
      for (int st = 0; st < ST; ++st) tokacc[st] = mma(ag.fx1, ag.tp[st][1], tokacc[st]);
    }
  };
  auto mfma_half = [&](int buf, int t, int slot, Tile &tl, const Agg &ag) {
    __builtin_amdgcn_s_setprio(3);  // goes first: its issue slots are few and feed the matrix pipe
    tl.dup = slot >= tpb;
    const int tb = tl.dup ? tpb - 1 : slot;
    tl.tile = (int64_t)b * tpb + tb;
    tl.valid = (int64_t)tb * 32 + i < N;
    const u32x4 *xb = xs + buf * SET_UNITS + t * TILE_UNITS + (i % NCK) * 65 + (i / NCK) * UPR + g;
    // x fragments are read AHEAD k-steps before the MFMAs that use them
    constexpr int RING = 4, AHEAD = RING - 1;
    u32x4 xf[RING];
#pragma unroll
    for (int q = 0; q < AHEAD; ++q) xf[q] = xb[2 * q];
    __builtin_amdgcn_sched_barrier(0);
    aggregate(ag);
    __builtin_amdgcn_sched_barrier(0);
    f32x16 ax, af;
#pragma unroll
    for (int r = 0; r < 16; ++r) ax[r] = af[r] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (ks + AHEAD < KS) xf[(ks + AHEAD) % RING] = xb[2 * (ks + AHEAD)];
      ax = mma(wx[ks], xf[ks % RING], ax);
      af = mma(xf[ks % RING], wf[ks], af);
      __builtin_amdgcn_sched_barrier(0);  // keeps the compiler from sinking the reads back next to their uses
    }
    tl.xb0 = pack_half<0>(ax);
    tl.xb1 = pack_half<1>(ax);
    tl.fx0 = pack_half<0>(af);
    tl.fx1 = pack_half<1>(af);
    if constexpr (!FUSED) {
      u32x4 *fdst = fx_pack + ((tl.tile * H + h) * 2) * 64 + lane;
      store_streaming(fdst, tl.fx0);
      store_streaming(fdst + 64, tl.fx1);
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  auto vector_half = [&](const Tile &tl, Agg &ag) {
    __builtin_amdgcn_s_setprio(0);  // fills the issue slots the other wave of the SIMD leaves
    f32x16 lg[ST];
#pragma unroll
    for (int st = 0; st < ST; ++st) {
#pragma unroll
      for (int r = 0; r < 16; ++r) lg[st][r] = bias_s[32 * st + rowmap(r, g)];
    }
#pragma unroll
    for (int st = 0; st < ST; ++st) lg[st] = mma(wsl[(st * 2 + 0) * 64 + lane], tl.xb0, lg[st]);
#pragma unroll
    for (int st = 0; st < ST; ++st) lg[st] = mma(wsl[(st * 2 + 1) * 64 + lane], tl.xb1, lg[st]);
    // one maximum chain per slice tile: the chain of the first tile runs while the MFMAs of the second complete
    float mx = -INFINITY;
#pragma unroll
    for (int r = 0; r < 16; ++r) mx = fmaxf(mx, lg[0][r]);
    if constexpr (ST > 1) {
      float mx2 = -INFINITY;
#pragma unroll
      for (int st = 1; st < ST; ++st)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx2 = fmaxf(mx2, lg[st][r]);
      mx = fmaxf(mx, mx2);
    }
    mx = half_max(mx);
    const float sc = tscale[h];
    const float off = mx * sc;
    float sum[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int st = 0; st < ST; ++st)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float e = __builtin_amdgcn_exp2f(fmaf(lg[st][r], sc, -off));
        lg[st][r] = e;
        sum[r & 3] += e;
      }
    const float tot = half_sum((sum[0] + sum[1]) + (sum[2] + sum[3]));
    const float inv = tl.valid ? __builtin_amdgcn_rcpf(tot) : 0.f;  // rows beyond N get zero weight
    u32x4 wp[2 * ST];
#pragma unroll
    for (int st = 0; st < ST; ++st) {
      wp[2 * st] = pack_half<0>(lg[st], inv);
      wp[2 * st + 1] = pack_half<1>(lg[st], inv);
    }
    u32x4 *wdst = w_pack + ((tl.tile * H + h) * NCH) * 64 + lane;
#pragma unroll
    for (int cq = 0; cq < NCH; ++cq) store_streaming(wdst + cq * 64, wp[cq]);
    if constexpr (FUSED) {
      // transposed weights (lanes <-> slices, registers <-> points); a slot past the batch's last tile multiplies by
      // the all-zero selection matrices instead and so adds nothing
      const u32x4 *sl = sel + (tl.dup ? 2 * 64 : 0) + lane;
      const u32x4 sel0 = sl[0], sel1 = sl[64];
      f32x16 tr[ST];
#pragma unroll
      for (int st = 0; st < ST; ++st) {
#pragma unroll
        for (int r = 0; r < 16; ++r) tr[st][r] = 0.f;
        tr[st] = mma(wp[2 * st], sel0, tr[st]);
      }
      if constexpr (NCH > 1) {
#pragma unroll
        for (int st = 0; st < ST; ++st) tr[st] = mma(wp[2 * st + 1], sel1, tr[st]);
      }
#pragma unroll
      for (int st = 0; st < ST; ++st) {
        float s0 = tr[st][0] + tr[st][1], s1 = tr[st][2] + tr[st][3];
#pragma unroll
        for (int r = 4; r < 16; r += 4) {
          s0 += tr[st][r] + tr[st][r + 1];
          s1 += tr[st][r + 2] + tr[st][r + 3];
        }
        nrmacc[st] += s0 + s1;
        ag.tp[st][0] = pack_half<0>(tr[st]);
        ag.tp[st][1] = pack_half<1>(tr[st]);
      }
      ag.fx0 = tl.fx0;
      ag.fx1 = tl.fx1;
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  auto wait_staged = [&]() {
    // the loads of the next set have landed once at most the stores of the last tile are still in flight
    if constexpr (STORES_PER_TILE == 1) asm volatile("s_waitcnt vmcnt(1)" ::: "memory");
    else if constexpr (STORES_PER_TILE == 2) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
    else if constexpr (STORES_PER_TILE == 3) asm volatile("s_waitcnt vmcnt(3)" ::: "memory");
    else if constexpr (STORES_PER_TILE == 4) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
    else if constexpr (STORES_PER_TILE == 6) asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
    else if constexpr (STORES_PER_TILE == 8) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  };
  // The two waves of a SIMD (waves w and w + 4 of an 8-wave workgroup) run the halves out of phase: the upper four
  // go MFMA half, then vector half of the same tile; the lower four start with the vector half of the tile before.
  // Between two barriers one wave of each SIMD is then feeding the matrix pipe while the other fills the issue slots
  // it leaves (lower priority) with vector work.  Both orders stage the next set at the same places and meet at the
  // same barriers.
  const bool lower = WAVES == 8 && wave < 4;
  // nothing to finish before the first tile: placeholders with zero operands; the w_pack store of the placeholder
  // tile (lower waves) lands on this workgroup's first tile with zero weights and is overwritten there by the real
  // one (same lanes, same addresses, later in program order); it is marked as a slot that adds nothing
  Tile tl;
  Agg ag;
#pragma unroll
  for (int st = 0; st < ST; ++st) ag.tp[st][0] = ag.tp[st][1] = u32x4{0, 0, 0, 0};
  ag.fx0 = ag.fx1 = u32x4{0, 0, 0, 0};
  tl.xb0 = tl.xb1 = tl.fx0 = tl.fx1 = u32x4{0, 0, 0, 0};
  tl.tile = (int64_t)b * tpb + min((int)blockIdx.x * TS, tpb - 1);
  tl.dup = true;
  tl.valid = false;
  int set = blockIdx.x;
  if (!lower) {
    for (int sl = 0; sl < nloc; ++sl) {
      const int buf = sl & 1;
      const int set_next = set + (int)gridDim.x < nsets ? set + (int)gridDim.x : set;  // the last set re-fetches itself
#pragma unroll
      for (int t = 0; t < TS; ++t) {
        __builtin_amdgcn_sched_barrier(0);  // keep each tile's work (and its register live ranges) to itself
        stage(set_next * TS + t, buf ^ 1, t);
        __builtin_amdgcn_sched_barrier(0);
        mfma_half(buf, t, set * TS + t, tl, ag);
        vector_half(tl, ag);
        __builtin_amdgcn_sched_barrier(0);
      }
      set = set_next;
      wait_staged();
      __syncthreads();
    }
    aggregate(ag);
  } else {
    for (int sl = 0; sl < nloc; ++sl) {
      const int buf = sl & 1;
      const int set_next = set + (int)gridDim.x < nsets ? set + (int)gridDim.x : set;
#pragma unroll
      for (int t = 0; t < TS; ++t) {
        __builtin_amdgcn_sched_barrier(0);
        stage(set_next * TS + t, buf ^ 1, t);
        __builtin_amdgcn_sched_barrier(0);
        vector_half(tl, ag);
        mfma_half(buf, t, set * TS + t, tl, ag);
        __builtin_amdgcn_sched_barrier(0);
      }
      set = set_next;
      wait_staged();
      __syncthreads();
    }
    vector_half(tl, ag);
    aggregate(ag);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing may still be landing in LDS when the workgroup ends
  if constexpr (CLOCKED) {
    if (blockIdx.x == gridDim.x / 2 && blockIdx.y == 0 && tid == 0) {
      clock_out[0] = __builtin_readcyclecounter() - cycles0;
      clock_out[1] = wall_clock64() - ticks0;
    }
  }
  if constexpr (FUSED) {
    // this wave's head: accumulators -> partials[g][b][h][s][d], [..][D] = count
    float *dst = partials + (((int64_t)blockIdx.x * gridDim.y + b) * H + h) * (S * D1);
#pragma unroll
    for (int st = 0; st < ST; ++st) {
      const int s = 32 * st + i;
      const float nrm = half_sum(nrmacc[st]);
      if (s < S) {
#pragma unroll
        for (int r = 0; r < 16; ++r) dst[s * D1 + rowmap(r, g)] = tokacc[st][r];
        if (g == 0) dst[s * D1 + 32] = nrm;
      }
    }
  }
}

template <int C, int S, bool FUSED>
__global__ __launch_bounds__((C / 32) * 64) void project_softmax_kernel(const u32x4 *__restrict__ blob,
                                                                        const uint16_t *__restrict__ x,
                                                                        u32x4 *__restrict__ fx_pack,
                                                                        u32x4 *__restrict__ w_pack,
                                                                        float *__restrict__ partials, int64_t N, int tpb) {
  project_softmax_body<C, S, FUSED, false>(blob, x, fx_pack, w_pack, partials, N, tpb, nullptr);
}

// the fused form with the clock reading
template <int C, int S>
__global__ __launch_bounds__((C / 32) * 64) void project_softmax_clocked_kernel(const u32x4 *__restrict__ blob,
                                                                                const uint16_t *__restrict__ x,
                                                                                u32x4 *__restrict__ w_pack,
                                                                                float *__restrict__ partials, int64_t N,
                                                                                int tpb, uint64_t *__restrict__ clock_out) {
  project_softmax_body<C, S, true, true>(blob, x, nullptr, w_pack, partials, N, tpb, clock_out);
}

// ------------------------------------------------------------------------------------------------
// Kernel (b): slice-token aggregation, streaming over the packed w / fx_mid.  grid (G groups, B*H), 4 waves.
// Each wave walks every 4th tile of its group's tile range for one (batch, head):
//   w^T (32 pts x 32 s, C/D layout: lane <-> slice, registers <-> points) = w_chunk . SEL     (an exact MFMA
//       "transpose": A = stored chunk (rows = points), B = 0/1 selection matrix)
//   norm[s]  += sum of those registers                       (fp32, in lane)
//   tok^T (32 d x 32 s) += fx_chunk (A, rows = d, k = points) . bf16(w^T) (B, k = points)
// The 4 waves' accumulators are summed through LDS in wave order and written as one partial
//   partials[g][b][h][s][0..D-1] = sum_n w fx,   [..][D] = sum_n w          (layout of the general combine kernel)
// ------------------------------------------------------------------------------------------------
template <int S>
__global__ __launch_bounds__(256) void slice_reduce_kernel(const u32x4 *__restrict__ w_pack, const u32x4 *__restrict__ fx_pack,
                                                           float *__restrict__ partials, int B, int H, int tpb,
                                                           int tiles_per_group) {
  constexpr int ST = (S + 31) / 32, NCH = S / 16, D = 32, D1 = D + 1;
  extern __shared__ float red[];  // [4 waves][ST][17][64]
  const int tid = threadIdx.x, lane = tid & 63, i = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: addresses derived from it stay scalar
  const int bh = blockIdx.y, b = bh / H, h = bh - b * H;
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
  const int t_begin = blockIdx.x * tiles_per_group;
  const int t_end = min(tpb, t_begin + tiles_per_group);
  for (int t = t_begin + wave; t < t_end; t += 4) {
    const int64_t gt = (int64_t)b * tpb + t;
    const u32x4 *wsrc = w_pack + ((gt * H + h) * NCH) * 64 + lane;
    const u32x4 *fsrc = fx_pack + ((gt * H + h) * 2) * 64 + lane;
    u32x4 wf[NCH];
#pragma unroll
    for (int cq = 0; cq < NCH; ++cq) wf[cq] = load_streaming(wsrc + cq * 64);
    const u32x4 f0 = load_streaming(fsrc), f1 = load_streaming(fsrc + 64);
#pragma unroll
    for (int st = 0; st < ST; ++st) {
      f32x16 tr;
#pragma unroll
      for (int r = 0; r < 16; ++r) tr[r] = 0.f;
      tr = mma(wf[2 * st], sel[0], tr);
      if (2 * st + 1 < NCH) tr = mma(wf[2 * st + 1 < NCH ? 2 * st + 1 : 0], sel[1], tr);
      float s16 = 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) s16 += tr[r];
      nrm[st] += s16;
      tok[st] = mma(f0, pack_half<0>(tr), tok[st]);
      tok[st] = mma(f1, pack_half<1>(tr), tok[st]);
    }
  }
  float *mine = red + (size_t)wave * ST * 17 * 64;
#pragma unroll
  for (int st = 0; st < ST; ++st) {
#pragma unroll
    for (int r = 0; r < 16; ++r) mine[(st * 17 + r) * 64 + lane] = tok[st][r];
    mine[(st * 17 + 16) * 64 + lane] = nrm[st];
  }
  __syncthreads();
  float *dst = partials + (((int64_t)blockIdx.x * B + b) * H + h) * (S * D1);
  for (int e = tid; e < ST * 17 * 64; e += 256) {
    const int l = e & 63, r = (e >> 6) % 17, st = (e >> 6) / 17;
    const int s = 32 * st + (l & 31);
    if (s >= S) continue;
    if (r < 16) {
      float acc = 0.f;
#pragma unroll
      for (int w4 = 0; w4 < 4; ++w4) acc += red[(size_t)w4 * ST * 17 * 64 + e];
      dst[s * D1 + rowmap(r, l >> 5)] = acc;
    } else if (l < 32) {
      float acc = 0.f;
#pragma unroll
      for (int w4 = 0; w4 < 4; ++w4) {
        acc += red[(size_t)w4 * ST * 17 * 64 + e];
        acc += red[(size_t)w4 * ST * 17 * 64 + e + 32];
      }
      dst[s * D1 + D] = acc;
    }
  }
}

// ------------------------------------------------------------------------------------------------
// Kernel (c): normalisation of the combined sums and the per-head slice self-attention, fp32 MFMA
// (v_mfma_f32_32x32x2_f32: A lane (i, g) holds A[i][k = g], B lane (i, g) holds B[k = g][i], C/D as above).
// One workgroup per (b, h), one wave per tile of 32 slices; lane (i, g) of wave w owns slice s = 32w + i.
//   tok[s][:]  = num[s][:] / (cnt[s] + 1e-2)                                    -> slice_token, slice_norm
//   q^T, k^T, v^T (32 e x 32 s) = Wq|k|v (A) . tok^T (B: lane <-> s, k <-> d)    registers <-> e = rowmap(r, g)
//   k, v -> LDS; scores^T (keys x queries) = k (A, from LDS) . q^T: register r of q^T is directly the B operand of
//   the step whose reduction pair is d = rowmap(r, 0 / 1)
//   softmax over the keys: in-lane over registers and key tiles + one exchange with lane ^ 32
//   out^T (32 d x 32 s) = v^T (A, from LDS) . P^T: register r of P^T is directly the B operand of the step whose
//   key pair is rowmap(r, 0 / 1)                                                -> out_token (fp32), tokp (bf16,
//   A-operand order of the deslice product: tokp[b][h][cq][lane'][j] = tok'[16cq + kperm(0, g', j)][d], lane' = 32g' + d)
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ f32x16 mma32(float a, float b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

template <int S>
__global__ __launch_bounds__(64 * ((S + 31) / 32)) void slice_attention_kernel(const float *__restrict__ combined,
                                                                               const float *__restrict__ fx_bias,
                                                                               const float *__restrict__ w_qkv,
                                                                               float *__restrict__ slice_token,
                                                                               float *__restrict__ slice_norm,
                                                                               float *__restrict__ out_token,
                                                                               uint16_t *__restrict__ tokp, int heads) {
  constexpr int NTILE = (S + 31) / 32, D = 32, D1 = 33, NCH = S / 16;
  __shared__ float ks[NTILE * 32 * D1], vs[NTILE * 32 * D1];
  const int bh = blockIdx.x, tid = threadIdx.x, lane = tid & 63, i = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int s = 32 * wave + i;
  const bool live = s < S;

  const float *src = combined + ((int64_t)bh * S + (live ? s : 0)) * D1;
  const float wsum = src[D], cnt = wsum + kSliceNormEps;
  // fx_bias (H*32, or NULL): bias of in_project_fx left out of the summed fx_mid: sum_n w (fx + b) = sum_n w fx + b sum_n w
  const float *fb = fx_bias ? fx_bias + (bh % heads) * D : nullptr;
  float tk[16];  // tok[s][2kk + g]
#pragma unroll
  for (int kk = 0; kk < 16; ++kk) {
    const float num = fb ? fmaf(fb[2 * kk + g], wsum, src[2 * kk + g]) : src[2 * kk + g];
    tk[kk] = live ? num / cnt : 0.f;
  }
  if (live) {
    if (slice_token) {
#pragma unroll
      for (int kk = 0; kk < 16; ++kk) slice_token[((int64_t)bh * S + s) * D + 2 * kk + g] = tk[kk];
    }
    if (slice_norm && g == 0) slice_norm[(int64_t)bh * S + s] = cnt;
  }

  f32x16 qT, kT, vT;
#pragma unroll
  for (int r = 0; r < 16; ++r) qT[r] = kT[r] = vT[r] = 0.f;
#pragma unroll
  for (int kk = 0; kk < 16; ++kk) {
    const float *wr = w_qkv + i * D + 2 * kk + g;  // row e = 32m + i of Wqkv, column d = 2kk + g
    qT = mma32(wr[0], tk[kk], qT);
    kT = mma32(wr[32 * D], tk[kk], kT);
    vT = mma32(wr[64 * D], tk[kk], vT);
  }
  // q scaled for a base-2 softmax: exp(x / sqrt(D)) = exp2(x * log2e / sqrt(D))
  const float qscale = kLog2e * 0.17677669529663687f;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    qT[r] *= qscale;
    ks[s * D1 + rowmap(r, g)] = kT[r];
    vs[s * D1 + rowmap(r, g)] = vT[r];
  }
  __syncthreads();

  f32x16 sc[NTILE];  // scores^T: lane <-> my query, register r <-> key 32tt + rowmap(r, g)
#pragma unroll
  for (int tt = 0; tt < NTILE; ++tt) {
#pragma unroll
    for (int r = 0; r < 16; ++r) sc[tt][r] = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) sc[tt] = mma32(ks[(32 * tt + i) * D1 + rowmap(r, g)], qT[r], sc[tt]);
  }
  float mx = -INFINITY;
#pragma unroll
  for (int tt = 0; tt < NTILE; ++tt)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      if constexpr (S % 32 != 0) {
        if (32 * tt + rowmap(r, g) >= S) sc[tt][r] = -INFINITY;  // keys beyond S
      }
      mx = fmaxf(mx, sc[tt][r]);
    }
  mx = half_max(mx);
  float sum = 0.f;
#pragma unroll
  for (int tt = 0; tt < NTILE; ++tt)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      sc[tt][r] = __builtin_amdgcn_exp2f(sc[tt][r] - mx);
      sum += sc[tt][r];
    }
  sum = half_sum(sum);

  f32x16 oT;  // out^T: lane <-> my query, register r <-> d = rowmap(r, g)
#pragma unroll
  for (int r = 0; r < 16; ++r) oT[r] = 0.f;
#pragma unroll
  for (int tt = 0; tt < NTILE; ++tt)
#pragma unroll
    for (int r = 0; r < 16; ++r) oT = mma32(vs[(32 * tt + rowmap(r, g)) * D1 + i], sc[tt][r], oT);
  const float inv = 1.f / sum;
  if (live) {
    float *dst = out_token + ((int64_t)bh * S + s) * D;
    const int cq = s >> 4, ss = s & 15, gp = (ss >> 2) & 1, j = 4 * (ss >> 3) + (ss & 3);
    uint16_t *pk = tokp + (((int64_t)bh * NCH + cq) * 64 + 32 * gp) * 8 + j;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float o = oT[r] * inv;
      dst[rowmap(r, g)] = o;
      pk[rowmap(r, g) * 8] = to_bf16_bits(o);
    }
  }
}

// ------------------------------------------------------------------------------------------------
// Kernel (d): deslice + out_linear (+ residual, + LayerNorm).  Persistent workgroups of H waves; one 32-point
// tile per iteration, worked on by the whole workgroup:
//   wave h   : out_x^T_h (32 d x 32 pts) = tok'^T_h . w^T_h   A = tokp frags (LDS, per batch), B = w_pack chunks
//              (global, fetched one tile ahead into registers)  -> bf16 A operands into LDS
//   wave ct  : y[:, 32ct .. 32ct+31] (32 pts x 32 ch) = out_x . Wout^T    A = out_x frags (LDS), B = its slice of
//              out_linear, register resident for the whole kernel        -> fp32 tile into LDS
//   wave r   : rows 32/H*r ..: + residual, rounding, LayerNorm statistics over the full row by a wave reduction,
//              full-row coalesced stores (C*2 bytes per store instruction).
// TAIL (compile time): 0 plain, 1 residual + LayerNorm, 2 residual only, 3 LayerNorm only.
// MASKED = false: the steady-state kernel, full tiles only; its loop body has no branch around a memory
// operation and issues the next tile's loads right after the last use of the current ones, so every wait
// counts exactly the younger operations.  MASKED = true: the ragged last tile of each batch (one per workgroup).
// ------------------------------------------------------------------------------------------------
template <int C, int S, int TAIL, bool MASKED>
__global__ __launch_bounds__(C * 2) void deslice_project_kernel(const u32x4 *__restrict__ blob, const u32x4 *__restrict__ w_pack,
                                                                const u32x4 *__restrict__ tokp, uint16_t *__restrict__ y,
                                                                const uint16_t *__restrict__ residual,
                                                                const float *__restrict__ ln_gamma,
                                                                const float *__restrict__ ln_beta, float ln_eps,
                                                                uint16_t *__restrict__ ln_out, int64_t N, int tpb,
                                                                int nfull, int64_t total_items) {
  constexpr bool HAS_RES = TAIL == 1 || TAIL == 2, HAS_LN = TAIL == 1 || TAIL == 3;
  constexpr int H = C / 32, NCH = S / 16, NT = C * 2;
  constexpr int ROWS = 32 / H;        // rows of the tile finished by each wave
  constexpr int CPL = C / 64;         // consecutive channels per lane in the epilogue
  constexpr int YS = C + 8;           // row stride (floats): rows 4 apart land 32 banks apart
  typedef uint32_t rowvec __attribute__((ext_vector_type(CPL / 2)));  // CPL bf16
  __shared__ u32x4 oxs[H * 2 * 64];
  __shared__ u32x4 tps[H * NCH * 64];
  __shared__ float ys[32 * YS];
  const BlobPlan bp = blob_plan(C, S);
  const int tid = threadIdx.x, lane = tid & 63, i = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: addresses derived from it stay scalar

  u32x4 wout[H][2];
#pragma unroll
  for (int h = 0; h < H; ++h) {
    wout[h][0] = blob[bp.wout + ((wave * H + h) * 2 + 0) * 64 + lane];
    wout[h][1] = blob[bp.wout + ((wave * H + h) * 2 + 1) * 64 + lane];
  }
  const float *fv = reinterpret_cast<const float *>(blob + bp.fvec) + bp.f_bias_out;
  const float bias = fv[wave * 32 + i];
  float gam[CPL], bet[CPL];
#pragma unroll
  for (int k = 0; k < CPL; ++k) {
    gam[k] = HAS_LN ? ln_gamma[lane * CPL + k] : 1.f;
    bet[k] = HAS_LN ? ln_beta[lane * CPL + k] : 0.f;
  }

  // item -> (batch, tile-in-batch): full tiles for the steady-state kernel, the last (ragged) tile otherwise
  int64_t item = blockIdx.x;
  int64_t b = MASKED ? item : item / nfull;
  int64_t t = MASKED ? (int64_t)tpb - 1 : item - b * nfull;
  u32x4 wcur[NCH];
  rowvec rcur[ROWS];
  {
    const u32x4 *wsrc = w_pack + (((b * tpb + t) * H + wave) * NCH) * 64 + lane;
#pragma unroll
    for (int cq = 0; cq < NCH; ++cq) wcur[cq] = load_streaming(wsrc + cq * 64);
    if constexpr (HAS_RES) {
#pragma unroll
      for (int rr = 0; rr < ROWS; ++rr) {
        int64_t n = t * 32 + wave * ROWS + rr;
        if (MASKED && n >= N) n = N - 1;
        rcur[rr] = load_streaming(reinterpret_cast<const rowvec *>(residual + (b * N + n) * C + lane * CPL));
      }
    }
  }
  if constexpr (!MASKED) {
    // Placeholder stores to this wave's first output rows (overwritten by the real results below).  They put the
    // loop entry in the same state as the loop back-edge -- prefetch loads followed by one epilogue's worth of
    // stores -- so the wait before the first use of wcur allows exactly those younger stores to stay in flight
    // instead of draining the memory pipeline every iteration.
    rowvec zero;
#pragma unroll
    for (int k = 0; k < CPL / 2; ++k) zero[k] = 0u;
#pragma unroll
    for (int rr = 0; rr < ROWS; ++rr) {
      const int64_t off = (b * N + t * 32 + wave * ROWS + rr) * C + lane * CPL;
      *reinterpret_cast<rowvec *>(y + off) = zero;
      if constexpr (HAS_LN) *reinterpret_cast<rowvec *>(ln_out + off) = zero;
    }
  }
  int64_t b_loaded = -1;
  while (true) {
    if (b != b_loaded) {  // workgroup-uniform: (re)load this batch's attended tokens
      __syncthreads();
      for (int u = tid; u < H * NCH * 64; u += NT) tps[u] = tokp[b * (H * NCH * 64) + u];
      __syncthreads();
      b_loaded = b;
    }
    const int64_t n0 = t * 32;
    // deslice this wave's head (last use of wcur)
    // (two interleaved accumulation chains: a dependent MFMA would wait for its predecessor's last pass)
    f32x16 ox, ox2;
#pragma unroll
    for (int r = 0; r < 16; ++r) ox[r] = ox2[r] = 0.f;
#pragma unroll
    for (int cq = 0; cq < NCH; cq += 2) {
      ox = mma(tps[(wave * NCH + cq) * 64 + lane], wcur[cq], ox);
      if (cq + 1 < NCH) ox2 = mma(tps[(wave * NCH + cq + 1) * 64 + lane], wcur[cq + 1 < NCH ? cq + 1 : 0], ox2);
    }
    if constexpr (NCH > 1) {
#pragma unroll
      for (int r = 0; r < 16; ++r) ox[r] += ox2[r];
    }
    // fetch the next item's slice weights and residual rows (the last iteration re-fetches its own)
    const int64_t item_next = item + gridDim.x;
    const bool more = !MASKED && item_next < total_items;
    const int64_t itn = more ? item_next : item;
    const int64_t bn = MASKED ? b : itn / nfull;
    const int64_t tn = MASKED ? t : itn - bn * nfull;
    u32x4 wnext[NCH];
    rowvec rnext[ROWS];
    {
      const u32x4 *wsrc = w_pack + (((bn * tpb + tn) * H + wave) * NCH) * 64 + lane;
#pragma unroll
      for (int cq = 0; cq < NCH; ++cq) wnext[cq] = load_streaming(wsrc + cq * 64);
      if constexpr (HAS_RES && !MASKED) {
#pragma unroll
        for (int rr = 0; rr < ROWS; ++rr)
          rnext[rr] = load_streaming(reinterpret_cast<const rowvec *>(residual + (bn * N + tn * 32 + wave * ROWS + rr) * C + lane * CPL));
      }
    }
    oxs[(wave * 2 + 0) * 64 + lane] = pack_half<0>(ox);
    oxs[(wave * 2 + 1) * 64 + lane] = pack_half<1>(ox);
    __syncthreads();
    // this wave's 32 output channels
    f32x16 acc, acc2;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      acc[r] = bias;
      acc2[r] = 0.f;
    }
#pragma unroll
    for (int hh = 0; hh < H; hh += 4) {
      u32x4 of[4][2];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        of[q][0] = oxs[((hh + q) * 2 + 0) * 64 + lane];
        of[q][1] = oxs[((hh + q) * 2 + 1) * 64 + lane];
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        acc = mma(of[q][0], wout[hh + q][0], acc);
        acc2 = mma(of[q][1], wout[hh + q][1], acc2);
      }
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) ys[rowmap(r, g) * YS + wave * 32 + i] = acc[r] + acc2[r];
    __syncthreads();
    // finish ROWS full rows per wave
#pragma unroll
    for (int rr = 0; rr < ROWS; ++rr) {
      const int row = wave * ROWS + rr;
      const int64_t n = n0 + row;
      const bool ok = !MASKED || n < N;
      const int64_t off = (b * N + n) * C + lane * CPL;
      float v[CPL];
      rowvec ob;
#pragma unroll
      for (int k = 0; k < CPL; k += 2) {
        float t0 = ys[row * YS + lane * CPL + k], t1 = ys[row * YS + lane * CPL + k + 1];
        if constexpr (HAS_RES) {
          // the residual is added to the fp32 result: one rounding for the sum instead of one per tensor op
          const uint32_t rv = rcur[rr][k / 2];
          t0 += bf16_bits_to_f32((uint16_t)(rv & 0xffffu));
          t1 += bf16_bits_to_f32((uint16_t)(rv >> 16));
        }
        const uint16_t o0 = to_bf16_bits(t0), o1 = to_bf16_bits(t1);
        v[k] = bf16_bits_to_f32(o0);
        v[k + 1] = bf16_bits_to_f32(o1);
        ob[k / 2] = (uint32_t)o0 | ((uint32_t)o1 << 16);
      }
      if (ok) store_streaming(reinterpret_cast<rowvec *>(y + off), ob);
      if constexpr (HAS_LN) {
        float s1 = 0.f;
#pragma unroll
        for (int k = 0; k < CPL; ++k) s1 += v[k];
        const float mean = wave_sum(s1) * (1.f / C);
        float s2 = 0.f;
#pragma unroll
        for (int k = 0; k < CPL; ++k) {
          const float dl = v[k] - mean;
          s2 = fmaf(dl, dl, s2);
        }
        const float rstd = rsqrtf(wave_sum(s2) * (1.f / C) + ln_eps);
        rowvec lb;
#pragma unroll
        for (int k = 0; k < CPL; k += 2) {
          const uint16_t l0 = to_bf16_bits((v[k] - mean) * rstd * gam[k] + bet[k]);
          const uint16_t l1 = to_bf16_bits((v[k + 1] - mean) * rstd * gam[k + 1] + bet[k + 1]);
          lb[k / 2] = (uint32_t)l0 | ((uint32_t)l1 << 16);
        }
        if (ok) store_streaming(reinterpret_cast<rowvec *>(ln_out + off), lb);
      }
    }
    if (!more) break;
    item = itn;
    b = bn;
    t = tn;
#pragma unroll
    for (int cq = 0; cq < NCH; ++cq) wcur[cq] = wnext[cq];
    if constexpr (HAS_RES) {
#pragma unroll
      for (int rr = 0; rr < ROWS; ++rr) rcur[rr] = rnext[rr];
    }
  }
}

// ------------------------------------------------------------------------------------------------
// Kernel (d) for S = 128, fed with x_mid as packed operand tiles ([tile][head][2][lane], what
// rows::project_rows_kernel writes) instead of slice weights: at this slice count the weights weigh 2 KB per point
// against 512 bytes of x_mid, so they are formed again here and never stored.  Forming them is vector work (128 exp2
// per point and head), the rest of the kernel is matrix, LDS and store work, so the waves split into two roles that
// share the SIMDs pairwise (wave w and wave w + H/2 sit on the same SIMD):
//   producers (waves 0 .. H/2-1, two heads each), one tile AHEAD of the consumers: slice weights of their heads from the
//              x_mid tile (logits against W_slice, softmax in the base-2 domain, un-normalised bf16 weights:
//              slice_weights_of_tile), out_x^T_h = tok'^T_h . w_h divided by the weights' sum (an all-ones MFMA)
//              -> bf16 A operands into the other half of a double-buffered LDS patch
//   consumers (waves H/2 .. H-1, two output tiles each): y = out_x . Wout^T with their slices of out_linear register
//              resident -> fp32 tile into LDS; then rows 64/H per wave: + residual, rounding, LayerNorm, full-row stores.
// Two barriers per tile: one hands the out_x patch over, one separates the consumers' two phases (the producers meet
// it between their two heads).  TAIL, MASKED: as in deslice_project_kernel.
// ------------------------------------------------------------------------------------------------
template <int C, int TAIL, bool MASKED>
__global__ __launch_bounds__(C * 2) void deslice_recompute_project_kernel(
    const u32x4 *__restrict__ blob, const u32x4 *__restrict__ xm_pack, const u32x4 *__restrict__ tokp,
    uint16_t *__restrict__ y, const uint16_t *__restrict__ residual, const float *__restrict__ ln_gamma,
    const float *__restrict__ ln_beta, float ln_eps, uint16_t *__restrict__ ln_out, int64_t N, int tpb, int nfull,
    int64_t total_items, const float *__restrict__ w_slice, const float *__restrict__ b_slice,
    const float *__restrict__ temperature) {
  constexpr bool HAS_RES = TAIL == 1 || TAIL == 2, HAS_LN = TAIL == 1 || TAIL == 3;
  constexpr int S = 128, H = C / 32, ST = S / 32, NCH = S / 16, CT = C / 32;
  constexpr int NPW = H / 2;          // producer waves = consumer waves
  constexpr int HPP = H / NPW;        // heads per producer (2)
  constexpr int CPC = CT / NPW;       // output tiles per consumer (2)
  constexpr int ROWS = 32 / NPW;      // rows of the tile finished by each consumer
  constexpr int CPL = C / 64;         // consecutive channels per lane in the epilogue
  constexpr int YS = C + 8;           // row stride (floats): rows 4 apart land 32 banks apart
  typedef uint32_t rowvec __attribute__((ext_vector_type(CPL / 2)));  // CPL bf16
  __shared__ u32x4 oxs[2][H * 2 * 64];
  __shared__ float ys[32 * YS];
  __shared__ u32x4 wsl[ST * 2 * 64];
  __shared__ float bsl[ST * 32];
  const BlobPlan bp = blob_plan(C, S);
  const int tid = threadIdx.x, lane = tid & 63, i = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: addresses derived from it stay scalar
  const bool producer = wave < NPW;
  stage_slice_projection<S, true>(w_slice, b_slice, wsl, bsl);
  __syncthreads();

  auto locate = [&](int64_t item, int64_t &b, int64_t &t) {
    b = MASKED ? item : item / nfull;
    t = MASKED ? (int64_t)tpb - 1 : item - b * nfull;
  };
  int64_t item = blockIdx.x;

  if (producer) {
    // ---- producers --------------------------------------------------------------------------------
    float sc[HPP];
#pragma unroll
    for (int hh = 0; hh < HPP; ++hh) sc[hh] = kLog2e / clamp_temperature(temperature[wave * HPP + hh]);
    u32x4 tp[HPP][NCH];
    int64_t b_loaded = -1;
    const u32x4 ones = u32x4{0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u};
    u32x4 xcur[HPP][2];
    auto fetch_x = [&](int64_t it, int hh) {  // the x_mid tile of head wave * HPP + hh of item `it`
      int64_t b, t;
      locate(it, b, t);
      const u32x4 *src = xm_pack + (((b * tpb + t) * H + wave * HPP + hh) * 2) * 64 + lane;
      xcur[hh][0] = load_streaming(src);
      xcur[hh][1] = load_streaming(src + 64);
    };
    // out_x of item `it` (its x_mid tiles in xcur) into patch `buf`; `mid`: meet the barrier between the two heads
    auto produce = [&](int64_t it, int buf, int64_t it_next, bool mid) {
      int64_t b, t;
      locate(it, b, t);
      if (b != b_loaded) {  // wave-uniform: this batch's attended tokens of the wave's heads
#pragma unroll
        for (int hh = 0; hh < HPP; ++hh)
#pragma unroll
          for (int cq = 0; cq < NCH; ++cq) tp[hh][cq] = tokp[((b * H + wave * HPP + hh) * NCH + cq) * 64 + lane];
        b_loaded = b;
      }
#pragma unroll
      for (int hh = 0; hh < HPP; ++hh) {
        u32x4 chunk[NCH];
        slice_weights_of_tile<S, true>(wsl, bsl, xcur[hh][0], xcur[hh][1], sc[hh], true, lane, g, chunk);
        fetch_x(it_next, hh);  // refilled in place for the next item, right behind their last use
        f32x16 ox, den;
#pragma unroll
        for (int r = 0; r < 16; ++r) ox[r] = den[r] = 0.f;
#pragma unroll
        for (int cq = 0; cq < NCH; ++cq) {
          ox = mma(tp[hh][cq], chunk[cq], ox);
          den = mma(ones, chunk[cq], den);
        }
        const float inv = __builtin_amdgcn_rcpf(den[0]);
#pragma unroll
        for (int r = 0; r < 16; ++r) ox[r] *= inv;
        const int h = wave * HPP + hh;
        oxs[buf][(h * 2 + 0) * 64 + lane] = pack_half<0>(ox);
        oxs[buf][(h * 2 + 1) * 64 + lane] = pack_half<1>(ox);
        if (hh == 0 && mid) __syncthreads();
        __builtin_amdgcn_sched_barrier(0);  // one head at a time: their registers are not live together
      }
    };
#pragma unroll
    for (int hh = 0; hh < HPP; ++hh) fetch_x(item, hh);
    {
      const int64_t nx = !MASKED && item + gridDim.x < total_items ? item + gridDim.x : item;
      produce(item, 0, nx, false);
    }
    __syncthreads();
    for (int k = 0;; ++k) {
      const int64_t next = item + gridDim.x;
      const bool more = !MASKED && next < total_items;
      if (more) {
        const int64_t nn = next + gridDim.x < total_items ? next + gridDim.x : next;
        produce(next, (k + 1) & 1, nn, true);
      } else {
        __syncthreads();
      }
      __syncthreads();
      if (!more) break;
      item = next;
    }
  } else {
    // ---- consumers --------------------------------------------------------------------------------
    const int cw = wave - NPW;
    u32x4 wout[CPC][H][2];
#pragma unroll
    for (int c = 0; c < CPC; ++c)
#pragma unroll
      for (int h = 0; h < H; ++h) {
        wout[c][h][0] = blob[bp.wout + (((cw * CPC + c) * H + h) * 2 + 0) * 64 + lane];
        wout[c][h][1] = blob[bp.wout + (((cw * CPC + c) * H + h) * 2 + 1) * 64 + lane];
      }
    const float *fv = reinterpret_cast<const float *>(blob + bp.fvec) + bp.f_bias_out;
    float bias[CPC];
#pragma unroll
    for (int c = 0; c < CPC; ++c) bias[c] = fv[(cw * CPC + c) * 32 + i];
    float gam[CPL], bet[CPL];
#pragma unroll
    for (int k = 0; k < CPL; ++k) {
      gam[k] = HAS_LN ? ln_gamma[lane * CPL + k] : 1.f;
      bet[k] = HAS_LN ? ln_beta[lane * CPL + k] : 0.f;
    }
    __syncthreads();  // the first patch is there
    for (int k = 0;; ++k) {
      int64_t b, t;
      locate(item, b, t);
      const int64_t n0 = t * 32;
      rowvec rcur[ROWS];
      if constexpr (HAS_RES) {
#pragma unroll
        for (int rr = 0; rr < ROWS; ++rr) {
          int64_t n = n0 + cw * ROWS + rr;
          if (MASKED && n >= N) n = N - 1;
          rcur[rr] = load_streaming(reinterpret_cast<const rowvec *>(residual + (b * N + n) * C + lane * CPL));
        }
      }
      const u32x4 *ob = oxs[k & 1];
      f32x16 acc[CPC];  // the output tiles take turns: two independent accumulation chains
#pragma unroll
      for (int c = 0; c < CPC; ++c)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[c][r] = bias[c];
#pragma unroll
      for (int hh = 0; hh < H; ++hh) {
        const u32x4 of0 = ob[(hh * 2 + 0) * 64 + lane], of1 = ob[(hh * 2 + 1) * 64 + lane];
#pragma unroll
        for (int c = 0; c < CPC; ++c) acc[c] = mma(of0, wout[c][hh][0], acc[c]);
#pragma unroll
        for (int c = 0; c < CPC; ++c) acc[c] = mma(of1, wout[c][hh][1], acc[c]);
      }
#pragma unroll
      for (int c = 0; c < CPC; ++c)
#pragma unroll
        for (int r = 0; r < 16; ++r) ys[rowmap(r, g) * YS + (cw * CPC + c) * 32 + i] = acc[c][r];
      __syncthreads();
      // finish ROWS full rows per consumer
#pragma unroll
      for (int rr = 0; rr < ROWS; ++rr) {
        const int row = cw * ROWS + rr;
        const int64_t n = n0 + row;
        const bool ok = !MASKED || n < N;
        const int64_t off = (b * N + n) * C + lane * CPL;
        float v[CPL];
        rowvec ov;
#pragma unroll
        for (int q = 0; q < CPL; q += 2) {
          float t0 = ys[row * YS + lane * CPL + q], t1 = ys[row * YS + lane * CPL + q + 1];
          if constexpr (HAS_RES) {
            // the residual is added to the fp32 result: one rounding for the sum instead of one per tensor op
            const uint32_t rv = rcur[rr][q / 2];
            t0 += bf16_bits_to_f32((uint16_t)(rv & 0xffffu));
            t1 += bf16_bits_to_f32((uint16_t)(rv >> 16));
          }
          const uint16_t o0 = to_bf16_bits(t0), o1 = to_bf16_bits(t1);
          v[q] = bf16_bits_to_f32(o0);
          v[q + 1] = bf16_bits_to_f32(o1);
          ov[q / 2] = (uint32_t)o0 | ((uint32_t)o1 << 16);
        }
        if (ok) store_streaming(reinterpret_cast<rowvec *>(y + off), ov);
        if constexpr (HAS_LN) {
          float s1 = 0.f;
#pragma unroll
          for (int q = 0; q < CPL; ++q) s1 += v[q];
          const float mean = wave_sum(s1) * (1.f / C);
          float s2 = 0.f;
#pragma unroll
          for (int q = 0; q < CPL; ++q) {
            const float dl = v[q] - mean;
            s2 = fmaf(dl, dl, s2);
          }
          const float rstd = rsqrtf(wave_sum(s2) * (1.f / C) + ln_eps);
          rowvec lb;
#pragma unroll
          for (int q = 0; q < CPL; q += 2) {
            const uint16_t l0 = to_bf16_bits((v[q] - mean) * rstd * gam[q] + bet[q]);
            const uint16_t l1 = to_bf16_bits((v[q + 1] - mean) * rstd * gam[q + 1] + bet[q + 1]);
            lb[q / 2] = (uint32_t)l0 | ((uint32_t)l1 << 16);
          }
          if (ok) store_streaming(reinterpret_cast<rowvec *>(ln_out + off), lb);
        }
      }
      __syncthreads();
      const int64_t next = item + gridDim.x;
      if (MASKED || next >= total_items) break;
      item = next;
    }
  }
}

// ================================================================================================
// host side
// ================================================================================================
bool supported(int dtype, const pa_shape &s) {
  if (dtype != PA_BF16 || s.conv_k != 0 || s.D != 32 || s.C != s.H * 32) return false;
  if (s.C != 128 && s.C != 256) return false;
  if (s.S != 16 && s.S != 32 && s.S != 64 && s.S != 128) return false;
  if ((s.N + 31) / 32 * s.B > ((int64_t)1 << 31) / 8 || s.B > 65535) return false;
  return true;
}

int64_t tiles_per_batch(const pa_shape &s) { return (s.N + 31) / 32; }

int64_t reduce_groups(const pa_shape &s) {
  const int64_t tpb = tiles_per_batch(s);
  int64_t g = (1024 + s.B * s.H - 1) / (s.B * s.H);
  const int64_t cap = (tpb + 7) / 8;
  if (g > cap) g = cap;
  return g < 1 ? 1 : g;
}

int64_t blob_bytes(const pa_shape &s) { return blob_plan((int)s.C, (int)s.S).total_units * 16; }
int64_t fx_pack_bytes(const pa_shape &s) { return s.B * tiles_per_batch(s) * s.H * 2 * 1024; }
int64_t w_pack_bytes(const pa_shape &s) { return s.B * tiles_per_batch(s) * s.H * (s.S / 16) * 1024; }
int64_t tokp_bytes(const pa_shape &s) { return s.B * s.H * (s.S / 16) * 1024; }

int pack_params(const pa_shape &s, const pa_params &p, void *blob, hipStream_t st) {
  hipLaunchKernelGGL(pack_params_kernel, dim3(64), dim3(256), 0, st, p, static_cast<u32x4 *>(blob), (int)s.C, (int)s.S, 0);
  return launch_status();
}

// the blob of kernel (d) alone, for layer variants that share only their hand-back with this family
int pack_out_linear(const pa_shape &s, const void *w_out, const float *w_scale, const float *b_out, void *blob,
                    hipStream_t st) {
  pa_params p{};
  p.out_linear_weight = w_out;
  p.out_linear_scale = w_scale;
  p.out_linear_bias = b_out;
  hipLaunchKernelGGL(pack_params_kernel, dim3(64), dim3(256), 0, st, p, static_cast<u32x4 *>(blob), (int)s.C, (int)s.S, 1);
  return launch_status();
}

// workgroups per batch of kernel (a): about one resident workgroup per CU in total
int64_t project_groups(const pa_shape &s, int num_cu, bool fused) {
  const int64_t ts = 4;
  (void)fused;
  const int64_t nsets = (tiles_per_batch(s) + ts - 1) / ts;
  int64_t g = num_cu / s.B;
  if (g < 1) g = 1;
  if (g > nsets) g = nsets;
  return g;
}

bool fuse_reduce(const pa_shape &s) { return s.S <= 64; }  // the LDS accumulators of the fused form fit up to S = 64

template <int C, int S, bool FUSED, bool CLOCKED = false>
static int project_softmax_f(const pa_shape &s, const void *blob, const void *x, void *fx_pack, void *w_pack,
                             float *partials, uint64_t *clock_out, int num_cu, hipStream_t st) {
  constexpr int ST = (S + 31) / 32, H = C / 32, TS = 4, UPR = C / 8, WAVES = H, NCK = 32 / (64 / UPR);
  const size_t lds = (size_t)(2 * TS * NCK * 65 + ST * 2 * 64 + 4 * 64) * 16 + (size_t)blob_plan(C, S).nfloat * 4;
  const int64_t tpb = tiles_per_batch(s);
  const int64_t G = project_groups(s, num_cu, FUSED);
  if constexpr (CLOCKED) {
    int rc = allow_dynamic_lds(project_softmax_clocked_kernel<C, S>, lds);
    if (rc) return rc;
    hipLaunchKernelGGL((project_softmax_clocked_kernel<C, S>), dim3((unsigned)G, (unsigned)s.B), dim3(WAVES * 64), lds, st,
                       static_cast<const u32x4 *>(blob), static_cast<const uint16_t *>(x), static_cast<u32x4 *>(w_pack),
                       partials, s.N, (int)tpb, clock_out);
  } else {
    int rc = allow_dynamic_lds(project_softmax_kernel<C, S, FUSED>, lds);
    if (rc) return rc;
    hipLaunchKernelGGL((project_softmax_kernel<C, S, FUSED>), dim3((unsigned)G, (unsigned)s.B), dim3(WAVES * 64), lds, st,
                       static_cast<const u32x4 *>(blob), static_cast<const uint16_t *>(x), static_cast<u32x4 *>(fx_pack),
                       static_cast<u32x4 *>(w_pack), partials, s.N, (int)tpb);
  }
  return launch_status();
}

template <int C, int S>
static int project_softmax_cs(const pa_shape &s, const void *blob, const void *x, void *fx_pack, void *w_pack,
                              float *partials, uint64_t *clock_out, int num_cu, hipStream_t st) {
  if constexpr (S <= 64) {
    if constexpr (C == 256) {  // the clocked twin exists for the width of the benchmark workload
      if (partials && clock_out)
        return project_softmax_f<C, S, true, true>(s, blob, x, fx_pack, w_pack, partials, clock_out, num_cu, st);
    }
    if (clock_out) return PA_ERR_UNSUPPORTED;
    if (partials) return project_softmax_f<C, S, true>(s, blob, x, fx_pack, w_pack, partials, nullptr, num_cu, st);
  }
  if (clock_out) return PA_ERR_UNSUPPORTED;
  return project_softmax_f<C, S, false>(s, blob, x, fx_pack, w_pack, nullptr, nullptr, num_cu, st);
}

template <int S>
static int slice_reduce_s(const pa_shape &s, const void *w_pack, const void *fx_pack, float *partials, hipStream_t st) {
  constexpr int ST = (S + 31) / 32;
  const size_t lds = (size_t)4 * ST * 17 * 64 * 4;
  int rc = allow_dynamic_lds(slice_reduce_kernel<S>, lds);
  if (rc) return rc;
  const int64_t tpb = tiles_per_batch(s), G = reduce_groups(s);
  const int tiles_per_group = (int)((tpb + G - 1) / G);
  hipLaunchKernelGGL((slice_reduce_kernel<S>), dim3((unsigned)G, (unsigned)(s.B * s.H)), dim3(256), lds, st,
                     static_cast<const u32x4 *>(w_pack), static_cast<const u32x4 *>(fx_pack), partials, (int)s.B, (int)s.H,
                     (int)tpb, tiles_per_group);
  return launch_status();
}

template <int C, int S, int TAIL>
static int deslice_project_t(const pa_shape &s, const void *blob, const void *w_pack, const void *tokp, void *y,
                             const pa_block_tail *tail, int num_cu, hipStream_t st) {
  const int64_t tpb = tiles_per_batch(s);
  const int nfull = (int)(s.N / 32);
  const u32x4 *bl = static_cast<const u32x4 *>(blob), *wp = static_cast<const u32x4 *>(w_pack),
              *tp = static_cast<const u32x4 *>(tokp);
  uint16_t *yo = static_cast<uint16_t *>(y);
  const uint16_t *res = static_cast<const uint16_t *>(tail ? tail->residual : nullptr);
  const float *gm = tail ? tail->ln_gamma : nullptr, *bt = tail ? tail->ln_beta : nullptr;
  const float eps = tail ? tail->ln_eps : 0.f;
  uint16_t *lo = static_cast<uint16_t *>(tail ? tail->ln_out : nullptr);
  if (nfull > 0) {
    static int per_cu = 0;  // resident workgroups per CU for this instantiation
    if (per_cu == 0) {
      int nb = 0;
      if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, deslice_project_kernel<C, S, TAIL, false>, C * 2, 0) !=
              hipSuccess || nb < 1)
        nb = 1;
      per_cu = nb;
    }
    const int64_t total = (int64_t)nfull * s.B;
    int64_t grid = (int64_t)num_cu * per_cu;
    if (grid > total) grid = total;
    hipLaunchKernelGGL((deslice_project_kernel<C, S, TAIL, false>), dim3((unsigned)grid), dim3(C * 2), 0, st, bl, wp, tp,
                       yo, res, gm, bt, eps, lo, s.N, (int)tpb, nfull, total);
    int rc = launch_status();
    if (rc) return rc;
  }
  if (s.N % 32 != 0) {
    hipLaunchKernelGGL((deslice_project_kernel<C, S, TAIL, true>), dim3((unsigned)s.B), dim3(C * 2), 0, st, bl, wp, tp, yo,
                       res, gm, bt, eps, lo, s.N, (int)tpb, nfull, s.B);
    return launch_status();
  }
  return PA_OK;
}

// the recomputing form (x_mid tiles in, slice weights never stored)
template <int C, int TAIL>
static int deslice_recompute_project_t(const pa_shape &s, const pa_params &p, const void *blob, const void *xm_pack,
                                       const void *tokp, void *y, const pa_block_tail *tail, int num_cu, hipStream_t st) {
  const int64_t tpb = tiles_per_batch(s);
  const int nfull = (int)(s.N / 32);
  const u32x4 *bl = static_cast<const u32x4 *>(blob), *xp = static_cast<const u32x4 *>(xm_pack),
              *tp = static_cast<const u32x4 *>(tokp);
  uint16_t *yo = static_cast<uint16_t *>(y);
  const uint16_t *res = static_cast<const uint16_t *>(tail ? tail->residual : nullptr);
  const float *gm = tail ? tail->ln_gamma : nullptr, *bt = tail ? tail->ln_beta : nullptr;
  const float eps = tail ? tail->ln_eps : 0.f;
  uint16_t *lo = static_cast<uint16_t *>(tail ? tail->ln_out : nullptr);
  if (nfull > 0) {
    const int64_t total = (int64_t)nfull * s.B;
    const int64_t grid = num_cu < total ? num_cu : total;  // its LDS leaves room for one workgroup per CU
    hipLaunchKernelGGL((deslice_recompute_project_kernel<C, TAIL, false>), dim3((unsigned)grid), dim3(C * 2), 0, st, bl, xp,
                       tp, yo, res, gm, bt, eps, lo, s.N, (int)tpb, nfull, total, p.in_project_slice_weight,
                       p.in_project_slice_bias, p.temperature);
    int rc = launch_status();
    if (rc) return rc;
  }
  if (s.N % 32 != 0) {
    hipLaunchKernelGGL((deslice_recompute_project_kernel<C, TAIL, true>), dim3((unsigned)s.B), dim3(C * 2), 0, st, bl, xp, tp,
                       yo, res, gm, bt, eps, lo, s.N, (int)tpb, nfull, s.B, p.in_project_slice_weight,
                       p.in_project_slice_bias, p.temperature);
    return launch_status();
  }
  return PA_OK;
}

template <int C, int S>
static int deslice_project_cs(const pa_shape &s, const void *blob, const void *w_pack, const void *tokp, void *y,
                              const pa_block_tail *tail, int num_cu, hipStream_t st) {
  const bool has_res = tail && tail->residual, has_ln = tail && tail->ln_out;
  if (has_res && has_ln) return deslice_project_t<C, S, 1>(s, blob, w_pack, tokp, y, tail, num_cu, st);
  if (has_res) return deslice_project_t<C, S, 2>(s, blob, w_pack, tokp, y, tail, num_cu, st);
  if (has_ln) return deslice_project_t<C, S, 3>(s, blob, w_pack, tokp, y, tail, num_cu, st);
  return deslice_project_t<C, S, 0>(s, blob, w_pack, tokp, y, tail, num_cu, st);
}

template <int C>
static int deslice_recompute_project_c(const pa_shape &s, const pa_params &p, const void *blob, const void *xm_pack,
                                       const void *tokp, void *y, const pa_block_tail *tail, int num_cu, hipStream_t st) {
  const bool has_res = tail && tail->residual, has_ln = tail && tail->ln_out;
  if (has_res && has_ln) return deslice_recompute_project_t<C, 1>(s, p, blob, xm_pack, tokp, y, tail, num_cu, st);
  if (has_res) return deslice_recompute_project_t<C, 2>(s, p, blob, xm_pack, tokp, y, tail, num_cu, st);
  if (has_ln) return deslice_recompute_project_t<C, 3>(s, p, blob, xm_pack, tokp, y, tail, num_cu, st);
  return deslice_recompute_project_t<C, 0>(s, p, blob, xm_pack, tokp, y, tail, num_cu, st);
}

#define PA_DISPATCH_CS(FN, ...)                                     \
  do {                                                              \
    if (s.C == 256) {                                               \
      if (s.S == 16) return FN<256, 16>(__VA_ARGS__);               \
      if (s.S == 32) return FN<256, 32>(__VA_ARGS__);               \
      if (s.S == 64) return FN<256, 64>(__VA_ARGS__);               \
      return FN<256, 128>(__VA_ARGS__);                             \
    }                                                               \
    if (s.S == 16) return FN<128, 16>(__VA_ARGS__);                 \
    if (s.S == 32) return FN<128, 32>(__VA_ARGS__);                 \
    if (s.S == 64) return FN<128, 64>(__VA_ARGS__);                 \
    return FN<128, 128>(__VA_ARGS__);                               \
  } while (0)

// partials != nullptr (and S <= 64): fused with the first reduction pass; fx_pack is then not written
int project_softmax(const pa_shape &s, const void *blob, const void *x, void *fx_pack, void *w_pack, float *partials,
                    int num_cu, hipStream_t st) {
  PA_DISPATCH_CS(project_softmax_cs, s, blob, x, fx_pack, w_pack, partials, nullptr, num_cu, st);
}

int project_softmax_clocked(const pa_shape &s, const void *blob, const void *x, void *w_pack, float *partials,
                            uint64_t *clock_out, int num_cu, hipStream_t st) {
  PA_DISPATCH_CS(project_softmax_cs, s, blob, x, nullptr, w_pack, partials, clock_out, num_cu, st);
}

int slice_reduce(const pa_shape &s, const void *w_pack, const void *fx_pack, float *partials, hipStream_t st) {
  if (s.S == 16) return slice_reduce_s<16>(s, w_pack, fx_pack, partials, st);
  if (s.S == 32) return slice_reduce_s<32>(s, w_pack, fx_pack, partials, st);
  if (s.S == 64) return slice_reduce_s<64>(s, w_pack, fx_pack, partials, st);
  return slice_reduce_s<128>(s, w_pack, fx_pack, partials, st);
}

template <int S>
static int slice_attention_s(const pa_shape &s, const float *combined, const float *fx_bias, const float *w_qkv,
                             float *slice_token, float *slice_norm, float *out_token, void *tokp, hipStream_t st) {
  hipLaunchKernelGGL((slice_attention_kernel<S>), dim3((unsigned)(s.B * s.H)), dim3(64 * ((S + 31) / 32)), 0, st, combined,
                     fx_bias, w_qkv, slice_token, slice_norm, out_token, static_cast<uint16_t *>(tokp), (int)s.H);
  return launch_status();
}

// second pass of the reduction + kernel (c); also leaves the attended tokens as bf16 operands of kernel (d).
// fx_bias: the in_project_fx bias when the partials come from project_softmax_kernel (which sums fx_mid without it),
// NULL when the summed values already carry their bias.
int combine_attention(const pa_shape &s, const pa_params &p, const float *fx_bias, const float *partials, int64_t G,
                      float *slice_token, float *slice_norm, float *out_token, void *tokp, hipStream_t st) {
  const float *combined = nullptr;
  int rc = pa::general::combine_partials(s, partials, G, &combined, st);
  if (rc) return rc;
  const float *wq = p.qkv_project_weight;
  switch (s.S) {
    case 16: return slice_attention_s<16>(s, combined, fx_bias, wq, slice_token, slice_norm, out_token, tokp, st);
    case 32: return slice_attention_s<32>(s, combined, fx_bias, wq, slice_token, slice_norm, out_token, tokp, st);
    case 64: return slice_attention_s<64>(s, combined, fx_bias, wq, slice_token, slice_norm, out_token, tokp, st);
    case 128: return slice_attention_s<128>(s, combined, fx_bias, wq, slice_token, slice_norm, out_token, tokp, st);
    default: return PA_ERR_UNSUPPORTED;
  }
}

int deslice_project(const pa_shape &s, const void *blob, const void *w_pack, const void *tokp, void *y,
                    const pa_block_tail *tail, int num_cu, hipStream_t st) {
  PA_DISPATCH_CS(deslice_project_cs, s, blob, w_pack, tokp, y, tail, num_cu, st);
}

bool deslice_recompute_project_supported(const pa_shape &s) { return s.S == 128 && (s.C == 256 || s.C == 128); }

int deslice_recompute_project(const pa_shape &s, const pa_params &p, const void *blob, const void *xm_pack,
                              const void *tokp, void *y, const pa_block_tail *tail, int num_cu, hipStream_t st) {
  if (!deslice_recompute_project_supported(s)) return PA_ERR_UNSUPPORTED;
  if (s.C == 256) return deslice_recompute_project_c<256>(s, p, blob, xm_pack, tokp, y, tail, num_cu, st);
  return deslice_recompute_project_c<128>(s, p, blob, xm_pack, tokp, y, tail, num_cu, st);
}

}  // namespace mfma
}  // namespace pa
