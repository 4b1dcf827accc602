// Float32 front end of the structured-grid layer (PhysicsAttentionStructuredMesh2D, PA.py:744-783 with the shared
// slice weights of PA.py:172-203): the two k x k convolutions of the input, the slice logits, the temperature
// softmax and the partial slice-token sums in one launch.
//
// Shape class: C = 128 channels, 8 heads of 16, 32 slices; 2-D grid with odd k, or Linear projections (the irregular
// mesh, PA.py:501-514) as the 1 x 1 case.
//
// The convolutions are one implicit GEMM, M = points, N = 256 (x_mid | fx_mid), K = k k 128 (tap-major), computed
// with float32 accuracy on the bf16 matrix cores: every float32 operand is cut into three bf16 pieces
// a = a1 + a2 + a3 (8 significant bits each, exact), and a . b is taken as the six bf16 products
// a1 b1 + a1 b2 + a2 b1 + a2 b2 + a1 b3 + a3 b1 accumulated in float32 (the dropped products are below 2^-23 |a b|).
// Six v_mfma_f32_32x32x16_bf16 cost 48 passes where the sixteen-times narrower v_mfma_f32_32x32x2_f32 needs 128.
// The weights are cut once per call by split_pack_kernel into the fragment order the waves read; the activations
// are cut in registers, once per k-step for all eight column tiles of a wave.
//
// Workgroup = 8 waves = 4 tiles of 32 points of one batch, two waves per tile and per SIMD: the x_mid wave owns the
// tile's 32 x 128 x_mid outputs, the fx_mid wave its 32 x 128 fx_mid outputs (64 accumulator registers each).  Weights
// (24 KB per k-step) and input rows (the x_mid wave fetches them for both) go from L2 into four-slot LDS rings with
// global_load_lds, three k-steps ahead; one barrier per k-step, and the waits on the in-order counter vmcnt leave the
// two newest groups in flight.  The x_mid tiles are computed with the weights as the A operand (lanes <-> points), the
// fx_mid tiles with the rows as the A operand (lanes <-> channels, registers <-> points), which is the form each is
// needed in afterwards:
//   logits^T = W_slice x_mid^T   (float32 MFMA, lanes <-> points)   -> per-point maximum and sum in registers
//   logits   = x_mid W_slice^T   (the same operands swapped, lanes <-> slices) -> w = exp(l / T - max) / sum
//   tokens  += w^T fx_mid        (float32 MFMA over the 32 points, by the fx_mid wave; w crosses through LDS in the
//                                 register layout of the A operand, one head behind the x_mid wave)
// w leaves in natural layout (B, N, H, S) for the hand-back to the points; the token sums of the four tiles are added
// through LDS in a fixed order and leave as one partial per workgroup, [g][b][h][S][D + 1] with the slice norm in the
// last column (the layout slice_combine_attn_kernel sums).
#include "pa_host.h"
#include "pa_mfma_ops.h"
#include "pa_split_ops.h"

namespace pa {
namespace conv {

using mfma::f32x16;
using mfma::half_max;
using mfma::half_sum;
using mfma::mma;
using mfma::rowmap;
using mfma::u32x4;
using namespace split;

constexpr int kC = 128, kH = 8, kD = 16, kS = 32, kD1 = kD + 1;
constexpr int kColTiles = 8;                       // 4 of x_mid, 4 of fx_mid
constexpr int kStepsPerTap = kC / 16;              // k-steps of 16 channels
constexpr int kStepUnits = kColTiles * 3 * 64;     // 16-byte units per k-step: 8 tiles x 3 pieces x 1 KB
constexpr int kRing = 4;
constexpr int kTokFloats = kH * kS * kD1;          // one partial
// the ring, reused after the convolution for 4 token sums, 4 x 4 accumulator tiles in transit between the two waves of
// a tile, and every wave's softmax statistics
constexpr size_t kEpilogueBytes = (size_t)4 * kTokFloats * 4 + 4 * 4 * 4096 + 8 * 128 * 4;
constexpr size_t kRingBytes = (size_t)kRing * kStepUnits * 16 + (size_t)kRing * 4 * 2048;  // weights + input rows
constexpr size_t kLdsBytes = kRingBytes > kEpilogueBytes ? kRingBytes : kEpilogueBytes;

// blob unit ((step 8 + ct) 3 + piece) 64 + lane: the B operand (lane (i, g): output channel 32 (ct % 4) + i of weight
// set ct / 4, k = 8 g .. 8 g + 7 of the step) of one bf16 piece.  step = tap 8 + channel block.
// The workgroups behind the first conv_blocks cut the weights of the same call's row kernel: out_linear's (8 units),
// then, with w1 given, the block MLP's per chunk of 128 hidden features (8 units of W1's rows, 8 of W2's columns) --
// all with the reduction index in register order (the layout f32rows::backend / block_tail read).
__global__ __launch_bounds__(256) void split_pack_kernel(const float *__restrict__ wx, const float *__restrict__ wfx,
                                                         u32x4 *__restrict__ blob, int taps, int tap_major,
                                                         int conv_blocks, const float *__restrict__ w_out,
                                                         const float *__restrict__ w1, const float *__restrict__ w2,
                                                         int F, u32x4 *__restrict__ blob_out) {
  if ((int)blockIdx.x >= conv_blocks) {
    const int u = blockIdx.x - conv_blocks;
    u32x4 *unit = blob_out + (int64_t)u * kUnit;
    if (u < 8) {
      pack_unit(w_out, kC, 16 * u, true, unit, threadIdx.x);
    } else {
      const int q = u - 8, c = q >> 4, v = q & 15;
      if (v < 8) pack_unit(w1 + (int64_t)c * 128 * kC, kC, 16 * v, true, unit, threadIdx.x);
      else pack_unit(w2 + c * 128, F, 16 * (v - 8), true, unit, threadIdx.x);
    }
    return;
  }
  const int64_t total = (int64_t)taps * kStepsPerTap * kColTiles * 64;
  for (int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x; u < total; u += (int64_t)conv_blocks * 256) {
    const int lane = (int)(u & 63), ct = (int)(u >> 6) & 7, step = (int)(u >> 9);
    const int tap = step / kStepsPerTap, c0 = (step % kStepsPerTap) * 16 + 8 * (lane >> 5);
    const int o = 32 * (ct & 3) + (lane & 31);
    const float *w = ct < 4 ? wx : wfx;
    uint32_t h[8][3];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int c = c0 + e;
      const int64_t idx = tap_major ? ((int64_t)o * taps + tap) * kC + c : ((int64_t)o * kC + c) * taps + tap;
      split3(w[idx], h[e]);
    }
#pragma unroll
    for (int pl = 0; pl < 3; ++pl) {
      u32x4 v;
#pragma unroll
      for (int q = 0; q < 4; ++q) v[q] = h[2 * q][pl] | (h[2 * q + 1][pl] << 16);
      blob[((int64_t)step * kColTiles + ct) * 192 + pl * 64 + lane] = v;
    }
  }
  if (blockIdx.x == 0 && threadIdx.x < 4) blob[total * 3 + threadIdx.x] = u32x4{0u, 0u, 0u, 0u};  // the zero page
}

__global__ __launch_bounds__(512) void conv_slice_kernel(
    const u32x4 *__restrict__ blob, const float *__restrict__ bias_x, const float *__restrict__ bias_fx,
    const float *__restrict__ w_slice, const float *__restrict__ b_slice, const float *__restrict__ temperature,
    const float *__restrict__ x, float *__restrict__ w_out, float *__restrict__ partials, int B, int N, int gh, int gw,
    int ks, int bpb) {
  extern __shared__ u32x4 smem[];
  const int tid = threadIdx.x, lane = tid & 63, i = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int t = wave & 3;        // the wave's tile of the workgroup's four
  const int role = wave >> 2;    // 0: the x_mid half of the columns and the slice weights, 1: fx_mid and the token sums
  const int b = blockIdx.x / bpb, gblk = blockIdx.x - b * bpb;
  const int n0 = (gblk * 4 + t) * 32;                    // first point of the tile (may lie past the end)
  const int valid = min(max(N - n0, 0), 32);             // its points that exist
  const int n = min(n0 + i, N - 1);                      // lanes past the end repeat the last point (weight 0 below)
  const int ci = n / gw, cj = n - ci * gw;
  const float *xb = x + (int64_t)b * N * kC + 8 * g;
  const int pad = ks >> 1, steps = ks * ks * kStepsPerTap;

  // this lane's 8 channels of the input row k-step `k` reads: the tap's neighbour, or 32 zero bytes outside the grid
  const float *zero_page = reinterpret_cast<const float *>(blob + (int64_t)steps * kStepUnits);
  auto row_ptr = [&](int k) -> const float * {
    const int tap = k >> 3, c0 = (k & 7) * 16;
    const int u = tap / ks, v = tap - u * ks;
    const int ii = ci + u - pad, jj = cj + v - pad;
    const bool ok = ii >= 0 && ii < gh && jj >= 0 && jj < gw;
    return ok ? xb + (int64_t)(ii * gw + jj) * kC + c0 : zero_page;
  };
  // the row as three bf16 A / B operands (lane (i, g): point i, k = 8 g .. 8 g + 7)
  auto split_row = [&](const u32x4 (&raw)[2], u32x4 (&pl)[3]) {
    uint32_t h[8][3];
#pragma unroll
    for (int e = 0; e < 8; ++e) split3(__uint_as_float(raw[e >> 2][e & 3]), h[e]);
#pragma unroll
    for (int p = 0; p < 3; ++p)
#pragma unroll
      for (int q = 0; q < 4; ++q) pl[p][q] = h[2 * q][p] | (h[2 * q + 1][p] << 16);
  };
  // Group k of the memory stream: the x_mid wave's rows of k-step k (lane (i, g): point i, two 16-byte halves of its
  // 8 channels) into the row ring, then every wave's eighth (3 KB) of the step's weights into the weight ring; both
  // with global_load_lds, slot k % 4.  Five (x_mid wave) or three operations on the in-order counter vmcnt.
  u32x4 *rowbuf = smem + kRing * kStepUnits + t * 128;  // + slot * 512: [half][lane]
  auto issue_group = [&](int k, auto role_) {
    if constexpr (decltype(role_)::value == 0) {
      const float *p = row_ptr(k);
      const unsigned dst = (unsigned)(uintptr_t)(rowbuf + (k % kRing) * 512);
      asm volatile(
          "s_mov_b32 m0, %1\n\t"
          "s_nop 0\n\t"
          "global_load_lds_dwordx4 %0, off" ::"v"(p), "s"(dst)
          : "memory");
      asm volatile(
          "s_mov_b32 m0, %1\n\t"
          "s_nop 0\n\t"
          "global_load_lds_dwordx4 %0, off offset:16" ::"v"(p), "s"(dst + 1024 - 16)  // the offset moves both addresses
          : "memory");
    }
    const u32x4 *src = blob + (int64_t)k * kStepUnits + wave * 192;
    const unsigned dst = (unsigned)(uintptr_t)(smem + (k % kRing) * kStepUnits + wave * 192);
    load_3k_to_lds(src, lane * 16, dst);
  };

  // role 0, x_mid tiles: lane (i, g) <-> point i, register r <-> channel 32 ct + rowmap(r, g)
  // role 1, fx_mid tiles: lane (i, g) <-> channel 32 ct + i, register r <-> point rowmap(r, g)
  f32x16 acc[4];
  // the k-steps, compiled once per role so that neither carries the other's operand order
  auto convolve = [&](auto role_) {
    constexpr int ROLE = decltype(role_)::value;
#pragma unroll
    for (int ct = 0; ct < 4; ++ct)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        if constexpr (ROLE == 0) acc[ct][r] = bias_x ? bias_x[32 * ct + rowmap(r, g)] : 0.f;
        else acc[ct][r] = bias_fx ? bias_fx[32 * ct + i] : 0.f;
      }
    u32x4 raw[2], cur[3], nxt[3];
    u32x4 fr[2][4][3];  // the weight fragments of the even / the odd k-steps
    auto read_rows = [&](int k) {
      const u32x4 *rb = rowbuf + (k % kRing) * 512 + lane;
      raw[0] = rb[0];
      raw[1] = rb[64];
    };
    auto read_fragments = [&](int k, u32x4 (&f)[4][3]) {
      const u32x4 *wb = smem + (k % kRing) * kStepUnits + ROLE * (4 * 192) + lane;
#pragma unroll
      for (int ct = 0; ct < 4; ++ct)
#pragma unroll
        for (int p = 0; p < 3; ++p) f[ct][p] = wb[(ct * 3 + p) * 64];
    };
    issue_group(0, role_);
    issue_group(1, role_);
    issue_group(2, role_);
    issue_group(3, role_);
    // vmcnt(0), as the builtin so that the compiler too knows the bias loads above are complete (it would otherwise
    // wait for them, and with them for everything in flight, at their first use inside the loop)
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
    read_rows(0);
    read_fragments(0, fr[0]);
    split_row(raw, cur);
    // One k-step.  Groups up to s + 3 are issued.  The step multiplies the fragments and rows of step s, read from LDS
    // one step ago, and reads those of step s + 1: group s + 1 must have landed, groups s + 2 and s + 3 may stay in
    // flight (5 operations each for an x_mid wave, 3 for an fx_mid wave).  Each wave waits for its own share, then all
    // meet; the slots of step s, read one step ago, are free once every wave is here.  TAIL: one of the last four
    // steps, where there is less to wait for, to read or to request.
    auto step = [&](int s, auto par_, auto tail_) {
      constexpr int par = decltype(par_)::value;
      constexpr bool TAIL = decltype(tail_)::value;
      if (!TAIL || s + 3 < steps) {
        if constexpr (ROLE == 0) asm volatile("s_waitcnt vmcnt(10)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
      } else if (s + 2 < steps) {
        if constexpr (ROLE == 0) asm volatile("s_waitcnt vmcnt(5)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(3)" ::: "memory");
      } else {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      }
      __syncthreads();
      if (!TAIL || s + 4 < steps) issue_group(s + 4, role_);
      if (!TAIL || s + 1 < steps) {
        read_rows(s + 1);
        read_fragments(s + 1, fr[1 - par]);
      }
      // the six products, the four column tiles taking turns
      auto product = [&](int pw, int pa) {
#pragma unroll
        for (int ct = 0; ct < 4; ++ct) {
          if constexpr (ROLE == 0) acc[ct] = mma(fr[par][ct][pw], cur[pa], acc[ct]);
          else acc[ct] = mma(cur[pa], fr[par][ct][pw], acc[ct]);
        }
      };
      product(0, 0);
      product(1, 0);
      product(0, 1);
      product(1, 1);
      product(2, 0);
      product(0, 2);
      if (!TAIL || s + 1 < steps) split_row(raw, nxt);
#pragma unroll
      for (int p = 0; p < 3; ++p) cur[p] = nxt[p];
      if constexpr (!TAIL) {
        // issue order: after every matrix instruction one LDS read (while there are any) and a few vector instructions,
        // so that the step's other work runs while the matrix core is busy instead of ahead of it
#pragma unroll
        for (int k = 0; k < 24; ++k) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
        }
      }
    };
    constexpr std::integral_constant<int, 0> even{};
    constexpr std::integral_constant<int, 1> odd{};
    int s2 = 0;
    for (; s2 + 5 < steps; s2 += 2) {
      step(s2, even, std::false_type{});
      step(s2 + 1, odd, std::false_type{});
    }
    for (; s2 < steps; s2 += 2) {
      step(s2, even, std::true_type{});
      step(s2 + 1, odd, std::true_type{});
    }
  };
  if (role == 0) convolve(std::integral_constant<int, 0>{});
  else convolve(std::integral_constant<int, 1>{});
  __syncthreads();  // the ring is free: it now holds the token sums, the weights in transit and the softmax statistics

  float *red = reinterpret_cast<float *>(smem);                     // [tile][h][s][D + 1]
  float *mine = red + t * kTokFloats;
  u32x4 *xchg = smem + (4 * kTokFloats) / 4 + t * (4 * 256);        // [tile][role of the writer][tile of the pair][q][lane]
  float *stat = reinterpret_cast<float *>(smem + (4 * kTokFloats) / 4 + 4 * 4 * 256) + wave * 128;  // [head][max | 1 / sum][point]
  // The two waves of a tile share the eight heads: the x_mid wave takes heads 0 .. 3 and needs the fx_mid tiles 0, 1,
  // the fx_mid wave takes heads 4 .. 7 and needs the x_mid tiles 2, 3.  One exchange of 32 registers each way through
  // LDS, then every wave runs its heads from the logits to the token sums on its own.
#pragma unroll
  for (int c = 0; c < 2; ++c) {
    f32x16 give;  // element by element: a select between the two arrays as wholes would keep them in memory
#pragma unroll
    for (int r = 0; r < 16; ++r) give[r] = role == 0 ? acc[2 + c][r] : acc[c][r];
#pragma unroll
    for (int q = 0; q < 4; ++q)
      xchg[(role * 2 + c) * 256 + q * 64 + lane] =
          u32x4{__float_as_uint(give[4 * q]), __float_as_uint(give[4 * q + 1]), __float_as_uint(give[4 * q + 2]),
                __float_as_uint(give[4 * q + 3])};
  }
  // W_slice[s][d] for MFMA m of a head: this lane's channel of the pair (k = g) is d = 8 (m / 4) + 4 g + m % 4, the
  // channel the x_mid registers hold in that position
  float ws[8], bs_r[16];
#pragma unroll
  for (int m = 0; m < 8; ++m) ws[m] = w_slice[i * kD + rowmap(m, g)];
#pragma unroll
  for (int r = 0; r < 16; ++r) bs_r[r] = b_slice ? b_slice[rowmap(r, g)] : 0.f;
  const float bs_i = b_slice ? b_slice[i] : 0.f;
  float *wpoint = w_out + ((int64_t)b * N + n0 + i) * (kH * kS);  // this lane's point (when it exists)
  __syncthreads();
  f32x16 xs[2], fs[2];  // this wave's two x_mid tiles (lanes <-> points) and fx_mid tiles (lanes <-> channels)
#pragma unroll
  for (int c = 0; c < 2; ++c) {
    f32x16 got;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const u32x4 v = xchg[((1 - role) * 2 + c) * 256 + q * 64 + lane];
      got[4 * q] = __uint_as_float(v[0]), got[4 * q + 1] = __uint_as_float(v[1]);
      got[4 * q + 2] = __uint_as_float(v[2]), got[4 * q + 3] = __uint_as_float(v[3]);
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      xs[c][r] = role == 0 ? acc[c][r] : got[r];
      fs[c][r] = role == 0 ? got[r] : acc[2 + c][r];
    }
  }
  // heads 4 role + 2 c + {0, 1} are the halves of tile c; the two heads' dependent MFMA chains take turns
  static_for<2>([&](auto c_) {
    constexpr int c = decltype(c_)::value;
    const int h0 = 4 * role + 2 * c;
    float inv_t[2];
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) inv_t[hf] = temperature ? kLog2e / clamp_temperature(temperature[h0 + hf]) : kLog2e;
    // lanes <-> points: the heads' softmax statistics, and the weights as they leave (a lane holds 4 consecutive slices
    // of its point per register quad)
    f32x16 lt[2];
#pragma unroll
    for (int r = 0; r < 16; ++r) lt[0][r] = lt[1][r] = bs_r[r];
#pragma unroll
    for (int m = 0; m < 8; ++m)
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) lt[hf] = mma32(ws[m], xs[c][8 * hf + m], lt[hf]);
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
      float mx = lt[hf][0] * inv_t[hf];
#pragma unroll
      for (int r = 1; r < 16; ++r) mx = fmaxf(mx, lt[hf][r] * inv_t[hf]);
      mx = half_max(mx);
      float sum = 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        lt[hf][r] = __builtin_amdgcn_exp2f(lt[hf][r] * inv_t[hf] - mx);
        sum += lt[hf][r];
      }
      sum = half_sum(sum);
      const float inv = 1.f / sum;
      if (g == 0) {
        stat[64 * hf + i] = mx;
        stat[64 * hf + 32 + i] = inv;
      }
      if (i < valid) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float4 o = {lt[hf][4 * q] * inv, lt[hf][4 * q + 1] * inv, lt[hf][4 * q + 2] * inv, lt[hf][4 * q + 3] * inv};
          *reinterpret_cast<float4 *>(wpoint + (h0 + hf) * kS + 8 * q + 4 * g) = o;
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
    // lanes <-> slices, register r <-> point rowmap(r, g): the weights as the A operand of the token sums
    f32x16 ln[2];
#pragma unroll
    for (int r = 0; r < 16; ++r) ln[0][r] = ln[1][r] = bs_i;
#pragma unroll
    for (int m = 0; m < 8; ++m)
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) ln[hf] = mma32(xs[c][8 * hf + m], ws[m], ln[hf]);
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
      float nrm = 0.f;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const float4 mq = *reinterpret_cast<const float4 *>(stat + 64 * hf + 8 * q + 4 * g);
        const float4 iq = *reinterpret_cast<const float4 *>(stat + 64 * hf + 32 + 8 * q + 4 * g);
        const float mqa[4] = {mq.x, mq.y, mq.z, mq.w}, iqa[4] = {iq.x, iq.y, iq.z, iq.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int r = 4 * q + e, pt = 8 * q + 4 * g + e;
          float wv = __builtin_amdgcn_exp2f(ln[hf][r] * inv_t[hf] - mqa[e]) * iqa[e];
          if (pt >= valid) wv = 0.f;
          ln[hf][r] = wv;
          nrm += wv;
        }
      }
      nrm = half_sum(nrm);
      if (g == 0) mine[(h0 + hf) * (kS * kD1) + i * kD1 + kD] = nrm;
    }
    __builtin_amdgcn_wave_barrier();  // the statistics are read before the next pair overwrites them
    f32x16 tk[2];
#pragma unroll
    for (int r = 0; r < 16; ++r) tk[0][r] = tk[1][r] = 0.f;
#pragma unroll
    for (int m = 0; m < 16; ++m)
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) tk[hf] = mma32(ln[hf][m], fs[c][m], tk[hf]);
    // lane (i, g): channel i of the fx_mid tile = channel i % 16 of head h0 + i / 16, register r <-> slice
    // rowmap(r, g); each lane keeps the sums taken with its own head's weights
    const int hf = i >> 4;
#pragma unroll
    for (int r = 0; r < 16; ++r)
      mine[(h0 + hf) * (kS * kD1) + rowmap(r, g) * kD1 + (i & 15)] = hf ? tk[1][r] : tk[0][r];
  });
  __syncthreads();
  float *dst = partials + ((int64_t)gblk * B + b) * kTokFloats;
  for (int idx = tid; idx < kTokFloats; idx += 512)
    dst[idx] = ((red[idx] + red[kTokFloats + idx]) + red[2 * kTokFloats + idx]) + red[3 * kTokFloats + idx];
}

int64_t groups(const pa_shape &s);

// Linear projections (conv_k == 0: the irregular mesh) are the 1 x 1 case on an N x 1 grid.  One workgroup per 128
// points leaves one partial token sum each (17 KB): beyond 4096 of them per call the workspace and the combine pass
// outgrow what the front end saves, and the shape goes to the general kernels (whose partial count is capped).
bool supported(int dtype, const pa_shape &s) {
  if (dtype != PA_F32 || s.C != kC || s.H != kH || s.D != kD || s.S != kS || s.N * kC >= (int64_t)1 << 29) return false;
  if (groups(s) * s.B > 4096) return false;
  if (s.conv_k == 0) return s.grid_d == 0;
  return s.conv_k % 2 == 1 && s.grid_d == 0 && s.grid_h * s.grid_w == s.N;
}

int64_t groups(const pa_shape &s) { return ((s.N + 31) / 32 + 3) / 4; }

int64_t blob_bytes(const pa_shape &s) {
  const int64_t k = s.conv_k > 0 ? s.conv_k : 1;
  return k * k * kStepsPerTap * (int64_t)kStepUnits * 16 + 64;
}

int front(const pa_shape &s, const pa_params &p, const void *x, void *blob, void *w, float *partials, void *blob_out,
          const pa_block_mlp *mlp, hipStream_t st) {
  if (!supported(PA_F32, s)) return PA_ERR_UNSUPPORTED;
  const int ks = s.conv_k > 0 ? (int)s.conv_k : 1, taps = ks * ks;
  const int gh = s.conv_k > 0 ? (int)s.grid_h : (int)s.N, gw = s.conv_k > 0 ? (int)s.grid_w : 1;
  const int64_t units = (int64_t)taps * kStepsPerTap * kColTiles * 64;
  const int conv_blocks = (int)((units + 255) / 256);
  const int extra = !blob_out ? 0 : 8 + (mlp ? (int)(mlp->F / 128) * 16 : 0);
  hipLaunchKernelGGL(split_pack_kernel, dim3((unsigned)(conv_blocks + extra)), dim3(256), 0, st,
                     static_cast<const float *>(p.in_project_x_weight), static_cast<const float *>(p.in_project_fx_weight),
                     static_cast<u32x4 *>(blob), taps, (int)s.conv_tap_major, conv_blocks,
                     static_cast<const float *>(p.out_linear_weight), mlp ? static_cast<const float *>(mlp->w1) : nullptr,
                     mlp ? static_cast<const float *>(mlp->w2) : nullptr, mlp ? (int)mlp->F : 0,
                     static_cast<u32x4 *>(blob_out));
  int rc = launch_status();
  if (rc) return rc;
  if ((rc = allow_dynamic_lds(conv_slice_kernel, kLdsBytes))) return rc;
  const int bpb = (int)groups(s);
  hipLaunchKernelGGL(conv_slice_kernel, dim3((unsigned)(s.B * bpb)), dim3(512), kLdsBytes, st,
                     static_cast<const u32x4 *>(blob), p.in_project_x_bias, p.in_project_fx_bias,
                     static_cast<const float *>(p.in_project_slice_weight), p.in_project_slice_bias, p.temperature,
                     static_cast<const float *>(x), static_cast<float *>(w), partials, (int)s.B, (int)s.N,
                     gh, gw, ks, bpb);
  return launch_status();
}

}  // namespace conv
}  // namespace pa
