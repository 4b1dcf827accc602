// Row GEMM on the matrix cores for the general kernel family: out[m, o] = bias[o] + sum_k A(m, k) W[o, k], where
// A is either the rows of the input (Linear) or the gathered k x k (x k) neighbourhood of a grid point (Conv2d /
// Conv3d as implicit GEMM).  fp32 storage uses v_mfma_f32_32x32x2_f32 (fp32 products and sums: the result stays in
// the rtol-1e-4 class of the fp32 path), bf16 storage uses v_mfma_f32_32x32x16_bf16.
//
// Workgroup: 4 waves, 128 rows x (32 * NT) output columns; wave v owns rows 32v..32v+31 and NT accumulator tiles.
// The reduction axis is walked in blocks of 128 bytes per row (32 fp32 / 64 bf16 values = 8 units of 16 bytes).
// Both operand tiles are staged in LDS as [row][unit] with a row stride of 9 units: the 16 lanes of one 128-bit access
// phase (rows r..r+15, same unit) then fall on 16 distinct bank groups.  A lane (i, g) reads unit 2p + g of its row
// for p = 0..3: that is one bf16 MFMA operand (k = 8 values), or four fp32 operands (k = one value each).  Which k a
// lane holds is the same for A and W, so any assignment is a valid reduction order.
// The next block is fetched from global memory into registers while the MFMAs of the current one run.
#include "pa_common.h"
#include "pa_host.h"
#include "pa_mfma_ops.h"

namespace pa {
namespace gemm {

using mfma::f32x16;
using mfma::u32x4;

constexpr int kRows = 128;   // rows per workgroup
constexpr int kUnits = 8;    // 16-byte units per row and reduction block
constexpr int kRowU = 9;     // LDS row stride in units

template <typename T>
struct Unit;
template <>
struct Unit<float> {
  static constexpr int kElems = 4;
};
template <>
struct Unit<bf16> {
  static constexpr int kElems = 8;
};

__device__ __forceinline__ f32x16 mma_unit(const float *, u32x4 a, u32x4 b, f32x16 c) {
#pragma unroll
  for (int j = 0; j < 4; ++j)
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a[j]), __uint_as_float(b[j]), c, 0, 0, 0);
  return c;
}
__device__ __forceinline__ f32x16 mma_unit(const bf16 *, u32x4 a, u32x4 b, f32x16 c) { return mfma::mma(a, b, c); }

template <typename T, int NT>
__global__ __launch_bounds__(256) void rows_gemm_mfma_kernel(GemmArgs a) {
  constexpr int UE = Unit<T>::kElems, KB = kUnits * UE, BN = 32 * NT;
  __shared__ u32x4 As[kRows * kRowU];
  __shared__ u32x4 Ws[BN * kRowU];
  const int z = blockIdx.z;
  const T *in = static_cast<const T *>(a.in);
  const T *W = static_cast<const T *>(a.w[z]);
  const float *bias = a.bias[z];
  T *out = static_cast<T *>(a.out[z]);
  const int t = threadIdx.x, lane = t & 63, i = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int64_t m0 = (int64_t)blockIdx.x * kRows;
  const int o0 = blockIdx.y * BN;
  const int q = t & 7;    // the unit of a row this thread stages
  const int r0 = t >> 3;  // its first row; the others follow in steps of 32

  const int gd = a.gd > 0 ? a.gd : 1;
  const int ksd = a.gd > 0 ? a.ks : 1;
  const int taps = a.ks * a.ks * ksd;
  const int pad = a.ks / 2;

  // Row numbering: the rows of `in` in order, or (pack_tpb > 0) batch by batch with every batch padded to whole
  // 32-point tiles, so that a wave's 32 rows are one tile of one batch.
  const int64_t padded = (int64_t)a.pack_tpb * 32;  // rows per batch in the padded numbering
  auto real_row = [&](int64_t vm) -> int64_t {
    if (a.pack_tpb == 0) return vm < a.M ? vm : -1;
    const int64_t b = vm / padded, n = vm - b * padded;
    return (n < a.N && b * a.N + n < a.M) ? b * a.N + n : -1;
  };

  // the 4 input rows this thread stages: global row, and for a convolution its batch offset and grid coordinates
  int64_t arow[4];
  int ci[4], cj[4], cl[4];
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const int64_t m = m0 + r0 + 32 * p;
    arow[p] = real_row(m);
    ci[p] = cj[p] = cl[p] = 0;
    if (a.ks > 0 && arow[p] >= 0) {  // grid coordinates from the real row (the padded numbering skips rows)
      const int64_t b = arow[p] / a.N;
      int n = (int)(arow[p] - b * a.N);
      cl[p] = n % gd;
      n /= gd;
      ci[p] = n / a.gw;
      cj[p] = n - ci[p] * a.gw;
      arow[p] = b * a.N;  // first point of the row's batch
    }
  }

  u32x4 pa[4], pw[NT];
  auto fetch = [&](int kb) {
    const int k = kb * KB + q * UE;
    const bool k_ok = k < a.K;
    if (a.ks == 0) {
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        pa[p] = u32x4{0, 0, 0, 0};
        if (k_ok && arow[p] >= 0) pa[p] = *reinterpret_cast<const u32x4 *>(in + arow[p] * a.K + k);
      }
#pragma unroll
      for (int p = 0; p < NT; ++p) {
        const int o = o0 + r0 + 32 * p;
        pw[p] = u32x4{0, 0, 0, 0};
        if (k_ok && o < a.O) pw[p] = *reinterpret_cast<const u32x4 *>(W + (int64_t)o * a.K + k);
      }
    } else {
      const int tap = k / a.C, c = k - tap * a.C;
      const int uv = tap / ksd, zz = tap - uv * ksd;
      const int u = uv / a.ks, v = uv - u * a.ks;
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        const int ii = ci[p] + u - pad, jj = cj[p] + v - pad, ll = cl[p] + (a.gd > 0 ? zz - pad : 0);
        pa[p] = u32x4{0, 0, 0, 0};
        if (k_ok && arow[p] >= 0 && ii >= 0 && ii < a.gh && jj >= 0 && jj < a.gw && ll >= 0 && ll < gd)
          pa[p] = *reinterpret_cast<const u32x4 *>(in + (arow[p] + ((int64_t)ii * a.gw + jj) * gd + ll) * a.C + c);
      }
#pragma unroll
      for (int p = 0; p < NT; ++p) {
        const int o = o0 + r0 + 32 * p;
        if (a.w_tap_major) {  // W[o][tap][c]: the unit is contiguous, as for a Linear
          pw[p] = u32x4{0, 0, 0, 0};
          if (k_ok && o < a.O) pw[p] = *reinterpret_cast<const u32x4 *>(W + (int64_t)o * a.K + k);
        } else {
          alignas(16) T e[UE];
#pragma unroll
          for (int j = 0; j < UE; ++j) {
            e[j] = T{};
            if (k_ok && o < a.O) e[j] = W[(int64_t)o * a.K + (int64_t)(c + j) * taps + tap];
          }
          pw[p] = *reinterpret_cast<const u32x4 *>(e);
        }
      }
    }
  };

  f32x16 acc[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[nt][r] = 0.f;

  const int nkb = (a.K + KB - 1) / KB;
  fetch(0);
  for (int kb = 0; kb < nkb; ++kb) {
#pragma unroll
    for (int p = 0; p < 4; ++p) As[(r0 + 32 * p) * kRowU + q] = pa[p];
#pragma unroll
    for (int p = 0; p < NT; ++p) Ws[(r0 + 32 * p) * kRowU + q] = pw[p];
    __syncthreads();
    fetch(kb + 1 < nkb ? kb + 1 : kb);  // the last block re-fetches itself: no branch around the loads
    const u32x4 *ar = As + (wave * 32 + i) * kRowU + g;
    const u32x4 *wr = Ws + i * kRowU + g;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const u32x4 av = ar[2 * p];
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) acc[nt] = mma_unit(in, av, wr[nt * 32 * kRowU + 2 * p], acc[nt]);
    }
    __syncthreads();
  }

  const int64_t tile = (int64_t)blockIdx.x * 4 + wave;  // this wave's 32 rows (one (batch, tile) when packing)
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int o = o0 + nt * 32 + i;
    if (o >= a.O) continue;
    const float bv = bias ? bias[o] : 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[nt][r] += bv;
    if (a.act == 1) {
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[nt][r] = gelu_erf(acc[nt][r]);
    }
    if (out) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int64_t m = real_row(tile * 32 + mfma::rowmap(r, g));
        if (m >= 0) store_from_f32(out + m * a.O + o, acc[nt][r]);
      }
    }
    if constexpr (sizeof(T) == 2) {
      u32x4 *pk = static_cast<u32x4 *>(a.out_pack[z]);
      const int head = (o0 >> 5) + nt;
      if (a.pack_tpb > 0 && pk && tile * 32 < (a.M / a.N) * padded) {
        pk[((tile * a.pack_heads + head) * 2 + 0) * 64 + lane] = mfma::pack_half<0>(acc[nt]);
        pk[((tile * a.pack_heads + head) * 2 + 1) * 64 + lane] = mfma::pack_half<1>(acc[nt]);
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------
// rows_linear_kernel: the bf16 Linear over very many rows, weights stationary.  out = in . W^T + bias with
// K = 16 * KS in {128, 256, 512} and up to 256 output columns per workgroup (grid.y walks wider outputs, grid.z the
// second (W, bias, out) set).  One wave per 32 output columns keeps its W rows in registers (KS operand fragments) for
// the whole kernel; the workgroup walks the 32-row tiles g, g + G, ... of its batch range; a tile's rows are staged in
// LDS by the whole workgroup with full-row coalesced loads ([row][unit] with one unit of stagger per row, see above)
// and read back as operand fragments by every wave; the next tile is fetched into registers while the current one is
// multiplied.  The product is formed as out^T (channels x rows: lanes <-> rows, registers <-> channels) so that a
// row's 32 channels leave as 16-byte stores; with packing on, the un-transposed tile (lanes <-> channels) is formed
// as well and written in the packed operand layout of the slice kernels.
// Rows are numbered as in rows_gemm_mfma_kernel (padded per batch when pack_tpb > 0).
// ------------------------------------------------------------------------------------------------
template <int KS>
__global__ __launch_bounds__(512) void rows_linear_kernel(GemmArgs a) {
  constexpr int K = 16 * KS, UPR = K / 8, ROWU = UPR + 1;
  extern __shared__ u32x4 xs_all[];
  u32x4(*xs)[32 * ROWU] = reinterpret_cast<u32x4(*)[32 * ROWU]>(xs_all);  // two tile buffers
  const int z = blockIdx.z;
  const uint16_t *in = static_cast<const uint16_t *>(a.in);
  const uint16_t *W = static_cast<const uint16_t *>(a.w[z]);
  uint16_t *out = static_cast<uint16_t *>(a.out[z]);
  u32x4 *pk = static_cast<u32x4 *>(a.out_pack[z]);
  const int tid = threadIdx.x, lane = tid & 63, i = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int NT = blockDim.x;
  const int o0 = blockIdx.y * 256 + wave * 32;  // this wave's output columns

  u32x4 wf[KS];  // W[o0 + i][16 ks + 8 g + j]: the A operand of out^T and the B operand of the un-transposed tile
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
    wf[ks] = *reinterpret_cast<const u32x4 *>(W + (int64_t)(o0 + i) * K + 16 * ks + 8 * g);
  float bias_t[16];  // bias of channel rowmap(r, g) (out^T: registers <-> channels)
#pragma unroll
  for (int r = 0; r < 16; ++r) bias_t[r] = a.bias[z] ? a.bias[z][o0 + mfma::rowmap(r, g)] : 0.f;
  const float bias_n = a.bias[z] ? a.bias[z][o0 + i] : 0.f;

  const int64_t padded = (int64_t)a.pack_tpb * 32;
  const int64_t ntiles = a.pack_tpb > 0 ? (a.M / a.N) * a.pack_tpb : (a.M + 31) / 32;
  auto real_row = [&](int64_t vm) -> int64_t {
    if (a.pack_tpb == 0) return vm < a.M ? vm : -1;
    const int64_t b = vm / padded, n = vm - b * padded;
    return (n < a.N && b * a.N + n < a.M) ? b * a.N + n : -1;
  };
  // staging: unit idx = k * NT + tid of the tile -> row idx / UPR, position idx % UPR; 32 * UPR units per tile
  const int per_thread = (32 * UPR + NT - 1) / NT;
  u32x4 stg[4];  // per_thread <= 4 for every supported (K, workgroup size) pair
  auto stage_load = [&](int64_t tile) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int idx = k * NT + tid;
      stg[k] = u32x4{0, 0, 0, 0};
      if (k < per_thread && idx < 32 * UPR) {
        const int rc = idx / UPR, pos = idx - rc * UPR;
        const int64_t m = real_row(tile * 32 + rc);
        if (m >= 0) stg[k] = *reinterpret_cast<const u32x4 *>(in + m * K + pos * 8);
      }
    }
  };
  auto stage_store = [&](int buf) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int idx = k * NT + tid;
      if (k < per_thread && idx < 32 * UPR) {
        const int rc = idx / UPR, pos = idx - rc * UPR;
        xs[buf][rc * ROWU + pos] = stg[k];
      }
    }
  };

  int64_t tile = blockIdx.x;
  if (tile < ntiles) {
    stage_load(tile);
    stage_store(0);
  }
  __syncthreads();
  int buf = 0;
  for (; tile < ntiles; tile += gridDim.x, buf ^= 1) {
    const int64_t next = tile + gridDim.x < ntiles ? tile + gridDim.x : tile;  // the last tile re-fetches itself
    stage_load(next);
    const u32x4 *xb = &xs[buf][i * ROWU + g];
    f32x16 acc_t, acc_n;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      acc_t[r] = bias_t[r];
      acc_n[r] = bias_n;
    }
    if (pk) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const u32x4 xf = xb[2 * ks];
        acc_t = mfma::mma(wf[ks], xf, acc_t);
        acc_n = mfma::mma(xf, wf[ks], acc_n);
      }
    } else {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) acc_t = mfma::mma(wf[ks], xb[2 * ks], acc_t);
    }
    if (out) {
      const int64_t m = real_row(tile * 32 + i);
      mfma::store_tile_natural(acc_t, out + (m >= 0 ? m : 0) * a.O + o0, g, m >= 0);
    }
    if (pk) {
      const int head = o0 >> 5;
      pk[((tile * a.pack_heads + head) * 2 + 0) * 64 + lane] = mfma::pack_half<0>(acc_n);
      pk[((tile * a.pack_heads + head) * 2 + 1) * 64 + lane] = mfma::pack_half<1>(acc_n);
    }
    stage_store(buf ^ 1);
    __syncthreads();
  }
}

bool linear_serves(const GemmArgs &a, int nsets, size_t elem_bytes) {
  if (elem_bytes != 2 || a.ks != 0 || a.act != 0) return false;  // activations: the tiled kernel
  if (a.K != 128 && a.K != 256 && a.K != 512) return false;
  if (a.O % 32 != 0 || (a.O > 256 && a.O % 256 != 0)) return false;
  if (a.M < 4096) return false;  // small problems: the tiled kernel has less fixed cost
  if ((a.O < 256 ? a.O : 256) * 2 < a.K) return false;  // staging: at most 4 units per thread and tile
  if (!aligned16(a.in)) return false;
  for (int z = 0; z < nsets; ++z)
    if (!aligned16(a.w[z]) || !aligned16(a.out[z]) || (!a.out[z] && !a.out_pack[z])) return false;
  return true;
}

int linear_launch(const GemmArgs &a, int nsets, int num_cu, hipStream_t st) {
  const int64_t ntiles = a.pack_tpb > 0 ? (a.M / a.N) * a.pack_tpb : (a.M + 31) / 32;
  const int waves = (a.O < 256 ? a.O : 256) / 32;
  // resident workgroups: the register-held weights leave room for one 8-wave workgroup per CU (two for K = 128)
  int64_t gx = (a.K == 128 ? 2 : 1) * (int64_t)num_cu / (((a.O + 255) / 256) * nsets);
  if (gx < 1) gx = 1;
  if (gx > ntiles) gx = ntiles;
  const dim3 grid((unsigned)gx, (unsigned)((a.O + 255) / 256), (unsigned)nsets), block((unsigned)(waves * 64));
  const size_t lds = (size_t)2 * 32 * (a.K / 8 + 1) * 16;  // only K = 512 exceeds the default limit
  if (int rc = allow_dynamic_lds(rows_linear_kernel<32>, a.K == 512 ? lds : 0)) return rc;
  switch (a.K) {
    case 128: hipLaunchKernelGGL((rows_linear_kernel<8>), grid, block, lds, st, a); break;
    case 256: hipLaunchKernelGGL((rows_linear_kernel<16>), grid, block, lds, st, a); break;
    case 512: hipLaunchKernelGGL((rows_linear_kernel<32>), grid, block, lds, st, a); break;
    default: return PA_ERR_UNSUPPORTED;
  }
  return launch_status();
}

// ------------------------------------------------------------------------------------------------
// cols_gemm_kernel: weight-gradient products  P[oa][ob] = sum_m A[m][oa] * B[m][ob]  over a huge row count m (bf16
// rows in natural layout, fp32 result).  grid (G row chunks, OA / 256); workgroup = one wave per 32 columns of A (up to
// 8); wave w owns output rows 32w..32w+31 and all NB = OB / 32 column groups.  Both operands have the reduction index m
// as their slow index in memory, so each 32-row block is transposed on the matrix cores first: the natural 16-byte
// loads are MFMA A operands (lane <-> row m, k <-> channel); multiplied by 0/1 selection matrices they give an exact copy
// of the block with lanes <-> channels and registers <-> rows, which, converted back to bf16, is an operand whose
// reduction index is m.  Every wave transposes its own A group; the B groups are transposed once per workgroup and
// shared through LDS (double buffered, one barrier per block).  Each chunk leaves one partial result
// partials[g][oa][ob]; the caller adds the G partials up in index order.
// ------------------------------------------------------------------------------------------------
template <int NB>
__global__ __launch_bounds__(512) void cols_gemm_kernel(const uint16_t *__restrict__ A, int lda, int OA,
                                                        const uint16_t *__restrict__ B, int ldb, int64_t M,
                                                        int64_t blocks_per_chunk, float *__restrict__ partials,
                                                        float *__restrict__ col_sums) {
  constexpr int OB = 32 * NB;
  __shared__ u32x4 bts[2][NB * 2 * 64];
  const int tid = threadIdx.x, lane = tid & 63, i = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nwaves = blockDim.x >> 6;
  const int a0 = blockIdx.y * 256 + wave * 32;  // first A column of this wave

  u32x4 sel[2];  // sel[kk]: column i receives the k element whose channel is 16kk + 8g + j
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) {
    mfma::bf16x8 s8;
#pragma unroll
    for (int j = 0; j < 8; ++j) s8[j] = (__bf16)((i == 16 * kk + 8 * g + j) ? 1.f : 0.f);
    sel[kk] = __builtin_bit_cast(u32x4, s8);
  }
  // a 32 x 32 block (rows m0.., columns c0..) of a natural-layout matrix -> two operands whose k index runs over m
  auto transposed = [&](const uint16_t *base, int ld, int64_t m0, int c0, u32x4 &t0, u32x4 &t1) {
    const int64_t m = m0 + i;
    u32x4 f0 = u32x4{0, 0, 0, 0}, f1 = f0;
    if (m < M) {
      const uint16_t *row = base + m * ld + c0 + 8 * g;
      f0 = *reinterpret_cast<const u32x4 *>(row);
      f1 = *reinterpret_cast<const u32x4 *>(row + 16);
    }
    f32x16 t;
#pragma unroll
    for (int r = 0; r < 16; ++r) t[r] = 0.f;
    t = mfma::mma(f0, sel[0], t);
    t = mfma::mma(f1, sel[1], t);
    t0 = mfma::pack_half<0>(t);
    t1 = mfma::pack_half<1>(t);
  };

  f32x16 acc[NB], acc_s;  // acc_s: A^T . 1 (every column the same): the column sums of A
#pragma unroll
  for (int r = 0; r < 16; ++r) acc_s[r] = 0.f;
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[nb][r] = 0.f;
  const u32x4 ones = u32x4{0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u};  // 8 x bf16(1.0)

  const int64_t blk0 = (int64_t)blockIdx.x * blocks_per_chunk;
  const int64_t nblk = (M + 31) / 32;
  int64_t blk_end = blk0 + blocks_per_chunk;
  if (blk_end > nblk) blk_end = nblk;
  int buf = 0;
  for (int64_t blk = blk0; blk < blk_end; ++blk, buf ^= 1) {
    const int64_t m0 = blk * 32;
    u32x4 at0, at1;
    transposed(A, lda, m0, a0, at0, at1);
    if (col_sums) {
      acc_s = mfma::mma(at0, ones, acc_s);
      acc_s = mfma::mma(at1, ones, acc_s);
    }
    for (int nb = wave; nb < NB; nb += nwaves) {
      u32x4 b0, b1;
      transposed(B, ldb, m0, 32 * nb, b0, b1);
      bts[buf][(nb * 2 + 0) * 64 + lane] = b0;
      bts[buf][(nb * 2 + 1) * 64 + lane] = b1;
    }
    __syncthreads();
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      acc[nb] = mfma::mma(at0, bts[buf][(nb * 2 + 0) * 64 + lane], acc[nb]);
      acc[nb] = mfma::mma(at1, bts[buf][(nb * 2 + 1) * 64 + lane], acc[nb]);
    }
  }
  float *dst = partials + ((int64_t)blockIdx.x * OA + a0) * OB;
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int r = 0; r < 16; ++r) dst[(int64_t)mfma::rowmap(r, g) * OB + 32 * nb + i] = acc[nb][r];
  if (col_sums && i == 0) {
#pragma unroll
    for (int r = 0; r < 16; ++r) col_sums[(int64_t)blockIdx.x * OA + a0 + mfma::rowmap(r, g)] = acc_s[r];
  }
}

// row chunks: about two workgroups per CU over all column groups, and at least 32 blocks of 32 rows per chunk so that
// ------------------------------------------------------------------------------------------------
// cols_gemm_f32_kernel: the float32 form of the weight-gradient product  P[oa][ob] = sum_m A[m][oa] * B[m][ob].
// v_mfma_f32_32x32x2_f32 reduces over two rows m per instruction with lane (i, g) supplying A[m0 + g][oa0 + i] and
// B[m0 + g][ob0 + i]: consecutive lanes read consecutive columns of a row, so natural row-major operands need no
// transposition.  A workgroup (4 waves) owns a 128 x 128 block of P for one chunk of rows: 32 rows of its 128 + 128
// operand columns at a time go through LDS (coalesced 16-byte loads, double buffered), wave w multiplies the 64 x 64
// sub-block (w & 1, w >> 1): per pair of rows 2 + 2 LDS words feed 4 MFMAs.  Row chunks come back as partials
// P[g][oa][ob] (fixed-order sum by the caller); col_sums[g][oa] = sum_m A[m][oa] from the same pass (blockIdx.z == 0).
// ------------------------------------------------------------------------------------------------
constexpr int kF32Tile = 128, kF32Rows = 32;

__global__ __launch_bounds__(256) void cols_gemm_f32_kernel(const float *__restrict__ A, int lda, int OA,
                                                            const float *__restrict__ B, int ldb, int OB, int64_t M,
                                                            int64_t rows_per_chunk, float *__restrict__ partials,
                                                            float *__restrict__ col_sums) {
  __shared__ float As[2][kF32Rows][kF32Tile];
  __shared__ float Bs[2][kF32Rows][kF32Tile];
  const int t = threadIdx.x, lane = t & 63, i = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int oa0 = blockIdx.y * kF32Tile, ob0 = blockIdx.z * kF32Tile;
  const int64_t m_begin = (int64_t)blockIdx.x * rows_per_chunk;
  const int64_t m_end = min(M, m_begin + rows_per_chunk);
  const int wa = (wave & 1) * 64, wb = (wave >> 1) * 64;  // this wave's sub-block of the tile

  f32x16 acc[2][2];
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int v = 0; v < 2; ++v)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[u][v][r] = 0.f;
  float csum[2] = {0.f, 0.f};

  // staging: 32 rows x 128 columns = 1024 float4 per operand, 4 per thread
  const int sr = t >> 5, sc = (t & 31) * 4;  // row 0..7 (+8 k), column of the float4
  float4 pa[4], pb[4];
  auto fetch = [&](int64_t m0) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int64_t m = m0 + sr + 8 * k;
      pa[k] = pb[k] = float4{0.f, 0.f, 0.f, 0.f};
      if (m < m_end) {
        if (oa0 + sc < OA) pa[k] = *reinterpret_cast<const float4 *>(A + m * lda + oa0 + sc);
        if (ob0 + sc < OB) pb[k] = *reinterpret_cast<const float4 *>(B + m * ldb + ob0 + sc);
      }
    }
  };
  auto stage = [&](int buf) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      *reinterpret_cast<float4 *>(&As[buf][sr + 8 * k][sc]) = pa[k];
      *reinterpret_cast<float4 *>(&Bs[buf][sr + 8 * k][sc]) = pb[k];
    }
  };
  fetch(m_begin);
  int buf = 0;
  for (int64_t m0 = m_begin; m0 < m_end; m0 += kF32Rows) {
    stage(buf);
    __syncthreads();
    fetch(m0 + kF32Rows < m_end ? m0 + kF32Rows : m0);  // the last block re-fetches itself: no branch around the loads
#pragma unroll 4
    for (int k = 0; k < kF32Rows; k += 2) {
      const float a0 = As[buf][k + g][wa + i], a1 = As[buf][k + g][wa + 32 + i];
      const float b0 = Bs[buf][k + g][wb + i], b1 = Bs[buf][k + g][wb + 32 + i];
      acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc[0][0], 0, 0, 0);
      acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b1, acc[0][1], 0, 0, 0);
      acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b0, acc[1][0], 0, 0, 0);
      acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b1, acc[1][1], 0, 0, 0);
      csum[0] += a0;
      csum[1] += a1;
    }
    buf ^= 1;
  }
  // C/D layout: lane (i, g) holds column ob = i, register r holds row oa = rowmap(r, g)
  float *dst = partials + (int64_t)blockIdx.x * OA * OB;
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int v = 0; v < 2; ++v) {
      const int ob = ob0 + wb + 32 * v + i;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int oa = oa0 + wa + 32 * u + mfma::rowmap(r, g);
        if (oa < OA && ob < OB) dst[(int64_t)oa * OB + ob] = acc[u][v][r];
      }
    }
  if (col_sums && blockIdx.z == 0 && (wave >> 1) == 0) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const float total = csum[u] + __shfl_xor(csum[u], 32, 64);  // the two row parities
      const int oa = oa0 + wa + 32 * u + i;
      if (g == 0 && oa < OA) col_sums[(int64_t)blockIdx.x * OA + oa] = total;
    }
  }
}

int64_t cols_gemm_f32_chunks(int64_t M, int64_t OA, int64_t OB, int num_cu) {
  const int64_t tiles = ((OA + kF32Tile - 1) / kF32Tile) * ((OB + kF32Tile - 1) / kF32Tile);
  int64_t g = (3 * (int64_t)num_cu + tiles - 1) / tiles;  // about three workgroups per compute unit in all
  const int64_t cap = (M + 1023) / 1024;                  // at least 1024 rows per chunk
  if (g > cap) g = cap;
  return g < 1 ? 1 : g;
}

int cols_gemm_f32(const void *A, int64_t lda, int64_t OA, const void *B, int64_t ldb, int64_t OB, int64_t M,
                  float *partials, float *col_sums, int num_cu, hipStream_t st) {
  if (OA <= 0 || OB <= 0 || OA % 4 != 0 || OB % 4 != 0 || lda % 4 != 0 || ldb % 4 != 0) return PA_ERR_UNSUPPORTED;
  const int64_t G = cols_gemm_f32_chunks(M, OA, OB, num_cu);
  int64_t per = (M + G - 1) / G;
  per = (per + kF32Rows - 1) / kF32Rows * kF32Rows;
  const dim3 grid((unsigned)G, (unsigned)((OA + kF32Tile - 1) / kF32Tile), (unsigned)((OB + kF32Tile - 1) / kF32Tile));
  hipLaunchKernelGGL(cols_gemm_f32_kernel, grid, dim3(256), 0, st, static_cast<const float *>(A), (int)lda, (int)OA,
                     static_cast<const float *>(B), (int)ldb, (int)OB, M, per, partials, col_sums);
  return launch_status();
}

// ------------------------------------------------------------------------------------------------
// cols_gemm_lds_kernel: the same product with the transposition done by the LDS read instead of on the matrix
// cores.  A workgroup (8 waves, 4 along A's columns x 2 along B's) owns a 256 x 256 block of P for its chunk of rows;
// 32 rows of both operands at a time are staged in LDS as they lie in memory (16-byte loads and writes; row stride 288
// elements), and a lane receives its operand -- eight consecutive rows m of one column -- from two transposing reads
// (ds_read_b64_tr_b16: within a group of 16 lanes, lane l receives element l % 4 of what lanes l / 4, 4 + l / 4,
// 8 + l / 4, 12 + l / 4 address; lane L addresses row m0 + L / 4, columns c0 + 4 (L % 4) .. + 3, so lane l ends up with
// column c0 + l of rows m0 .. m0 + 3).  With 144 words between rows the four rows a half-wave reads fall on four
// different quarters of the banks.  Wave tile 64 x 128: 6 operand fragments (12 reads) feed 8 MFMAs.
// grid (G row chunks, ceil(OA / 256)); OB <= 256.
// ------------------------------------------------------------------------------------------------
constexpr int kColsLd = 288;

__global__ __launch_bounds__(512) void cols_gemm_lds_kernel(const uint16_t *__restrict__ A, int lda, int OA,
                                                            const uint16_t *__restrict__ B, int ldb, int OB, int64_t M,
                                                            int64_t per, float *__restrict__ partials,
                                                            float *__restrict__ col_sums) {
  typedef short v4i16 __attribute__((ext_vector_type(4)));
  typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
  typedef __attribute__((address_space(3))) v4i16 *lds_v4i16;
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  extern __shared__ u32x4 cols_smem[];
  uint16_t *As = reinterpret_cast<uint16_t *>(cols_smem);  // [2][32 * kColsLd]
  uint16_t *Bs = As + 2 * 32 * kColsLd;                     // [2][32 * kColsLd]
  const int t = threadIdx.x, lane = t & 63, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int wa = (wave & 3) * 64, wb = (wave >> 2) * 128;
  const int oa0 = blockIdx.y * 256;
  const int64_t blk0 = (int64_t)blockIdx.x * per, nblk = (M + 31) / 32;
  const int64_t blk1 = blk0 + per < nblk ? blk0 + per : nblk;

  f32x16 acc[2][4];
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int v = 0; v < 4; ++v)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[u][v][r] = 0.f;
  float csum[2] = {0.f, 0.f};

  // staging: 32 rows x 32 units of 8 columns per operand = 1024 units, two per thread
  const int sr = t >> 5, su = (t & 31) * 8;  // row (and row + 16), first column of the unit
  u32x4 pa[2], pb[2];
  auto fetch = [&](int64_t blk) {
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const int64_t m = blk * 32 + sr + 16 * k;
      pa[k] = pb[k] = u32x4{0, 0, 0, 0};
      if (m < M) {
        if (oa0 + su < OA) pa[k] = *reinterpret_cast<const u32x4 *>(A + m * lda + oa0 + su);
        if (su < OB) pb[k] = *reinterpret_cast<const u32x4 *>(B + m * ldb + su);
      }
    }
  };
  auto stage = [&](int buf) {
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      *reinterpret_cast<u32x4 *>(&As[(buf * 32 + sr + 16 * k) * kColsLd + su]) = pa[k];
      *reinterpret_cast<u32x4 *>(&Bs[(buf * 32 + sr + 16 * k) * kColsLd + su]) = pb[k];
    }
  };
  // this lane's address inside a 32-row tile for the rows 8 g .. 8 g + 3 of k-step 0 and the 16 columns its group
  // of lanes stands for (see above); k-step, upper four rows and column tile are constant offsets
  const int l16 = lane & 15, q1 = (lane >> 4) & 1;
  const int lane_off = (8 * g + (l16 >> 2)) * kColsLd + 16 * q1 + 4 * (l16 & 3);
  auto operand = [&](const uint16_t *tile, int ks, int col) {  // rows 16 ks + 8 g .. + 7 of column col + (lane & 31)
    const uint16_t *p = tile + lane_off + 16 * ks * kColsLd + col;
    const u32x2 lo = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16)(uintptr_t)p));
    const u32x2 hi =
        __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16)(uintptr_t)(p + 4 * kColsLd)));
    return u32x4{lo[0], lo[1], hi[0], hi[1]};
  };
  const bf16x2 ones = {(__bf16)1.f, (__bf16)1.f};
  if (blk0 < blk1) fetch(blk0);
  int buf = 0;
  for (int64_t blk = blk0; blk < blk1; ++blk) {
    stage(buf);
    __syncthreads();
    if (blk + 1 < blk1) fetch(blk + 1);
    const uint16_t *at = As + buf * 32 * kColsLd, *bt = Bs + buf * 32 * kColsLd;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      u32x4 af[2], bf[4];
#pragma unroll
      for (int u = 0; u < 2; ++u) af[u] = operand(at, ks, wa + 32 * u);
#pragma unroll
      for (int v = 0; v < 4; ++v) bf[v] = operand(bt, ks, wb + 32 * v);
#pragma unroll
      for (int u = 0; u < 2; ++u) {
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[u][v] = mfma::mma(af[u], bf[v], acc[u][v]);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t word = af[u][j];
          csum[u] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, word), ones, csum[u], false);
        }
      }
    }
    buf ^= 1;
  }
  const int i = lane & 31;
  float *dst = partials + (int64_t)blockIdx.x * OA * OB;
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int ob = wb + 32 * v + i;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int oa = oa0 + wa + 32 * u + mfma::rowmap(r, g);
        if (oa < OA && ob < OB) dst[(int64_t)oa * OB + ob] = acc[u][v][r];
      }
    }
  if (col_sums && (wave >> 2) == 0) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const float total = csum[u] + __shfl_xor(csum[u], 32, 64);
      const int oa = oa0 + wa + 32 * u + i;
      if (g == 0 && oa < OA) col_sums[(int64_t)blockIdx.x * OA + oa] = total;
    }
  }
}

// the partial results stay small next to the rows a chunk reads
int64_t cols_gemm_chunks(int64_t M, int64_t OA, int num_cu) {
  const int64_t nblk = (M + 31) / 32, gy = (OA + 255) / 256;
  int64_t g = 2 * (int64_t)num_cu / gy;
  if (g > nblk / 32) g = nblk / 32;
  return g < 1 ? 1 : g;
}

int cols_gemm(const void *A, int64_t lda, int64_t OA, const void *B, int64_t ldb, int64_t OB, int64_t M,
              float *partials, float *col_sums, int num_cu, hipStream_t st) {
  if (OA % 32 != 0 || OB % 32 != 0 || OA <= 0 || OB <= 0 || lda % 8 != 0 || ldb % 8 != 0) return PA_ERR_UNSUPPORTED;
  if (OA > 256 && OA % 256 != 0) return PA_ERR_UNSUPPORTED;
  const int64_t G = cols_gemm_chunks(M, OA, num_cu);
  const int64_t nblk = (M + 31) / 32;
  const int64_t per = (nblk + G - 1) / G;
  const dim3 grid((unsigned)G, (unsigned)((OA + 255) / 256)), block((unsigned)((OA < 256 ? OA : 256) * 2));
  const uint16_t *a = static_cast<const uint16_t *>(A), *b = static_cast<const uint16_t *>(B);
  if (OA >= 128 && OB >= 128 && OB <= 256) {  // wide products: the LDS-gather kernel (its 256 x 256 tile would idle on narrow ones)
    const size_t lds = (size_t)4 * 32 * kColsLd * 2;
    const int rc = allow_dynamic_lds(cols_gemm_lds_kernel, lds);
    if (rc) return rc;
    hipLaunchKernelGGL(cols_gemm_lds_kernel, dim3((unsigned)G, (unsigned)((OA + 255) / 256)), dim3(512), lds, st, a,
                       (int)lda, (int)OA, b, (int)ldb, (int)OB, M, per, partials, col_sums);
    return launch_status();
  }
#define PA_COLS(NBV) \
  hipLaunchKernelGGL((cols_gemm_kernel<NBV>), grid, block, 0, st, a, (int)lda, (int)OA, b, (int)ldb, M, per, partials, col_sums)
  switch (OB / 32) {
    case 1: PA_COLS(1); break;
    case 2: PA_COLS(2); break;
    case 4: PA_COLS(4); break;
    case 8: PA_COLS(8); break;
    default: return PA_ERR_UNSUPPORTED;
  }
#undef PA_COLS
  return launch_status();
}

bool serves(const GemmArgs &a, int nsets, size_t elem_bytes) {
  const int ue = (int)(16 / elem_bytes);
  if (a.K % ue != 0) return false;                      // rows must be whole 16-byte units
  if (a.ks > 0 && a.C % ue != 0) return false;          // a unit must not straddle two taps
  if (!aligned16(a.in)) return false;
  for (int z = 0; z < nsets; ++z)
    if (!aligned16(a.w[z]) || (!a.out[z] && !a.out_pack[z])) return false;
  return true;
}

template <typename T, int NT>
static int launch_t(const GemmArgs &a, int nsets, hipStream_t st) {
  const int64_t rows = a.pack_tpb > 0 ? (a.M / a.N) * a.pack_tpb * 32 : a.M;
  dim3 grid((unsigned)((rows + kRows - 1) / kRows), (unsigned)((a.O + 32 * NT - 1) / (32 * NT)), (unsigned)nsets);
  hipLaunchKernelGGL((rows_gemm_mfma_kernel<T, NT>), grid, dim3(256), 0, st, a);
  return launch_status();
}

template <typename T>
static int launch_n(const GemmArgs &a, int nsets, hipStream_t st) {
  if (a.O <= 64) return launch_t<T, 2>(a, nsets, st);
  if (a.O <= 128) return launch_t<T, 4>(a, nsets, st);
  return launch_t<T, 8>(a, nsets, st);
}

int launch(const GemmArgs &a, int nsets, int dtype, hipStream_t st) {
  if (dtype == PA_BF16 && linear_serves(a, nsets, 2)) {
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
      cus = 256;
    return linear_launch(a, nsets, cus, st);
  }
  return dtype == PA_F32 ? launch_n<float>(a, nsets, st) : launch_n<bf16>(a, nsets, st);
}

}  // namespace gemm
}  // namespace pa
