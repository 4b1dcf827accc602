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
    if (a.ks > 0 && m < a.M) {  // convolutions never use the padded numbering
      const int64_t b = m / a.N;
      int n = (int)(m - b * a.N);
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
        alignas(16) T e[UE];
#pragma unroll
        for (int j = 0; j < UE; ++j) {
          e[j] = T{};
          if (k_ok && o < a.O) e[j] = W[(int64_t)o * a.K + (int64_t)(c + j) * taps + tap];
        }
        pw[p] = *reinterpret_cast<const u32x4 *>(e);
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
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? PA_OK : (int)e;
}

template <typename T>
static int launch_n(const GemmArgs &a, int nsets, hipStream_t st) {
  if (a.O <= 64) return launch_t<T, 2>(a, nsets, st);
  if (a.O <= 128) return launch_t<T, 4>(a, nsets, st);
  return launch_t<T, 8>(a, nsets, st);
}

int launch(const GemmArgs &a, int nsets, int dtype, hipStream_t st) {
  return dtype == PA_F32 ? launch_n<float>(a, nsets, st) : launch_n<bf16>(a, nsets, st);
}

}  // namespace gemm
}  // namespace pa
