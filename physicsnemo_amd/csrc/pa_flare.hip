// FLARE attention (physicsnemo/nn/module/flare_attention.py:38-72, :195-255): low-rank attention through S learned global
// queries per head.  With the scores A[b,n,h,s] = k[b,n,h,:] . q_global[h,s,:] (scale 1) the two passes are
//   z[b,h,s,:] = sum_n softmax_n(A[b,:,h,s])[n] v[b,n,h,:]       (the queries gather from all points)
//   y[b,n,h,:] = sum_s softmax_s(A[b,n,h,:])[s] z[b,h,s,:]       (every point reads the S summaries back)
// which is the slice aggregation and the deslice of the PhysicsAttention layer with two different normalisations of
// the same score matrix.  The scores and v come from the row GEMM kernels (the caller folds in_project_x, self_k /
// self_v and q_global into two weight matrices); this file holds what is particular to FLARE:
//   column_max_kernel(s)     m[b,h,s] = max_n A[b,n,h,s]                     two passes, like the slice aggregation
//   column_weights_kernel    wc = exp(A - m)                                   -> pa_slice_reduce(wc, v) gives z
//   softmax_rows_kernel      A <- softmax_s(A) in place                        -> pa_deslice_project(A, z) gives y
//   flare_backward_kernel    per-point part of the backward pass: d A, d v
// fp32 arithmetic, fp32 or bf16 storage, natural layouts.
#include "pa_common.h"
#include "pa_host.h"
#include "pa_mfma_ops.h"

namespace pa {
namespace flare {

constexpr int kChunkRows = 256;  // points per workgroup of the first column-max pass

// grid (chunks, B).  Workgroup (g, b): column maxima of rows [g*256, g*256+256) of batch b over all H*S columns.
template <typename T>
__global__ __launch_bounds__(256) void column_max_partial_kernel(const T *__restrict__ a, float *__restrict__ partial,
                                                                 int64_t N, int HS) {
  const int g = blockIdx.x, b = blockIdx.y;
  const int64_t n0 = (int64_t)g * kChunkRows;
  const int rows = (int)min((int64_t)kChunkRows, N - n0);
  const T *src = a + ((int64_t)b * N + n0) * HS;
  for (int c = threadIdx.x; c < HS; c += 256) {  // consecutive threads <-> consecutive columns: coalesced rows
    float m = -INFINITY;
    for (int r = 0; r < rows; ++r) m = fmaxf(m, load_as_f32(src + (int64_t)r * HS + c));
    partial[((int64_t)g * gridDim.y + b) * HS + c] = m;
  }
}

// The same with 16-byte loads, for rows that are whole numbers of 16-byte units: a thread keeps the running maxima of
// its unit of columns; when a row has fewer than 256 units several row groups share the chunk and meet in LDS.
template <typename T>
__global__ __launch_bounds__(256) void column_max_partial_vec_kernel(const T *__restrict__ a, float *__restrict__ partial,
                                                                     int64_t N, int HS) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  constexpr int UE = 16 / sizeof(T);
  __shared__ float red[256 * UE];
  const int g = blockIdx.x, b = blockIdx.y, t = threadIdx.x;
  const int64_t n0 = (int64_t)g * kChunkRows;
  const int rows = (int)min((int64_t)kChunkRows, N - n0);
  const T *src = a + ((int64_t)b * N + n0) * HS;
  const int units = HS / UE;
  const int upb = units < 256 ? units : 256;  // units per pass
  const int groups = 256 / upb;               // row groups per pass
  const int rg = t / upb, u_in = t - rg * upb;
  float *dst = partial + ((int64_t)g * gridDim.y + b) * HS;
  for (int u0 = 0; u0 < units; u0 += upb) {
    const int u = u0 + u_in;
    float m[UE];
#pragma unroll
    for (int j = 0; j < UE; ++j) m[j] = -INFINITY;
    if (rg < groups && u < units) {
      for (int r = rg; r < rows; r += groups) {
        const u32x4 raw = *reinterpret_cast<const u32x4 *>(src + (int64_t)r * HS + u * UE);
        const T *e = reinterpret_cast<const T *>(&raw);
#pragma unroll
        for (int j = 0; j < UE; ++j) m[j] = fmaxf(m[j], load_as_f32(e + j));
      }
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < UE; ++j) red[t * UE + j] = m[j];
    __syncthreads();
    // column c of this pass: the maximum over the row groups
    for (int c = t; c < upb * UE && u0 * UE + c < HS; c += 256) {
      float v = -INFINITY;
      for (int q = 0; q < groups; ++q) v = fmaxf(v, red[(q * upb) * UE + c]);
      dst[u0 * UE + c] = v;
    }
  }
}

// grid (ceil(B*H*S / 16)): maximum over the G partials; 16 outputs x 16 interleaved slices of the partials per
// workgroup, the slices meet in LDS.
__global__ __launch_bounds__(256) void column_max_combine_kernel(const float *__restrict__ partial, int G, int64_t BHS,
                                                                 float *__restrict__ colmax) {
  __shared__ float red[16][17];
  const int oc = threadIdx.x & 15, q = threadIdx.x >> 4;
  const int64_t o = (int64_t)blockIdx.x * 16 + oc;
  float m = -INFINITY;
  if (o < BHS)
    for (int g = q; g < G; g += 16) m = fmaxf(m, partial[(int64_t)g * BHS + o]);
  red[q][oc] = m;
  __syncthreads();
  if (q == 0 && o < BHS) {
#pragma unroll
    for (int k = 1; k < 16; ++k) m = fmaxf(m, red[k][oc]);
    colmax[o] = m;
  }
}

// wc[b,n,c] = exp(A[b,n,c] - m[b,c]), c = h*S + s; element-wise over (B*N, H*S).
template <typename T>
__global__ __launch_bounds__(256) void column_weights_kernel(const T *__restrict__ a, const float *__restrict__ colmax,
                                                             T *__restrict__ wc, int64_t N, int HS, int64_t total) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t row = i / HS;
    const int c = (int)(i - row * HS);
    const int64_t b = row / N;
    store_from_f32(wc + i, expf(load_as_f32(a + i) - colmax[b * HS + c]));
  }
}

// The same with 16-byte accesses (H*S a multiple of the 16-byte unit).
template <typename T>
__global__ __launch_bounds__(256) void column_weights_vec_kernel(const T *__restrict__ a,
                                                                 const float *__restrict__ colmax, T *__restrict__ wc,
                                                                 int64_t N, int HS, int64_t total_units) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  constexpr int UE = 16 / sizeof(T);
  const int units = HS / UE;
  const bool narrow = total_units < (int64_t)1 << 32;  // 64-bit divisions cost more than the exponentials
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total_units; i += (int64_t)gridDim.x * 256) {
    int64_t row, b;
    if (narrow) {
      const uint32_t r32 = (uint32_t)i / (uint32_t)units;
      row = r32;
      b = N < ((int64_t)1 << 32) ? (int64_t)(r32 / (uint32_t)N) : 0;
    } else {
      row = i / units;
      b = row / N;
    }
    const int c = (int)(i - row * units) * UE;
    const u32x4 raw = *reinterpret_cast<const u32x4 *>(a + i * UE);
    const T *e = reinterpret_cast<const T *>(&raw);
    float cm[UE];  // the unit's column maxima with 16-byte loads (c is a multiple of UE, UE a multiple of 4)
#pragma unroll
    for (int j = 0; j < UE; j += 4) {
      const float4 q = *reinterpret_cast<const float4 *>(colmax + b * HS + c + j);
      cm[j] = q.x, cm[j + 1] = q.y, cm[j + 2] = q.z, cm[j + 3] = q.w;
    }
    alignas(16) T o[UE];
#pragma unroll
    for (int j = 0; j < UE; ++j) store_from_f32(o + j, expf(load_as_f32(e + j) - cm[j]));
    *reinterpret_cast<u32x4 *>(wc + i * UE) = *reinterpret_cast<const u32x4 *>(o);
  }
}

// In-place softmax over the S entries of every (point, head) row; L lanes share a row (L a power of two <= 64).
// temperature != nullptr: the entries are divided by clamp(temperature[head], 0.5, 5) first (row = point * H + head),
// which makes this the softmax of the PhysicsAttention slice weights (PA.py:172-181).
template <typename T, int L>
__global__ __launch_bounds__(256) void softmax_rows_kernel(T *__restrict__ a, int64_t rows, int S,
                                                           const float *__restrict__ temperature, int H) {
  const int per_wg = 256 / L;
  const int sub = threadIdx.x / L, l = threadIdx.x % L;
  for (int64_t row = (int64_t)blockIdx.x * per_wg + sub; row < rows; row += (int64_t)gridDim.x * per_wg) {
    T *p = a + row * S;
    const float inv_t = temperature ? 1.f / clamp_temperature(temperature[row % H]) : 1.f;
    float mx = -INFINITY;
    for (int s = l; s < S; s += L) mx = fmaxf(mx, load_as_f32(p + s) * inv_t);
#pragma unroll
    for (int off = L >> 1; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
    float sum = 0.f;
    for (int s = l; s < S; s += L) sum += expf(load_as_f32(p + s) * inv_t - mx);
#pragma unroll
    for (int off = L >> 1; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
    const float inv = 1.f / sum;
    for (int s = l; s < S; s += L) store_from_f32(p + s, expf(load_as_f32(p + s) * inv_t - mx) * inv);
  }
}

// The same with 16-byte accesses, for rows that are a whole number of 16-byte units (S a multiple of 8 in bf16, of 4
// in float32): LR lanes share a row (a power of two >= S / unit), a lane keeps its unit in registers between the load
// and the store, so every element is read once, exponentiated once and written once.
template <typename T, int LR>
__global__ __launch_bounds__(256) void softmax_rows_vec_kernel(T *__restrict__ a, int64_t rows, int S,
                                                               const float *__restrict__ temperature, int H) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  constexpr int UE = 16 / sizeof(T);
  constexpr int per_wg = 256 / LR;
  const int sub = threadIdx.x / LR, l = threadIdx.x % LR;
  const bool mine = l * UE < S;
  for (int64_t row = (int64_t)blockIdx.x * per_wg + sub; row < rows; row += (int64_t)gridDim.x * per_wg) {
    T *p = a + row * S + l * UE;
    const float inv_t = temperature ? 1.f / clamp_temperature(temperature[row % H]) : 1.f;
    float v[UE];
    float mx = -INFINITY;
    if (mine) {
      const u32x4 raw = *reinterpret_cast<const u32x4 *>(p);
      const T *e = reinterpret_cast<const T *>(&raw);
#pragma unroll
      for (int j = 0; j < UE; ++j) {
        v[j] = load_as_f32(e + j) * inv_t;
        mx = fmaxf(mx, v[j]);
      }
    }
#pragma unroll
    for (int off = LR >> 1; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
    float sum = 0.f;
    if (mine) {
#pragma unroll
      for (int j = 0; j < UE; ++j) {
        v[j] = expf(v[j] - mx);
        sum += v[j];
      }
    }
#pragma unroll
    for (int off = LR >> 1; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
    if (mine) {
      const float inv = 1.f / sum;
      alignas(16) T o[UE];
#pragma unroll
      for (int j = 0; j < UE; ++j) store_from_f32(o + j, v[j] * inv);
      *reinterpret_cast<u32x4 *>(p) = *reinterpret_cast<const u32x4 *>(o);
    }
  }
}

// ------------------------------------------------------------------------------------------------
// flare_backward_kernel: per-point part of the FLARE backward pass.  grid (row tiles of R points per batch, H).
// With wr = softmax_s(A) (hand-back weights), wc = exp(A - max_n A) (gather weights), z the gathered summaries,
// g = d y, and d num / d den the gradients of the un-normalised gather sums (z = num / den):
//   d wr[n,s] = g[n,:] . z[s,:];        d A += wr (d wr - sum_s wr d wr)          (row softmax backward)
//   d wc[n,s] = v[n,:] . d num[s,:] + d den[s];   d A += wc d wc                   (the column shift max_n A has no
//                                                                                  gradient: z does not depend on it)
//   d v[n,:]  = sum_s wc[n,s] d num[s,:]
// LDS: the head's tables z, d num (row stride D+1), d den; the tile's rows of v, g (row stride D+1) and wr, wc, d wr,
// wc d wc (row stride S+1).  R is a power of two <= 32; 256 / R threads share a row in the row reduction.
// ------------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void flare_backward_kernel(
    const T *__restrict__ wr, const T *__restrict__ wc, const T *__restrict__ v, const T *__restrict__ g,
    const float *__restrict__ z, const float *__restrict__ d_num, const float *__restrict__ d_den,
    T *__restrict__ d_a, T *__restrict__ d_v, int64_t N, int H, int D, int S, int R, int tiles_per_batch) {
  extern __shared__ float lds[];
  const int D1 = D + 1, S1 = S + 1;
  float *zt = lds;               // S * D1
  float *dn = zt + S * D1;       // S * D1
  float *dd = dn + S * D1;       // S
  float *vl = dd + S;            // R * D1
  float *gl = vl + R * D1;       // R * D1
  float *wrl = gl + R * D1;      // R * S1
  float *wcl = wrl + R * S1;     // R * S1
  float *dwl = wcl + R * S1;     // R * S1: d wr, then d A
  float *dcl = dwl + R * S1;     // R * S1: wc d wc
  const int t = threadIdx.x;
  const int h = blockIdx.y;
  const int b = blockIdx.x / tiles_per_batch;
  const int64_t n0 = (int64_t)(blockIdx.x % tiles_per_batch) * R;
  const int rows = (int)min((int64_t)R, N - n0);
  const int64_t m0 = (int64_t)b * N + n0;
  const int HD = H * D, HS = H * S;
  const int64_t bh = (int64_t)b * H + h;
  for (int i = t; i < S * D; i += 256) {
    const int s = i / D, d = i - s * D;
    zt[s * D1 + d] = z[bh * S * D + i];
    dn[s * D1 + d] = d_num[bh * S * D + i];
  }
  for (int i = t; i < S; i += 256) dd[i] = d_den[bh * S + i];
  for (int i = t; i < R * D; i += 256) {
    const int r = i / D, d = i - r * D;
    const bool ok = r < rows;
    const int64_t off = (m0 + r) * HD + h * D + d;
    vl[r * D1 + d] = ok ? load_as_f32(v + off) : 0.f;
    gl[r * D1 + d] = ok ? load_as_f32(g + off) : 0.f;
  }
  for (int i = t; i < R * S; i += 256) {
    const int r = i / S, s = i - r * S;
    const bool ok = r < rows;
    const int64_t off = (m0 + r) * HS + h * S + s;
    wrl[r * S1 + s] = ok ? load_as_f32(wr + off) : 0.f;
    wcl[r * S1 + s] = ok ? load_as_f32(wc + off) : 0.f;
  }
  __syncthreads();
  for (int i = t; i < R * S; i += 256) {
    const int r = i / S, s = i - r * S;
    const float *vr = vl + r * D1, *gr = gl + r * D1, *zr = zt + s * D1, *nr = dn + s * D1;
    float dwr = 0.f, dwc = dd[s];
    for (int d = 0; d < D; ++d) {
      dwr = fmaf(gr[d], zr[d], dwr);
      dwc = fmaf(vr[d], nr[d], dwc);
    }
    dwl[r * S1 + s] = dwr;
    dcl[r * S1 + s] = wcl[r * S1 + s] * dwc;
  }
  __syncthreads();
  const int tpr = 256 / R;
  const int r_own = t / tpr, j_own = t - r_own * tpr;
  float dot = 0.f;
  for (int s = j_own; s < S; s += tpr) dot = fmaf(wrl[r_own * S1 + s], dwl[r_own * S1 + s], dot);
  for (int off = tpr >> 1; off > 0; off >>= 1) dot += __shfl_xor(dot, off, 64);
  for (int s = j_own; s < S; s += tpr)
    dwl[r_own * S1 + s] = wrl[r_own * S1 + s] * (dwl[r_own * S1 + s] - dot) + dcl[r_own * S1 + s];
  __syncthreads();
  for (int i = t; i < rows * S; i += 256) {
    const int r = i / S, s = i - r * S;
    store_from_f32(d_a + (m0 + r) * HS + h * S + s, dwl[r * S1 + s]);
  }
  for (int i = t; i < rows * D; i += 256) {
    const int r = i / D, d = i - r * D;
    const float *wcr = wcl + r * S1;
    float acc = 0.f;
    for (int s = 0; s < S; ++s) acc = fmaf(wcr[s], dn[s * D1 + d], acc);
    store_from_f32(d_v + (m0 + r) * HD + h * D + d, acc);
  }
}

int64_t column_max_chunks(const pa_shape &s) { return (s.N + kChunkRows - 1) / kChunkRows; }

int backward_tile_rows(const pa_shape &s) {
  const size_t fixed = (size_t)(2 * s.S * (s.D + 1) + s.S) * 4;
  for (int R = 32; R >= 4; R >>= 1) {
    const size_t per = (size_t)R * (2 * (s.D + 1) + 4 * (s.S + 1)) * 4;
    if (fixed + per <= 120 * 1024) return R;
  }
  return 0;
}

template <typename T>
static int backward_points_t(const pa_shape &s, const void *wr, const void *wc, const void *v, const void *g,
                             const float *z, const float *d_num, const float *d_den, void *d_a, void *d_v,
                             hipStream_t st) {
  const int R = backward_tile_rows(s);
  if (R == 0) return PA_ERR_UNSUPPORTED;
  const size_t lds = (size_t)(2 * s.S * (s.D + 1) + s.S + (size_t)R * (2 * (s.D + 1) + 4 * (s.S + 1))) * 4;
  int rc = allow_dynamic_lds(flare_backward_kernel<T>, lds);
  if (rc) return rc;
  const int tiles = (int)((s.N + R - 1) / R);
  hipLaunchKernelGGL((flare_backward_kernel<T>), dim3((unsigned)(tiles * s.B), (unsigned)s.H), dim3(256), lds, st,
                     static_cast<const T *>(wr), static_cast<const T *>(wc), static_cast<const T *>(v),
                     static_cast<const T *>(g), z, d_num, d_den, static_cast<T *>(d_a), static_cast<T *>(d_v), s.N,
                     (int)s.H, (int)s.D, (int)s.S, R, tiles);
  return launch_status();
}

int backward_points(int dtype, const pa_shape &s, const void *wr, const void *wc, const void *v, const void *g,
                    const float *z, const float *d_num, const float *d_den, void *d_a, void *d_v, hipStream_t st) {
  return dtype == PA_F32 ? backward_points_t<float>(s, wr, wc, v, g, z, d_num, d_den, d_a, d_v, st)
                         : backward_points_t<bf16>(s, wr, wc, v, g, z, d_num, d_den, d_a, d_v, st);
}

// ------------------------------------------------------------------------------------------------
// pack_weights_kernel: both normalisations of the scores in the packed operand layout of the bf16 MFMA slice kernels
// (what their own softmax kernel writes: wave = head, lanes <-> the tile's points, registers <-> slices), read from
// the natural-layout scores with 8-byte loads:
//   wc_pack = exp(A - max_n A)    gather weights   -> slice_reduce_kernel with the packed values gives num | den
//   wr_pack = softmax_s(A)        hand-back weights -> deslice_natural_kernel with the packed summaries gives y
// grid (G, B, head groups), one wave per head of the group; rows beyond N get zero weights.
// ------------------------------------------------------------------------------------------------
template <int S>
__global__ __launch_bounds__(512) void pack_weights_kernel(const uint16_t *__restrict__ scores,
                                                           const float *__restrict__ colmax,
                                                           mfma::u32x4 *__restrict__ wc_pack,
                                                           mfma::u32x4 *__restrict__ wr_pack, int64_t N, int tpb, int H) {
  using mfma::f32x16;
  using mfma::rowmap;
  constexpr int ST = (S + 31) / 32, NCH = S / 16;
  const int tid = threadIdx.x, lane = tid & 63, i = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int h = blockIdx.z * (blockDim.x >> 6) + wave;
  const int b = blockIdx.y;
  const int HS = H * S;
  float cm[ST][16];
#pragma unroll
  for (int st = 0; st < ST; ++st)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int sl = 32 * st + rowmap(r, g);
      cm[st][r] = sl < S ? colmax[((int64_t)b * H + h) * S + sl] : 0.f;
    }
  for (int t = blockIdx.x; t < tpb; t += gridDim.x) {
    const int64_t n = (int64_t)t * 32 + i;
    const bool valid = n < N;
    const uint16_t *srow = scores + ((int64_t)b * N + (valid ? n : N - 1)) * HS + h * S;
    f32x16 a[ST];
#pragma unroll
    for (int st = 0; st < ST; ++st)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int s0 = 32 * st + 8 * q + 4 * g;  // slices rowmap(4 q .. 4 q + 3, g)
        if (s0 < S) {
          const uint2 raw = *reinterpret_cast<const uint2 *>(srow + s0);
          a[st][4 * q + 0] = __uint_as_float(raw.x << 16);
          a[st][4 * q + 1] = __uint_as_float(raw.x & 0xffff0000u);
          a[st][4 * q + 2] = __uint_as_float(raw.y << 16);
          a[st][4 * q + 3] = __uint_as_float(raw.y & 0xffff0000u);
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j) a[st][4 * q + j] = -1e30f;  // slices beyond S: weight 0
        }
      }
    const int64_t base = ((((int64_t)b * tpb + t) * H + h) * NCH) * 64 + lane;
    const float keep = valid ? 1.f : 0.f;
    float mx = -INFINITY;
#pragma unroll
    for (int st = 0; st < ST; ++st) {
      f32x16 e;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        e[r] = __builtin_amdgcn_exp2f((a[st][r] - cm[st][r]) * kLog2e);
        mx = fmaxf(mx, a[st][r]);
      }
      if (2 * st < NCH) wc_pack[base + (2 * st) * 64] = mfma::pack_half<0>(e, keep);
      if (2 * st + 1 < NCH) wc_pack[base + (2 * st + 1) * 64] = mfma::pack_half<1>(e, keep);
    }
    mx = mfma::half_max(mx);
    float sum = 0.f;
#pragma unroll
    for (int st = 0; st < ST; ++st)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        a[st][r] = __builtin_amdgcn_exp2f((a[st][r] - mx) * kLog2e);
        sum += a[st][r];
      }
    sum = mfma::half_sum(sum);
    const float inv = valid ? __builtin_amdgcn_rcpf(sum) : 0.f;
#pragma unroll
    for (int cq = 0; cq < NCH; ++cq)
      wr_pack[base + cq * 64] = (cq & 1) ? mfma::pack_half<1>(a[cq >> 1], inv) : mfma::pack_half<0>(a[cq >> 1], inv);
  }
}

int pack_weights(const pa_shape &s, const void *scores, const float *colmax, void *wc_pack, void *wr_pack, int num_cu,
                 hipStream_t st) {
  const int waves = (int)(s.H < 8 ? s.H : 8);
  if (s.H % waves != 0 || s.S % 16 != 0) return PA_ERR_UNSUPPORTED;
  const int groups = (int)(s.H / waves);
  int64_t gx = (4 * (int64_t)num_cu + s.B * groups - 1) / (s.B * groups);
  const int64_t tpb = (s.N + 31) / 32;
  if (gx > tpb) gx = tpb;
  if (gx < 1) gx = 1;
  const dim3 grid((unsigned)gx, (unsigned)s.B, (unsigned)groups), block((unsigned)(waves * 64));
#define PA_LAUNCH_PW(SS)                                                                                       \
  hipLaunchKernelGGL((pack_weights_kernel<SS>), grid, block, 0, st, static_cast<const uint16_t *>(scores), colmax, \
                     static_cast<mfma::u32x4 *>(wc_pack), static_cast<mfma::u32x4 *>(wr_pack), s.N, (int)tpb, (int)s.H)
  switch (s.S) {
    case 16: PA_LAUNCH_PW(16); break;
    case 32: PA_LAUNCH_PW(32); break;
    case 64: PA_LAUNCH_PW(64); break;
    case 128: PA_LAUNCH_PW(128); break;
    default: return PA_ERR_UNSUPPORTED;
  }
#undef PA_LAUNCH_PW
  return launch_status();
}

// z[b,h,s,:] = num / den from the (D + 1)-wide sums of the aggregation (den = the count column)
__global__ __launch_bounds__(256) void normalise_kernel(const float *__restrict__ sums, float *__restrict__ z,
                                                        int64_t total, int D) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const int64_t row = idx / D;
  const int d = (int)(idx - row * D);
  z[idx] = sums[row * (D + 1) + d] / sums[row * (D + 1) + D];
}

int normalise(const pa_shape &s, const float *sums, float *z, hipStream_t st) {
  const int64_t total = s.B * s.H * s.S * s.D;
  hipLaunchKernelGGL(normalise_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, sums, z, total,
                     (int)s.D);
  return launch_status();
}

template <typename T>
static int column_max_t(const pa_shape &s, const void *a, float *partial, float *colmax, hipStream_t st) {
  const int HS = (int)(s.H * s.S);
  const int64_t G = column_max_chunks(s), BHS = s.B * HS;
  constexpr int UE = 16 / sizeof(T);
  if (HS % UE == 0 && reinterpret_cast<uintptr_t>(a) % 16 == 0)
    hipLaunchKernelGGL((column_max_partial_vec_kernel<T>), dim3((unsigned)G, (unsigned)s.B), dim3(256), 0, st,
                       static_cast<const T *>(a), partial, s.N, HS);
  else
    hipLaunchKernelGGL((column_max_partial_kernel<T>), dim3((unsigned)G, (unsigned)s.B), dim3(256), 0, st,
                       static_cast<const T *>(a), partial, s.N, HS);
  int rc = launch_status();
  if (rc) return rc;
  hipLaunchKernelGGL(column_max_combine_kernel, dim3((unsigned)((BHS + 15) / 16)), dim3(256), 0, st, partial, (int)G,
                     BHS, colmax);
  return launch_status();
}

int column_max(int dtype, const pa_shape &s, const void *a, float *partial, float *colmax, hipStream_t st) {
  return dtype == PA_F32 ? column_max_t<float>(s, a, partial, colmax, st) : column_max_t<bf16>(s, a, partial, colmax, st);
}

template <typename T>
static int column_weights_t(const pa_shape &s, const void *a, float *partial, float *colmax, void *wc, hipStream_t st) {
  const int HS = (int)(s.H * s.S);
  const int64_t G = column_max_chunks(s), BHS = s.B * HS, total = s.B * s.N * HS;
  constexpr int UE = 16 / sizeof(T);
  const bool vec = HS % UE == 0 && (reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(wc) |
                                    reinterpret_cast<uintptr_t>(colmax)) % 16 == 0;
  if (vec)
    hipLaunchKernelGGL((column_max_partial_vec_kernel<T>), dim3((unsigned)G, (unsigned)s.B), dim3(256), 0, st,
                       static_cast<const T *>(a), partial, s.N, HS);
  else
    hipLaunchKernelGGL((column_max_partial_kernel<T>), dim3((unsigned)G, (unsigned)s.B), dim3(256), 0, st,
                       static_cast<const T *>(a), partial, s.N, HS);
  int rc = launch_status();
  if (rc) return rc;
  hipLaunchKernelGGL(column_max_combine_kernel, dim3((unsigned)((BHS + 15) / 16)), dim3(256), 0, st, partial, (int)G,
                     BHS, colmax);
  rc = launch_status();
  if (rc) return rc;
  if (vec) {
    const int64_t total_units = total / UE;
    int64_t blocks = (total_units + 255) / 256;
    if (blocks > 16384) blocks = 16384;
    hipLaunchKernelGGL((column_weights_vec_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, st,
                       static_cast<const T *>(a), colmax, static_cast<T *>(wc), s.N, HS, total_units);
    return launch_status();
  }
  int64_t blocks = (total + 255) / 256;
  if (blocks > 8192) blocks = 8192;
  hipLaunchKernelGGL((column_weights_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, st, static_cast<const T *>(a),
                     colmax, static_cast<T *>(wc), s.N, HS, total);
  return launch_status();
}

int column_weights(int dtype, const pa_shape &s, const void *a, float *partial, float *colmax, void *wc,
                   hipStream_t st) {
  return dtype == PA_F32 ? column_weights_t<float>(s, a, partial, colmax, wc, st)
                         : column_weights_t<bf16>(s, a, partial, colmax, wc, st);
}

template <typename T, int L>
static int softmax_rows_l(const pa_shape &s, void *a, const float *temperature, hipStream_t st) {
  const int64_t rows = s.B * s.N * s.H;
  int64_t blocks = (rows + (256 / L) - 1) / (256 / L);
  if (blocks > 16384) blocks = 16384;
  hipLaunchKernelGGL((softmax_rows_kernel<T, L>), dim3((unsigned)blocks), dim3(256), 0, st, static_cast<T *>(a), rows,
                     (int)s.S, temperature, (int)s.H);
  return launch_status();
}

template <typename T, int LR>
static int softmax_rows_vec(const pa_shape &s, void *a, const float *temperature, hipStream_t st) {
  const int64_t rows = s.B * s.N * s.H;
  int64_t blocks = (rows + (256 / LR) - 1) / (256 / LR);
  if (blocks > 16384) blocks = 16384;
  hipLaunchKernelGGL((softmax_rows_vec_kernel<T, LR>), dim3((unsigned)blocks), dim3(256), 0, st, static_cast<T *>(a),
                     rows, (int)s.S, temperature, (int)s.H);
  return launch_status();
}

template <typename T>
static int softmax_rows_t(const pa_shape &s, void *a, const float *temperature, hipStream_t st) {
  constexpr int UE = 16 / sizeof(T);
  if (s.S % UE == 0 && s.S / UE <= 64 && reinterpret_cast<uintptr_t>(a) % 16 == 0) {
    const int64_t units = s.S / UE;
    if (units <= 1) return softmax_rows_vec<T, 1>(s, a, temperature, st);
    if (units <= 2) return softmax_rows_vec<T, 2>(s, a, temperature, st);
    if (units <= 4) return softmax_rows_vec<T, 4>(s, a, temperature, st);
    if (units <= 8) return softmax_rows_vec<T, 8>(s, a, temperature, st);
    if (units <= 16) return softmax_rows_vec<T, 16>(s, a, temperature, st);
    if (units <= 32) return softmax_rows_vec<T, 32>(s, a, temperature, st);
    return softmax_rows_vec<T, 64>(s, a, temperature, st);
  }
  if (s.S <= 8) return softmax_rows_l<T, 8>(s, a, temperature, st);
  if (s.S <= 16) return softmax_rows_l<T, 16>(s, a, temperature, st);
  if (s.S <= 32) return softmax_rows_l<T, 32>(s, a, temperature, st);
  return softmax_rows_l<T, 64>(s, a, temperature, st);
}

int softmax_rows(int dtype, const pa_shape &s, void *a, const float *temperature, hipStream_t st) {
  return dtype == PA_F32 ? softmax_rows_t<float>(s, a, temperature, st) : softmax_rows_t<bf16>(s, a, temperature, st);
}

}  // namespace flare
}  // namespace pa
