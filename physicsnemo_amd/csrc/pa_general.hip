// General PhysicsAttention kernels: any (C, H, D, S) within the library limits, fp32 or bf16 storage,
// fp32 arithmetic on the vector ALUs, natural tensor layouts.  They serve fp32 runs (rtol 1e-4 class),
// the structured-2D (Conv2d) projections and every shape the MFMA kernels do not cover.
//
// Stage map (reference lines in include/physattn.h):
//   rows_gemm_kernel          in_project_x / in_project_fx (Linear or k x k Conv2d as implicit GEMM), out_linear
//   rows GEMM + softmax_rows  in_project_slice, then clamp(temperature) + softmax over S in place (pa_flare.hip)
//   slice_partial_kernel      per-chunk sums  sum_n w[n,s] * [fx_mid[n,:], 1]
//   slice_combine_attn_kernel fixed-order combine, / (norm + 1e-2), qkv, softmax(q k^T / sqrt D) v   (LDS resident)
//   deslice_kernel            out_x[n,h,:] = sum_s w[n,h,s] * tok'[h,s,:]
//   residual_ln_kernel        fx_new = y + residual; ln_out = LayerNorm(fx_new)
#include "pa_common.h"
#include "pa_host.h"

namespace pa {
namespace general {

// ------------------------------------------------------------------------------------------------
// rows_gemm_kernel: out[m, o] = bias[o] + sum_k A(m, k) * W[o, k]
//   linear: A(m, k) = in[m*K + k]
//   conv  : K = taps*C, k = tap*C + c; 2-D: taps = ks^2, tap = u*ks + v, A(m,k) = in[b, (i+u-p)*gw + (j+v-p), c];
//           3-D: taps = ks^3, tap = (u*ks + v)*ks + z, A(m,k) = in[b, ((i+u-p)*gw + (j+v-p))*gd + (l+z-p), c];
//           0 outside the grid; the PyTorch weight element is W[o, c, u, v(, z)] = W[o*K + c*taps + tap].
// 64x64 output tile per 256-thread workgroup, 4x4 outputs per thread, K staged 16 at a time through LDS.
// blockIdx.z selects one of two (W, bias, out) sets that share the same input (x_mid and fx_mid).
// ------------------------------------------------------------------------------------------------
// four consecutive elements with one 8- or 16-byte access
template <typename T>
__device__ __forceinline__ void load4(const T *p, float (&v)[4]) {
  if constexpr (sizeof(T) == 2) {
    const uint2 r = *reinterpret_cast<const uint2 *>(p);
    const T *e = reinterpret_cast<const T *>(&r);
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = load_as_f32(e + j);
  } else {
    const float4 r = *reinterpret_cast<const float4 *>(p);
    v[0] = r.x, v[1] = r.y, v[2] = r.z, v[3] = r.w;
  }
}
template <typename T>
__device__ __forceinline__ void store4(T *p, const float (&v)[4]) {
  if constexpr (sizeof(T) == 2) {
    alignas(8) T o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) store_from_f32(o + j, v[j]);
    *reinterpret_cast<uint2 *>(p) = *reinterpret_cast<const uint2 *>(o);
  } else {
    *reinterpret_cast<float4 *>(p) = float4{v[0], v[1], v[2], v[3]};
  }
}

template <typename TA, typename TW>
__global__ __launch_bounds__(256) void rows_gemm_kernel(GemmArgs a) {
  __shared__ float As[16][64 + 4];
  __shared__ float Ws[16][64 + 4];
  const int z = blockIdx.z;
  const TA *in = static_cast<const TA *>(a.in);
  const TW *W = static_cast<const TW *>(a.w[z]);
  const float *bias = a.bias[z];
  TA *out = static_cast<TA *>(a.out[z]);
  const int t = threadIdx.x;
  const int tx = t & 15, ty = t >> 4;
  const int64_t m0 = (int64_t)blockIdx.x * 64;
  const int o0 = blockIdx.y * 64;
  const int lr = t >> 2;         // tile row / tile out column this thread stages
  const int lk = (t & 3) * 4;    // first of 4 consecutive k it stages
  const int pad = a.ks / 2;
  const int gd = a.gd > 0 ? a.gd : 1;          // a 2-D grid is a 3-D grid of depth 1 with a single depth tap
  const int ksd = a.gd > 0 ? a.ks : 1;
  const int taps = a.ks * a.ks * ksd;

  // decode the staged row once
  const int64_t m_ld = m0 + lr;
  const bool m_ok = m_ld < a.M;
  int64_t b_ld = 0;
  int i_ld = 0, j_ld = 0, l_ld = 0;
  if (a.ks > 0 && m_ok) {
    b_ld = m_ld / a.N;
    int n = (int)(m_ld - b_ld * a.N);
    l_ld = n % gd;
    n /= gd;
    i_ld = n / a.gw;
    j_ld = n - i_ld * a.gw;
  }
  const int o_ld = o0 + lr;

  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  // a Linear whose rows are whole numbers of four elements is staged with 8- / 16-byte loads
  const bool vec = a.ks == 0 && a.K % 4 == 0 && reinterpret_cast<uintptr_t>(in) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(W) % 16 == 0;
  const bool vec_out = a.O % 4 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
  for (int k0 = 0; k0 < a.K; k0 += 16) {
    if (vec) {
      float av4[4] = {0.f, 0.f, 0.f, 0.f}, wv4[4] = {0.f, 0.f, 0.f, 0.f};
      if (k0 + lk < a.K) {
        if (m_ok) load4(in + m_ld * a.K + k0 + lk, av4);
        if (o_ld < a.O) load4(W + (int64_t)o_ld * a.K + k0 + lk, wv4);
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        As[lk + q][lr] = av4[q];
        Ws[lk + q][lr] = wv4[q];
      }
    } else
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int k = k0 + lk + q;
      float av = 0.f, wv = 0.f;
      if (k < a.K) {
        if (a.ks == 0) {
          if (m_ok) av = load_as_f32(in + m_ld * a.K + k);
          if (o_ld < a.O) wv = load_as_f32(W + (int64_t)o_ld * a.K + k);
        } else {
          const int tap = k / a.C, c = k - tap * a.C;
          const int uv = tap / ksd, z = tap - uv * ksd;
          const int u = uv / a.ks, v = uv - u * a.ks;
          const int ii = i_ld + u - pad, jj = j_ld + v - pad, ll = l_ld + (a.gd > 0 ? z - pad : 0);
          if (m_ok && ii >= 0 && ii < a.gh && jj >= 0 && jj < a.gw && ll >= 0 && ll < gd)
            av = load_as_f32(in + ((b_ld * a.N + ((int64_t)ii * a.gw + jj) * gd + ll) * a.C + c));
          if (o_ld < a.O)
            wv = load_as_f32(W + (int64_t)o_ld * a.K + (a.w_tap_major ? (int64_t)k : (int64_t)c * taps + tap));
        }
      }
      As[lk + q][lr] = av;
      Ws[lk + q][lr] = wv;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 16; ++kk) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) wv[j] = Ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t m = m0 + ty * 4 + i;
    if (m >= a.M) continue;
    if (vec_out && o0 + tx * 4 < a.O) {
      float v4[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float v = acc[i][j] + (bias ? bias[o0 + tx * 4 + j] : 0.f);
        v4[j] = a.act == 1 ? gelu_erf(v) : v;
      }
      store4(out + m * a.O + o0 + tx * 4, v4);
      continue;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int o = o0 + tx * 4 + j;
      if (o < a.O) {
        const float v = acc[i][j] + (bias ? bias[o] : 0.f);
        store_from_f32(out + m * a.O + o, a.act == 1 ? gelu_erf(v) : v);
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------
// slice_softmax_plus_kernel: the Transolver++ form of slice_softmax_kernel (PA.py:166-170, gumbel_softmax.py:49-57).
//   temp[r,h]  = max(temperature[h] + gelu(b2 + sum_s w2[s] gelu(b1[s] + x_mid[r,h,:] . w1[s,:])), 0.01)
//   w[r,h,:]   = softmax_s((logits[r,h,s] - log(-log(u[r,h,s] + 1e-8) + 1e-8)) / temp[r,h])
// `uniform` holds the caller's U[0,1) samples in the activation type (what torch.rand_like(logits) draws).
// ------------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void slice_softmax_plus_kernel(
    const T *__restrict__ x_mid, const T *__restrict__ uniform, const float *__restrict__ w_slice,
    const float *__restrict__ b_slice, const float *__restrict__ temperature, const float *__restrict__ pt_w1,
    const float *__restrict__ pt_b1, const float *__restrict__ pt_w2, const float *__restrict__ pt_b2,
    T *__restrict__ w_out, int64_t M, int H, int D, int S, int R) {
  extern __shared__ float lds[];
  float *xs = lds;                       // R * H * (D+1)
  float *wsl = xs + R * H * (D + 1);     // S * D
  float *bsl = wsl + S * D;              // S
  float *w1 = bsl + S;                   // S * D
  float *b1 = w1 + S * D;                // S
  float *w2 = b1 + S;                    // S
  float *lg = w2 + S;                    // R * H * (S+1)
  const int t = threadIdx.x;
  const int64_t m0 = (int64_t)blockIdx.x * R;
  const int rows = (int)min((int64_t)R, M - m0);
  const int HD = H * D, HS = H * S;
  for (int i = t; i < rows * HD; i += 256) {
    const int r = i / HD, c = i - r * HD;
    const int h = c / D, d = c - h * D;
    xs[(r * H + h) * (D + 1) + d] = load_as_f32(x_mid + (m0 + r) * HD + c);
  }
  for (int i = t; i < S * D; i += 256) {
    wsl[i] = w_slice[i];
    w1[i] = pt_w1[i];
  }
  for (int i = t; i < S; i += 256) {
    bsl[i] = b_slice[i];
    b1[i] = pt_b1[i];
    w2[i] = pt_w2[i];
  }
  for (int i = t; i < rows * HS; i += 256) {
    const int pair = i / S, s = i - pair * S;
    lg[pair * (S + 1) + s] = load_as_f32(uniform + m0 * HS + i);
  }
  __syncthreads();
  for (int pair = t; pair < rows * H; pair += 256) {
    const int h = pair % H;
    const float *xr = xs + pair * (D + 1);
    float *lrow = lg + pair * (S + 1);
    float tacc = pt_b2[0];
    for (int s = 0; s < S; ++s) {
      float acc = b1[s];
      const float *wr = w1 + s * D;
      for (int d = 0; d < D; ++d) acc = fmaf(xr[d], wr[d], acc);
      tacc = fmaf(w2[s], gelu_erf(acc), tacc);
    }
    const float temp = round_to(w_out, fmaxf(temperature[h] + gelu_erf(tacc), 0.01f));
    float mx = -INFINITY;
    for (int s = 0; s < S; ++s) {
      float acc = 0.f;
      const float *wr = wsl + s * D;
      for (int d = 0; d < D; ++d) acc = fmaf(xr[d], wr[d], acc);
      const float noise = -logf(-logf(lrow[s] + 1e-8f) + 1e-8f);
      const float z = (round_to(w_out, acc + bsl[s]) + noise) / temp;
      lrow[s] = z;
      mx = fmaxf(mx, z);
    }
    float sum = 0.f;
    for (int s = 0; s < S; ++s) {
      const float e = expf(lrow[s] - mx);
      lrow[s] = e;
      sum += e;
    }
    const float inv = 1.f / sum;
    for (int s = 0; s < S; ++s) lrow[s] *= inv;
  }
  __syncthreads();
  for (int i = t; i < rows * HS; i += 256) {
    const int pair = i / S, s = i - pair * S;
    store_from_f32(w_out + m0 * HS + i, lg[pair * (S + 1) + s]);
  }
}

// ------------------------------------------------------------------------------------------------
// softmax_rows_plus_kernel: the row stage of the Transolver++ slice weights when the two Linears over the
// (point, head) rows -- the slice logits and the hidden layer gelu(b1 + W1 x_mid) of proj_temperature -- were formed by
// the row GEMM kernels (logits in `w`, hidden in `hidden`, both (rows, S)).  L lanes share a row:
//   temp = max(temperature[h] + gelu(b2 + sum_s w2[s] hidden[s]), 0.01);  w <- softmax_s((w + noise(u)) / temp) in place
// ------------------------------------------------------------------------------------------------
template <typename T, int L>
__global__ __launch_bounds__(256) void softmax_rows_plus_kernel(T *__restrict__ w, const T *__restrict__ hidden,
                                                                const T *__restrict__ uniform,
                                                                const float *__restrict__ temperature,
                                                                const float *__restrict__ pt_w2,
                                                                const float *__restrict__ pt_b2, int64_t rows, int S,
                                                                int H) {
  const int per_wg = 256 / L;
  const int sub = threadIdx.x / L, l = threadIdx.x % L;
  for (int64_t row = (int64_t)blockIdx.x * per_wg + sub; row < rows; row += (int64_t)gridDim.x * per_wg) {
    T *p = w + row * S;
    const T *hp = hidden + row * S, *up = uniform + row * S;
    float tacc = 0.f;
    for (int s = l; s < S; s += L) tacc = fmaf(pt_w2[s], load_as_f32(hp + s), tacc);
#pragma unroll
    for (int off = L >> 1; off > 0; off >>= 1) tacc += __shfl_xor(tacc, off, 64);
    const float temp = round_to(w, fmaxf(temperature[row % H] + gelu_erf(tacc + pt_b2[0]), 0.01f));
    const float inv_t = 1.f / temp;
    auto arg = [&](int s) {
      return (load_as_f32(p + s) - logf(-logf(load_as_f32(up + s) + 1e-8f) + 1e-8f)) * inv_t;
    };
    float mx = -INFINITY;
    for (int s = l; s < S; s += L) mx = fmaxf(mx, arg(s));
#pragma unroll
    for (int off = L >> 1; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
    float sum = 0.f;
    for (int s = l; s < S; s += L) sum += expf(arg(s) - mx);
#pragma unroll
    for (int off = L >> 1; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
    const float inv = 1.f / sum;
    for (int s = l; s < S; s += L) store_from_f32(p + s, expf(arg(s) - mx) * inv);
  }
}

// The same with 16-byte accesses, for rows that are a whole number of 16-byte units: LR lanes share a row (a power of
// two >= S / unit), a lane keeps its unit of softmax arguments in registers, so every element is read once and its
// Gumbel noise (two logarithms) is formed once.
template <typename T, int LR>
__global__ __launch_bounds__(256) void softmax_rows_plus_vec_kernel(T *__restrict__ w, const T *__restrict__ hidden,
                                                                    const T *__restrict__ uniform,
                                                                    const float *__restrict__ temperature,
                                                                    const float *__restrict__ pt_w2,
                                                                    const float *__restrict__ pt_b2, int64_t rows, int S,
                                                                    int H) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  constexpr int UE = 16 / sizeof(T);
  constexpr int per_wg = 256 / LR;
  const int sub = threadIdx.x / LR, l = threadIdx.x % LR;
  const bool mine = l * UE < S;
  float w2[UE];
#pragma unroll
  for (int j = 0; j < UE; ++j) w2[j] = mine ? pt_w2[l * UE + j] : 0.f;
  const float b2 = pt_b2[0];
  for (int64_t row = (int64_t)blockIdx.x * per_wg + sub; row < rows; row += (int64_t)gridDim.x * per_wg) {
    const int64_t off0 = row * S + l * UE;
    float v[UE];
    float tacc = 0.f;
    if (mine) {
      const u32x4 rw = *reinterpret_cast<const u32x4 *>(w + off0);
      const u32x4 rh = *reinterpret_cast<const u32x4 *>(hidden + off0);
      const u32x4 ru = *reinterpret_cast<const u32x4 *>(uniform + off0);
      const T *ew = reinterpret_cast<const T *>(&rw), *eh = reinterpret_cast<const T *>(&rh),
              *eu = reinterpret_cast<const T *>(&ru);
#pragma unroll
      for (int j = 0; j < UE; ++j) {
        tacc = fmaf(w2[j], load_as_f32(eh + j), tacc);
        v[j] = load_as_f32(ew + j) - logf(-logf(load_as_f32(eu + j) + 1e-8f) + 1e-8f);
      }
    }
#pragma unroll
    for (int off = LR >> 1; off > 0; off >>= 1) tacc += __shfl_xor(tacc, off, 64);
    const float temp = round_to(w, fmaxf(temperature[row % H] + gelu_erf(tacc + b2), 0.01f));
    const float inv_t = 1.f / temp;
    float mx = -INFINITY;
    if (mine) {
#pragma unroll
      for (int j = 0; j < UE; ++j) {
        v[j] *= inv_t;
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
      *reinterpret_cast<u32x4 *>(w + off0) = *reinterpret_cast<const u32x4 *>(o);
    }
  }
}

// ------------------------------------------------------------------------------------------------
// slice_partial_kernel: grid (G chunks, B*H, output slabs).  For its chunk of points of one (b, h):
//   partial[s, d] = sum_n w[n, s] * fx_mid[n, d]   (d < D),   partial[s, D] = sum_n w[n, s]
// The (S x D+1) output is cut into 4 x 4 register tiles; a thread owns NS of them (tile t + 256 i of its slab of
// 256 NS tiles) and walks the chunk 64 points at a time through LDS: per point and tile two 16-byte LDS reads
// (4 slice weights, 4 features) feed 16 FMAs.  LDS rows are padded to multiples of four (zeros; column D of the
// feature rows holds 1 for the count).  Sums run in a fixed order, so the result is bit-reproducible.
// ------------------------------------------------------------------------------------------------
constexpr int kAttnThreads = 1024;  // slice_combine_attn_kernel: 16 waves, one query row per wave at a time
constexpr int kPartialTile = 64;
constexpr int kPartialMaxNS = 4;

template <typename T, int NS>
__global__ __launch_bounds__(256) void slice_partial_kernel(const T *__restrict__ w, const T *__restrict__ fx_mid,
                                                            float *__restrict__ partials, int B, int64_t N, int H, int D,
                                                            int S, int64_t chunk) {
  extern __shared__ float4 lds4[];
  const int D1 = D + 1, SB = (S + 3) / 4, DB = (D1 + 3) / 4;  // tiles along the slices / the features
  float4 *wl = lds4;                      // kPartialTile * SB
  float4 *fl = wl + kPartialTile * SB;    // kPartialTile * DB
  float *wlf = reinterpret_cast<float *>(wl), *flf = reinterpret_cast<float *>(fl);
  const int t = threadIdx.x;
  const int g = blockIdx.x;
  const int b = blockIdx.y / H, h = blockIdx.y % H;
  const int n_tiles = SB * DB;
  const int slab0 = blockIdx.z * 256 * NS;
  int sb[NS], db[NS];
  float acc[NS][4][4];
#pragma unroll
  for (int i = 0; i < NS; ++i) {
    const int tile = slab0 + t + 256 * i;
    const bool ok = tile < n_tiles;
    sb[i] = ok ? tile % SB : 0;
    db[i] = ok ? tile / SB : 0;
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[i][u][v] = 0.f;
  }
  const int64_t n_begin = (int64_t)g * chunk;
  const int64_t n_end = min(N, n_begin + chunk);
  const int HS = H * S, HD = H * D;
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  constexpr int UE = 16 / sizeof(T);
  const bool vec_w = S % UE == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0;
  const bool vec_f = D % UE == 0 && reinterpret_cast<uintptr_t>(fx_mid) % 16 == 0;
  for (int64_t n0 = n_begin; n0 < n_end; n0 += kPartialTile) {
    const int pts = (int)min((int64_t)kPartialTile, n_end - n0);
    if (vec_w) {  // 16-byte loads: the rows are whole numbers of 16-byte units
      const int units = S / UE;
      for (int i = t; i < kPartialTile * units; i += 256) {
        const int p = i / units, u = i - p * units;
        u32x4 raw = {0u, 0u, 0u, 0u};
        if (p < pts) raw = *reinterpret_cast<const u32x4 *>(w + ((int64_t)b * N + n0 + p) * HS + h * S + u * UE);
        const T *e = reinterpret_cast<const T *>(&raw);
#pragma unroll
        for (int j = 0; j < UE; ++j) wlf[p * (SB * 4) + u * UE + j] = load_as_f32(e + j);
      }
    } else {
      for (int i = t; i < kPartialTile * SB * 4; i += 256) {
        const int p = i / (SB * 4), s = i - p * (SB * 4);
        wlf[i] = (p < pts && s < S) ? load_as_f32(w + ((int64_t)b * N + n0 + p) * HS + h * S + s) : 0.f;
      }
    }
    if (vec_f) {
      const int units = D / UE;
      for (int i = t; i < kPartialTile * units; i += 256) {
        const int p = i / units, u = i - p * units;
        u32x4 raw = {0u, 0u, 0u, 0u};
        if (p < pts) raw = *reinterpret_cast<const u32x4 *>(fx_mid + ((int64_t)b * N + n0 + p) * HD + h * D + u * UE);
        const T *e = reinterpret_cast<const T *>(&raw);
#pragma unroll
        for (int j = 0; j < UE; ++j) flf[p * (DB * 4) + u * UE + j] = load_as_f32(e + j);
      }
      for (int i = t; i < kPartialTile * (DB * 4 - D); i += 256) {  // the count column and the padding behind it
        const int p = i / (DB * 4 - D), d = D + i - p * (DB * 4 - D);
        flf[p * (DB * 4) + d] = (p < pts && d == D) ? 1.f : 0.f;
      }
    } else {
      for (int i = t; i < kPartialTile * DB * 4; i += 256) {
        const int p = i / (DB * 4), d = i - p * (DB * 4);
        float v = 0.f;
        if (p < pts && d < D) v = load_as_f32(fx_mid + ((int64_t)b * N + n0 + p) * HD + h * D + d);
        if (p < pts && d == D) v = 1.f;
        flf[i] = v;
      }
    }
    __syncthreads();
#pragma unroll 2
    for (int p = 0; p < kPartialTile; ++p) {
#pragma unroll
      for (int i = 0; i < NS; ++i) {
        const float4 wv = wl[p * SB + sb[i]];
        const float4 fv = fl[p * DB + db[i]];
        const float ws[4] = {wv.x, wv.y, wv.z, wv.w}, fs[4] = {fv.x, fv.y, fv.z, fv.w};
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
          for (int v = 0; v < 4; ++v) acc[i][u][v] = fmaf(ws[u], fs[v], acc[i][u][v]);
      }
    }
    __syncthreads();
  }
  float *dst = partials + (((int64_t)g * B + b) * H + h) * (S * D1);
#pragma unroll
  for (int i = 0; i < NS; ++i) {
    if (slab0 + t + 256 * i >= n_tiles) continue;
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int s = 4 * sb[i] + u, d = 4 * db[i] + v;
        if (s < S && d < D1) dst[s * D1 + d] = acc[i][u][v];
      }
  }
}

// ------------------------------------------------------------------------------------------------
// combine_partials_kernel: second pass of the reduction, parallel over outputs.  grid (ceil(n_out/64), B*H);
// 64 outputs x 4 quarter-ranges of the G partials per workgroup; each thread adds its quarter in index order,
// the four quarter sums are then added in a fixed order ((q0 + q1) + q2) + q3: bit-reproducible, no atomics.
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void combine_partials_kernel(const float *__restrict__ partials, int G,
                                                               int64_t partial_stride, float *__restrict__ combined,
                                                               int n_out) {
  __shared__ float quarter[4][64];
  const int t = threadIdx.x, q = t >> 6, l = t & 63;
  const int o = blockIdx.x * 64 + l;
  const int bh = blockIdx.y;
  const int per = (G + 3) / 4;
  const int g0 = q * per, g1 = min(G, g0 + per);
  float acc = 0.f;
  if (o < n_out) {
    const float *src = partials + (int64_t)bh * n_out + o;
    for (int g = g0; g < g1; ++g) acc += src[(int64_t)g * partial_stride];
  }
  quarter[q][l] = acc;
  __syncthreads();
  if (q == 0 && o < n_out)
    combined[(int64_t)bh * n_out + o] = ((quarter[0][l] + quarter[1][l]) + quarter[2][l]) + quarter[3][l];
}

// ------------------------------------------------------------------------------------------------
// slice_combine_attn_kernel: one workgroup per (b, h), everything after the load stays in LDS.
//   1. num[s, :], cnt[s] = sum over the G partials in index order
//   2. tok = num / (cnt + 1e-2)            -> slice_token, slice_norm (optional outputs)
//   3. q|k|v = tok Wqkv^T                  (rows of Wqkv: [0,D) q, [D,2D) k, [2D,3D) v)
//   4. out[s, :] = softmax_t(q[s].k[t] / sqrt(D)) v[t, :], one wave per query row
// `partial_stride` = elements between consecutive partials of the same (b, h).  G == 0: `partials` holds
// finished tokens (steps 1-2 skipped); out_token == nullptr: stop after step 2.
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kAttnThreads) void slice_combine_attn_kernel(const float *__restrict__ partials, int G,
                                                                 int64_t partial_stride, const float *__restrict__ w_qkv,
                                                                 float *__restrict__ slice_token,
                                                                 float *__restrict__ slice_norm,
                                                                 float *__restrict__ out_token, int D, int S,
                                                                 int stage_w) {
  extern __shared__ float lds[];
  const int D1 = D + 1;
  float *tok = lds;              // S * D1 (column D holds the count, then the norm)
  float *q = tok + S * D1;       // S * D1
  float *k = q + S * D1;
  float *v = k + S * D1;
  float *prow = v + S * D1;      // one row of S per wave
  float *wq = prow + (kAttnThreads / 64) * S;      // 3D * D1 (only when stage_w)
  const int t = threadIdx.x;
  const int bh = blockIdx.x;
  const int n_out = S * D1;
  if (G > 0) {
    const float *src = partials + (int64_t)bh * n_out;
    for (int o = t; o < n_out; o += kAttnThreads) {
      float acc = 0.f;
      for (int g = 0; g < G; ++g) acc += src[(int64_t)g * partial_stride + o];
      tok[o] = acc;
    }
    __syncthreads();
    for (int s = t; s < S; s += kAttnThreads) tok[s * D1 + D] += kSliceNormEps;
    __syncthreads();
    for (int i = t; i < S * D; i += kAttnThreads) {
      const int s = i / D, d = i - s * D;
      const float val = tok[s * D1 + d] / tok[s * D1 + D];
      tok[s * D1 + d] = val;
      if (slice_token) slice_token[(int64_t)bh * S * D + i] = val;
    }
    if (slice_norm)
      for (int s = t; s < S; s += kAttnThreads) slice_norm[(int64_t)bh * S + s] = tok[s * D1 + D];
  } else {
    // G == 0: `partials` already holds finished slice tokens (B, H, S, D)
    for (int i = t; i < S * D; i += kAttnThreads) tok[(i / D) * D1 + (i % D)] = partials[(int64_t)bh * S * D + i];
  }
  if (!out_token) return;  // reduction-only call (uniform across the workgroup)
  if (stage_w)
    for (int i = t; i < 3 * D * D; i += kAttnThreads) wq[(i / D) * D1 + (i % D)] = w_qkv[i];
  __syncthreads();
  for (int i = t; i < S * 3 * D; i += kAttnThreads) {
    const int s = i / (3 * D), e = i - s * 3 * D;
    const float *wr = stage_w ? wq + e * D1 : w_qkv + (int64_t)e * D;
    const float *tr = tok + s * D1;
    float acc = 0.f;
#pragma unroll 8
    for (int d = 0; d < D; ++d) acc = fmaf(tr[d], wr[d], acc);
    float *dst = e < D ? q : (e < 2 * D ? k : v);
    dst[s * D1 + (e % D)] = acc;
  }
  __syncthreads();
  const int wave = t >> 6, lane = t & 63;
  const float scale = rsqrtf((float)D);
  float *pr = prow + wave * S;
  for (int s = wave; s < S; s += kAttnThreads / 64) {
    const float *qs = q + s * D1;
    float mx = -INFINITY;
    for (int u = lane; u < S; u += 64) {
      const float *ku = k + u * D1;
      float acc = 0.f;
#pragma unroll 8
      for (int e = 0; e < D; ++e) acc = fmaf(qs[e], ku[e], acc);
      acc *= scale;
      pr[u] = acc;
      mx = fmaxf(mx, acc);
    }
    mx = wave_max(mx);
    float sum = 0.f;
    for (int u = lane; u < S; u += 64) {
      const float e = expf(pr[u] - mx);
      pr[u] = e;
      sum += e;
    }
    sum = wave_sum(sum);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    const float inv = 1.f / sum;
    for (int e = lane; e < D; e += 64) {
      float acc = 0.f;
#pragma unroll 8
      for (int u = 0; u < S; ++u) acc = fmaf(pr[u], v[u * D1 + e], acc);
      out_token[((int64_t)bh * S + s) * D + e] = acc * inv;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
}

// ------------------------------------------------------------------------------------------------
// deslice_kernel: grid (row tiles of R, B-independent; H).  out_x[m, h*D + d] = sum_s w[m, h, s] * tok'[b, h, s, d]
// A row tile never straddles two batches (the host picks tiles per batch).
// ------------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void deslice_kernel(const T *__restrict__ w, const float *__restrict__ out_token,
                                                      T *__restrict__ out_x, int64_t N, int H, int D, int S, int R,
                                                      int tiles_per_batch) {
  extern __shared__ float lds[];
  float *tk = lds;            // S * D
  float *wl = tk + S * D;     // R * (S+1)
  const int t = threadIdx.x;
  const int h = blockIdx.y;
  const int b = blockIdx.x / tiles_per_batch;
  const int64_t n0 = (int64_t)(blockIdx.x % tiles_per_batch) * R;
  const int rows = (int)min((int64_t)R, N - n0);
  const int64_t m0 = (int64_t)b * N + n0;
  for (int i = t; i < S * D; i += 256) tk[i] = out_token[((int64_t)b * H + h) * S * D + i];
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
  constexpr int UE = 16 / sizeof(T);
  if (S % UE == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0) {  // 16-byte loads of the slice weights
    const int units = S / UE;
    for (int i = t; i < R * units; i += 256) {  // rows past the end of the batch: zeros
      const int r = i / units, u = i - r * units;
      u32x4 raw = {0u, 0u, 0u, 0u};
      if (r < rows) raw = *reinterpret_cast<const u32x4 *>(w + (m0 + r) * H * S + h * S + u * UE);
      const T *e = reinterpret_cast<const T *>(&raw);
#pragma unroll
      for (int j = 0; j < UE; ++j) wl[r * (S + 1) + u * UE + j] = load_as_f32(e + j);
    }
  } else {
    for (int i = t; i < R * S; i += 256) {
      const int r = i / S, s = i - r * S;
      wl[r * (S + 1) + s] = r < rows ? load_as_f32(w + (m0 + r) * H * S + h * S + s) : 0.f;
    }
  }
  __syncthreads();
  if (D % 4 == 0 && reinterpret_cast<uintptr_t>(out_x) % 16 == 0) {
    // a thread owns 4 rows x 4 adjacent features: one 16-byte and four 4-byte LDS reads per 16 multiply-adds, and the
    // results leave as 8- or 16-byte stores
    const int DQ4 = D >> 2, S1 = S + 1;
    for (int tile = t; tile < (R >> 2) * DQ4; tile += 256) {
      const int rq = tile / DQ4, dq = tile - rq * DQ4, r0 = 4 * rq;
      if (r0 >= rows) continue;
      const float *w0 = wl + r0 * S1;
      float acc[4][4];
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int k = 0; k < 4; ++k) acc[j][k] = 0.f;
      for (int sl = 0; sl < S; ++sl) {
        const float4 tv = *reinterpret_cast<const float4 *>(tk + sl * D + 4 * dq);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float wv = w0[j * S1 + sl];
          acc[j][0] = fmaf(wv, tv.x, acc[j][0]);
          acc[j][1] = fmaf(wv, tv.y, acc[j][1]);
          acc[j][2] = fmaf(wv, tv.z, acc[j][2]);
          acc[j][3] = fmaf(wv, tv.w, acc[j][3]);
        }
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (r0 + j >= rows) continue;
        alignas(16) T o4[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) store_from_f32(o4 + k, acc[j][k]);
        T *dst = out_x + (m0 + r0 + j) * H * D + h * D + 4 * dq;
        if constexpr (sizeof(T) == 2) *reinterpret_cast<u32x2 *>(dst) = *reinterpret_cast<const u32x2 *>(o4);
        else *reinterpret_cast<u32x4 *>(dst) = *reinterpret_cast<const u32x4 *>(o4);
      }
    }
    return;
  }
  // a thread owns 4 rows x 2 features (features dq and dq + DQ): 6 LDS reads per 8 multiply-adds
  const int DQ = (D + 1) >> 1, S1 = S + 1;
  for (int tile = t; tile < (R >> 2) * DQ; tile += 256) {
    const int rq = tile / DQ, dq = tile - rq * DQ, r0 = 4 * rq;
    if (r0 >= rows) continue;
    const int d1 = min(dq + DQ, D - 1);
    const float *w0 = wl + r0 * S1;
    float acc[4][2] = {{0.f, 0.f}, {0.f, 0.f}, {0.f, 0.f}, {0.f, 0.f}};
    for (int sl = 0; sl < S; ++sl) {
      const float t0 = tk[sl * D + dq], t1 = tk[sl * D + d1];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float wv = w0[j * S1 + sl];
        acc[j][0] = fmaf(wv, t0, acc[j][0]);
        acc[j][1] = fmaf(wv, t1, acc[j][1]);
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (r0 + j >= rows) continue;
      T *o = out_x + (m0 + r0 + j) * H * D + h * D;
      store_from_f32(o + dq, acc[j][0]);
      if (dq + DQ < D) store_from_f32(o + dq + DQ, acc[j][1]);
    }
  }
}

// ------------------------------------------------------------------------------------------------
// residual_ln_kernel: one wave per row.  y <- y + residual (rounded to the storage type);
// ln_out = (y - mean) / sqrt(var + eps) * gamma + beta with the biased variance, all statistics in fp32.
// ------------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void residual_ln_kernel(T *__restrict__ y, const T *__restrict__ residual,
                                                          const float *__restrict__ gamma, const float *__restrict__ beta,
                                                          float eps, T *__restrict__ ln_out, int64_t M, int C) {
  const int lane = threadIdx.x & 63;
  const int64_t m = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (m >= M) return;
  T *yr = y + m * C;
  float sum = 0.f;
  for (int c = lane; c < C; c += 64) {
    float v = load_as_f32(yr + c);
    if (residual) {
      v = round_to(yr, v + load_as_f32(residual + m * C + c));
      store_from_f32(yr + c, v);
    }
    sum += v;
  }
  if (!ln_out) return;
  const float mean = wave_sum(sum) / (float)C;
  float sq = 0.f;
  for (int c = lane; c < C; c += 64) {
    const float dlt = load_as_f32(yr + c) - mean;
    sq = fmaf(dlt, dlt, sq);
  }
  const float rstd = rsqrtf(wave_sum(sq) / (float)C + eps);
  for (int c = lane; c < C; c += 64) {
    const float v = (load_as_f32(yr + c) - mean) * rstd;
    store_from_f32(ln_out + m * C + c, v * gamma[c] + beta[c]);
  }
}

// residual_ln_vec_kernel: the same with 16-byte accesses for rows that are whole 16-byte units (C % UE == 0,
// C <= 64 * UPL * UE): lane l owns units l, l + 64, ... of its row and keeps them in registers between the passes.
template <typename T, int UPL>
__global__ __launch_bounds__(256) void residual_ln_vec_kernel(T *__restrict__ y, const T *__restrict__ residual,
                                                              const float *__restrict__ gamma,
                                                              const float *__restrict__ beta, float eps,
                                                              T *__restrict__ ln_out, int64_t M, int C) {
  constexpr int UE = 16 / sizeof(T);
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  const int lane = threadIdx.x & 63;
  const int units = C / UE;
  float gam[UPL][UE], bet[UPL][UE];  // this lane's LayerNorm parameters stay in registers across its rows
#pragma unroll
  for (int k = 0; k < UPL; ++k)
#pragma unroll
    for (int e = 0; e < UE; ++e) {
      const int c = (lane + 64 * k) * UE + e;
      gam[k][e] = (ln_out && c < C) ? gamma[c] : 1.f;
      bet[k][e] = (ln_out && c < C) ? beta[c] : 0.f;
    }
  // one wave per row at a time; the grid is sized to the machine and every wave walks rows a grid apart
  for (int64_t m = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); m < M; m += (int64_t)gridDim.x * 4) {
  T *yr = y + m * C;
  float v[UPL][UE];
  float sum = 0.f;
#pragma unroll
  for (int k = 0; k < UPL; ++k) {
    const int u = lane + 64 * k;
    if (u < units) {
      u32x4 a = *reinterpret_cast<const u32x4 *>(yr + u * UE);
      const T *ae = reinterpret_cast<const T *>(&a);
      if (residual) {
        u32x4 r = *reinterpret_cast<const u32x4 *>(residual + m * C + u * UE);
        const T *re = reinterpret_cast<const T *>(&r);
        alignas(16) T o[UE];
#pragma unroll
        for (int e = 0; e < UE; ++e) {
          v[k][e] = round_to(yr, load_as_f32(ae + e) + load_as_f32(re + e));
          store_from_f32(o + e, v[k][e]);
        }
        *reinterpret_cast<u32x4 *>(yr + u * UE) = *reinterpret_cast<const u32x4 *>(o);
      } else {
#pragma unroll
        for (int e = 0; e < UE; ++e) v[k][e] = load_as_f32(ae + e);
      }
#pragma unroll
      for (int e = 0; e < UE; ++e) sum += v[k][e];
    }
  }
  if (!ln_out) continue;
  const float mean = wave_sum(sum) / (float)C;
  float sq = 0.f;
#pragma unroll
  for (int k = 0; k < UPL; ++k)
    if (lane + 64 * k < units) {
#pragma unroll
      for (int e = 0; e < UE; ++e) {
        const float d = v[k][e] - mean;
        sq = fmaf(d, d, sq);
      }
    }
  const float rstd = rsqrtf(wave_sum(sq) / (float)C + eps);
#pragma unroll
  for (int k = 0; k < UPL; ++k) {
    const int u = lane + 64 * k;
    if (u < units) {
      alignas(16) T o[UE];
#pragma unroll
      for (int e = 0; e < UE; ++e)
        store_from_f32(o + e, (v[k][e] - mean) * rstd * gam[k][e] + bet[k][e]);
      *reinterpret_cast<u32x4 *>(ln_out + m * C + u * UE) = *reinterpret_cast<const u32x4 *>(o);
    }
  }
  }
}

// layernorm_backward_kernel: backward of y = (x - mean) * rstd * gamma + beta over rows of whole 16-byte units.
//   xh = (x - mean) rstd;  g = dy gamma;  dx = rstd (g - mean_c(g) - xh mean_c(g xh));  d gamma = sum_rows dy xh;
//   d beta = sum_rows dy.   One wave per row at a time (statistics recomputed from x), lane l owns units l, l + 64, ...;
// every wave accumulates d gamma / d beta of its columns over the rows it walks, the four waves of a workgroup add up
// through LDS and each workgroup leaves one partial [2][C] (the caller adds the partials in index order).
template <typename T, int UPL>
__global__ __launch_bounds__(256) void layernorm_backward_kernel(const T *__restrict__ x, const T *__restrict__ dy,
                                                                 const float *__restrict__ gamma, float eps,
                                                                 T *__restrict__ dx, float *__restrict__ partials,
                                                                 int64_t M, int C) {
  constexpr int UE = 16 / sizeof(T);
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  extern __shared__ float red[];  // [4 waves][2][C]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int units = C / UE;
  float gam[UPL][UE], dg[UPL][UE], db[UPL][UE];
#pragma unroll
  for (int k = 0; k < UPL; ++k)
#pragma unroll
    for (int e = 0; e < UE; ++e) {
      const int c = (lane + 64 * k) * UE + e;
      gam[k][e] = c < C ? gamma[c] : 0.f;
      dg[k][e] = db[k][e] = 0.f;
    }
  const float inv_c = 1.f / (float)C;
  for (int64_t m = (int64_t)blockIdx.x * 4 + wave; m < M; m += (int64_t)gridDim.x * 4) {
    float xv[UPL][UE], gv[UPL][UE];
    float sum = 0.f;
#pragma unroll
    for (int k = 0; k < UPL; ++k) {
      const int u = lane + 64 * k;
#pragma unroll
      for (int e = 0; e < UE; ++e) xv[k][e] = gv[k][e] = 0.f;
      if (u < units) {
        u32x4 a = *reinterpret_cast<const u32x4 *>(x + m * C + u * UE);
        u32x4 d = *reinterpret_cast<const u32x4 *>(dy + m * C + u * UE);
        const T *ae = reinterpret_cast<const T *>(&a), *de = reinterpret_cast<const T *>(&d);
#pragma unroll
        for (int e = 0; e < UE; ++e) {
          xv[k][e] = load_as_f32(ae + e);
          gv[k][e] = load_as_f32(de + e);  // dy for now
          sum += xv[k][e];
        }
      }
    }
    const float mean = wave_sum(sum) * inv_c;
    float sq = 0.f;
#pragma unroll
    for (int k = 0; k < UPL; ++k)
      if (lane + 64 * k < units) {
#pragma unroll
        for (int e = 0; e < UE; ++e) {
          const float dlt = xv[k][e] - mean;
          sq = fmaf(dlt, dlt, sq);
        }
      }
    const float rstd = rsqrtf(wave_sum(sq) * inv_c + eps);
    float s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int k = 0; k < UPL; ++k)
      if (lane + 64 * k < units) {
#pragma unroll
        for (int e = 0; e < UE; ++e) {
          const float xh = (xv[k][e] - mean) * rstd, dyv = gv[k][e];
          dg[k][e] = fmaf(dyv, xh, dg[k][e]);
          db[k][e] += dyv;
          const float g = dyv * gam[k][e];
          xv[k][e] = xh;
          gv[k][e] = g;
          s1 += g;
          s2 = fmaf(g, xh, s2);
        }
      }
    s1 = wave_sum(s1) * inv_c;
    s2 = wave_sum(s2) * inv_c;
#pragma unroll
    for (int k = 0; k < UPL; ++k) {
      const int u = lane + 64 * k;
      if (u < units) {
        alignas(16) T o[UE];
#pragma unroll
        for (int e = 0; e < UE; ++e) store_from_f32(o + e, rstd * (gv[k][e] - s1 - xv[k][e] * s2));
        *reinterpret_cast<u32x4 *>(dx + m * C + u * UE) = *reinterpret_cast<const u32x4 *>(o);
      }
    }
  }
#pragma unroll
  for (int k = 0; k < UPL; ++k)
#pragma unroll
    for (int e = 0; e < UE; ++e) {
      const int c = (lane + 64 * k) * UE + e;
      if (c < C) {
        red[(wave * 2 + 0) * C + c] = dg[k][e];
        red[(wave * 2 + 1) * C + c] = db[k][e];
      }
    }
  __syncthreads();
  for (int i = threadIdx.x; i < 2 * C; i += 256)
    partials[(int64_t)blockIdx.x * 2 * C + i] = ((red[i] + red[2 * C + i]) + red[4 * C + i]) + red[6 * C + i];
}

// ------------------------------------------------------------------------------------------------
// dequant_e4m3_kernel: out[o, k] = bf16(scale[o] * decode_e4m3fn(in[o, k])), for the shapes whose kernels read the
// large weights in natural layout (the repacking kernels of the MFMA paths read the e4m3 bytes themselves).
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void dequant_e4m3_kernel(const uint8_t *__restrict__ in, const float *__restrict__ scale,
                                                           bf16 *__restrict__ out, int64_t rows, int64_t cols) {
  const int64_t n = rows * cols;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256)
    store_from_f32(out + i, scale[i / cols] * decode_e4m3fn(in[i]));
}

// ================================================================================================
// host launchers
// ================================================================================================
template <typename TA, typename TW>
static int launch_gemm(const GemmArgs &a, int nsets, hipStream_t st) {
  if constexpr (sizeof(TA) == sizeof(TW))  // the MFMA kernels take both operands in one type
    if (gemm::serves(a, nsets, sizeof(TA))) return gemm::launch(a, nsets, sizeof(TA) == 4 ? PA_F32 : PA_BF16, st);
  dim3 grid((unsigned)((a.M + 63) / 64), (unsigned)((a.O + 63) / 64), (unsigned)nsets);
  hipLaunchKernelGGL((rows_gemm_kernel<TA, TW>), grid, dim3(256), 0, st, a);
  return launch_status();
}

int dequant_e4m3(const void *in, const float *scale, void *out, int64_t rows, int64_t cols, hipStream_t st) {
  int64_t blocks = (rows * cols + 255) / 256;
  if (blocks > 1024) blocks = 1024;
  hipLaunchKernelGGL(dequant_e4m3_kernel, dim3((unsigned)blocks), dim3(256), 0, st, static_cast<const uint8_t *>(in),
                     scale, static_cast<bf16 *>(out), rows, cols);
  return launch_status();
}

int project_inputs(int dtype, const pa_shape &s, const pa_params &p, const void *x, void *x_mid, void *fx_mid,
                   hipStream_t st) {
  GemmArgs a{};
  a.in = x;
  a.w[0] = p.in_project_x_weight;
  a.w[1] = p.in_project_fx_weight;
  a.bias[0] = p.in_project_x_bias;
  a.bias[1] = p.in_project_fx_bias;
  a.out[0] = x_mid;
  a.out[1] = fx_mid;
  a.M = s.B * s.N;
  a.O = (int)(s.H * s.D);
  a.C = (int)s.C;
  a.N = (int)s.N;
  a.gh = (int)s.grid_h;
  a.gw = (int)s.grid_w;
  a.ks = (int)s.conv_k;
  a.gd = (int)s.grid_d;
  a.w_tap_major = (int)s.conv_tap_major;
  a.K = s.conv_k > 0 ? (int)(s.conv_k * s.conv_k * (s.grid_d > 0 ? s.conv_k : 1) * s.C) : (int)s.C;
  const int nsets = fx_mid ? 2 : 1;  // Transolver++ has a single projection
  return dtype == PA_F32 ? launch_gemm<float, float>(a, nsets, st) : launch_gemm<bf16, bf16>(a, nsets, st);
}

// out[m, o] = bias[o] + sum_k A(m, k) weight[o, k] for any (c_in, c_out): a Linear over the rows when grid.conv_k == 0,
// else the k x k (x k) convolution over grid's point grid with weight (c_out, c_in, k, k(, k)).
int rows_gemm(int dtype, const pa_shape &grid, int64_t c_in, int64_t c_out, const void *in, const void *weight,
              const float *bias, int act, void *out, hipStream_t st) {
  GemmArgs a{};
  a.act = act;
  a.in = in;
  a.w[0] = weight;
  a.bias[0] = bias;
  a.out[0] = out;
  a.M = grid.B * grid.N;
  a.O = (int)c_out;
  a.C = (int)c_in;
  a.N = (int)grid.N;
  a.gh = (int)grid.grid_h;
  a.gw = (int)grid.grid_w;
  a.ks = (int)grid.conv_k;
  a.gd = (int)grid.grid_d;
  a.w_tap_major = (int)grid.conv_tap_major;
  a.K = grid.conv_k > 0 ? (int)(grid.conv_k * grid.conv_k * (grid.grid_d > 0 ? grid.conv_k : 1) * c_in) : (int)c_in;
  return dtype == PA_F32 ? launch_gemm<float, float>(a, 1, st) : launch_gemm<bf16, bf16>(a, 1, st);
}

// bf16 Linear over the rows with the result in natural layout (`out`, may be NULL) and in the packed operand layout of
// the MFMA slice kernels (`out_pack`, (B * tiles * H * 2) KiB as fx_pack); c_out = H * 32.
int rows_gemm_packed(const pa_shape &s, int64_t c_in, const void *in, const void *weight, const float *bias, void *out,
                     void *out_pack, hipStream_t st) {
  GemmArgs a{};
  a.in = in;
  a.w[0] = weight;
  a.bias[0] = bias;
  a.out[0] = out;
  a.out_pack[0] = out_pack;
  a.M = s.B * s.N;
  a.N = (int)s.N;
  a.K = (int)c_in;
  a.O = (int)(s.H * 32);
  a.C = (int)c_in;
  a.pack_tpb = (int)((s.N + 31) / 32);
  a.pack_heads = (int)s.H;
  if (c_in % 8 != 0 || !gemm::serves(a, 1, 2)) return PA_ERR_UNSUPPORTED;
  return gemm::launch(a, 1, PA_BF16, st);
}

int out_linear(int dtype, const pa_shape &s, const pa_params &p, const void *out_x, void *y, hipStream_t st) {
  GemmArgs a{};
  a.in = out_x;
  a.w[0] = p.out_linear_weight;
  a.bias[0] = p.out_linear_bias;
  a.out[0] = y;
  a.M = s.B * s.N;
  a.K = (int)(s.H * s.D);
  a.O = (int)s.C;
  a.ks = 0;
  return dtype == PA_F32 ? launch_gemm<float, float>(a, 1, st) : launch_gemm<bf16, bf16>(a, 1, st);
}

// Slice weights (PA.py:537, :172-181): the logits are a Linear over the (point, head) rows -- D inputs, S outputs,
// one weight for all heads -- so they come from the row GEMM kernels (MFMA for float32; the float32 weight against
// bf16 rows takes the FMA kernel), written in the storage type as the reference's Linear output is; the softmax with
// the head's clamped temperature then runs in place over each row of S.
template <typename T>
static int slice_softmax_t(const pa_shape &s, const pa_params &p, const void *x_mid, void *w, hipStream_t st) {
  GemmArgs a{};
  a.in = x_mid;
  a.w[0] = p.in_project_slice_weight;
  a.bias[0] = p.in_project_slice_bias;
  a.out[0] = w;
  a.M = s.B * s.N * s.H;
  a.K = (int)s.D;
  a.O = (int)s.S;
  int rc = launch_gemm<T, float>(a, 1, st);
  if (rc) return rc;
  return flare::softmax_rows(sizeof(T) == 4 ? PA_F32 : PA_BF16, s, w, p.temperature, st);
}

int slice_softmax(int dtype, const pa_shape &s, const pa_params &p, const void *x_mid, void *w, hipStream_t st) {
  return dtype == PA_F32 ? slice_softmax_t<float>(s, p, x_mid, w, st) : slice_softmax_t<bf16>(s, p, x_mid, w, st);
}

template <typename T, int L>
static int softmax_rows_plus_l(const pa_shape &s, const pa_params &p, const pa_plus_params &pp, void *w,
                               const void *hidden, const void *uniform, hipStream_t st) {
  const int64_t rows = s.B * s.N * s.H;
  int64_t blocks = (rows + (256 / L) - 1) / (256 / L);
  if (blocks > 16384) blocks = 16384;
  hipLaunchKernelGGL((softmax_rows_plus_kernel<T, L>), dim3((unsigned)blocks), dim3(256), 0, st, static_cast<T *>(w),
                     static_cast<const T *>(hidden), static_cast<const T *>(uniform), p.temperature,
                     pp.proj_temperature_2_weight, pp.proj_temperature_2_bias, rows, (int)s.S, (int)s.H);
  return launch_status();
}

template <typename T, int LR>
static int softmax_rows_plus_vec(const pa_shape &s, const pa_params &p, const pa_plus_params &pp, void *w,
                                 const void *hidden, const void *uniform, hipStream_t st) {
  const int64_t rows = s.B * s.N * s.H;
  int64_t blocks = (rows + (256 / LR) - 1) / (256 / LR);
  if (blocks > 16384) blocks = 16384;
  hipLaunchKernelGGL((softmax_rows_plus_vec_kernel<T, LR>), dim3((unsigned)blocks), dim3(256), 0, st,
                     static_cast<T *>(w), static_cast<const T *>(hidden), static_cast<const T *>(uniform), p.temperature,
                     pp.proj_temperature_2_weight, pp.proj_temperature_2_bias, rows, (int)s.S, (int)s.H);
  return launch_status();
}

// With a scratch buffer of B*N*H*S elements the two Linears run on the row GEMM kernels (several times faster than the
// single kernel below, which forms them per point on the vector ALUs).
template <typename T>
static int slice_softmax_plus_staged(const pa_shape &s, const pa_params &p, const pa_plus_params &pp, const void *x_mid,
                                     const void *uniform, void *w, void *scratch, hipStream_t st) {
  GemmArgs a{};
  a.in = x_mid;
  a.M = s.B * s.N * s.H;
  a.K = (int)s.D;
  a.O = (int)s.S;
  a.w[0] = p.in_project_slice_weight;
  a.bias[0] = p.in_project_slice_bias;
  a.out[0] = w;
  int rc = launch_gemm<T, float>(a, 1, st);
  if (rc) return rc;
  a.w[0] = pp.proj_temperature_0_weight;
  a.bias[0] = pp.proj_temperature_0_bias;
  a.out[0] = scratch;
  a.act = 1;
  if ((rc = launch_gemm<T, float>(a, 1, st))) return rc;
  constexpr int UE = 16 / sizeof(T);
  if (s.S % UE == 0 && s.S / UE <= 64 && (reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(scratch) |
                                          reinterpret_cast<uintptr_t>(uniform)) % 16 == 0) {
    const int64_t units = s.S / UE;
    if (units <= 1) return softmax_rows_plus_vec<T, 1>(s, p, pp, w, scratch, uniform, st);
    if (units <= 2) return softmax_rows_plus_vec<T, 2>(s, p, pp, w, scratch, uniform, st);
    if (units <= 4) return softmax_rows_plus_vec<T, 4>(s, p, pp, w, scratch, uniform, st);
    if (units <= 8) return softmax_rows_plus_vec<T, 8>(s, p, pp, w, scratch, uniform, st);
    if (units <= 16) return softmax_rows_plus_vec<T, 16>(s, p, pp, w, scratch, uniform, st);
    if (units <= 32) return softmax_rows_plus_vec<T, 32>(s, p, pp, w, scratch, uniform, st);
    return softmax_rows_plus_vec<T, 64>(s, p, pp, w, scratch, uniform, st);
  }
  if (s.S <= 8) return softmax_rows_plus_l<T, 8>(s, p, pp, w, scratch, uniform, st);
  if (s.S <= 16) return softmax_rows_plus_l<T, 16>(s, p, pp, w, scratch, uniform, st);
  if (s.S <= 32) return softmax_rows_plus_l<T, 32>(s, p, pp, w, scratch, uniform, st);
  return softmax_rows_plus_l<T, 64>(s, p, pp, w, scratch, uniform, st);
}

template <typename T>
static int slice_softmax_plus_t(const pa_shape &s, const pa_params &p, const pa_plus_params &pp, const void *x_mid,
                                const void *uniform, void *w, void *scratch, hipStream_t st) {
  if (scratch) return slice_softmax_plus_staged<T>(s, p, pp, x_mid, uniform, w, scratch, st);
  const int H = (int)s.H, D = (int)s.D, S = (int)s.S;
  const size_t fixed = (size_t)(2 * S * D + 3 * S) * 4;
  const size_t per_row = (size_t)(H * (D + 1) + H * (S + 1)) * 4;
  if (fixed + per_row > 60 * 1024) return PA_ERR_UNSUPPORTED;
  int R = (int)((60 * 1024 - fixed) / per_row);
  if (R > 8) R = 8;
  const size_t lds = fixed + per_row * R;
  int rc = allow_dynamic_lds(slice_softmax_plus_kernel<T>, lds);
  if (rc) return rc;
  const int64_t M = s.B * s.N;
  hipLaunchKernelGGL((slice_softmax_plus_kernel<T>), dim3((unsigned)((M + R - 1) / R)), dim3(256), lds, st,
                     static_cast<const T *>(x_mid), static_cast<const T *>(uniform), p.in_project_slice_weight,
                     p.in_project_slice_bias, p.temperature, pp.proj_temperature_0_weight, pp.proj_temperature_0_bias,
                     pp.proj_temperature_2_weight, pp.proj_temperature_2_bias, static_cast<T *>(w), M, H, D, S, R);
  return launch_status();
}

int slice_softmax_plus(int dtype, const pa_shape &s, const pa_params &p, const pa_plus_params &pp, const void *x_mid,
                       const void *uniform, void *w, void *scratch, hipStream_t st) {
  return dtype == PA_F32 ? slice_softmax_plus_t<float>(s, p, pp, x_mid, uniform, w, scratch, st)
                         : slice_softmax_plus_t<bf16>(s, p, pp, x_mid, uniform, w, scratch, st);
}

// Number of point chunks of the first reduction pass: enough workgroups to fill 256 CUs several times
// over, at least 256 points per chunk.  Depends on the shape only, so results are reproducible.
int64_t partial_count(const pa_shape &s) {
  int64_t by_size = (s.N + 255) / 256;
  int64_t by_grid = (4096 + s.B * s.H - 1) / (s.B * s.H);
  int64_t g = by_size < by_grid ? by_size : by_grid;
  return g < 1 ? 1 : g;
}

size_t combine_attn_lds_bytes(const pa_shape &s) {
  return (size_t)(4 * s.S * (s.D + 1) + (kAttnThreads / 64) * s.S) * 4;
}

template <typename T>
static int slice_partial_t(const pa_shape &s, const void *w, const void *fx_mid, float *partials, hipStream_t st) {
  const int64_t G = partial_count(s);
  const int64_t chunk = (s.N + G - 1) / G;
  const int SB = (int)((s.S + 3) / 4), DB = (int)((s.D + 1 + 3) / 4);
  const int n_tiles = SB * DB;
  const size_t lds = (size_t)kPartialTile * (SB + DB) * 16;
  const int per_thread = (n_tiles + 255) / 256;
  const int ns = per_thread <= 1 ? 1 : (per_thread <= 2 ? 2 : kPartialMaxNS);
  dim3 grid((unsigned)G, (unsigned)(s.B * s.H), (unsigned)((n_tiles + 256 * ns - 1) / (256 * ns)));
  auto launch = [&](auto kernel) {
    int rc = allow_dynamic_lds(kernel, lds);
    if (rc) return rc;
    hipLaunchKernelGGL(kernel, grid, dim3(256), lds, st, static_cast<const T *>(w), static_cast<const T *>(fx_mid),
                       partials, (int)s.B, s.N, (int)s.H, (int)s.D, (int)s.S, chunk);
    return launch_status();
  };
  if (ns == 1) return launch(slice_partial_kernel<T, 1>);
  if (ns == 2) return launch(slice_partial_kernel<T, 2>);
  return launch(slice_partial_kernel<T, kPartialMaxNS>);
}

// `partials` holds G partial sums followed by one spare slot (index G) that receives their fixed-order total.
// G == 0: `partials` holds finished slice tokens (attention only).
// Fixed-order total of the G partial sums [G][B][H][S][D+1]; the total goes to slot G of the same buffer.  Returns
// where the totals are (the partials themselves when G == 1).
int combine_partials(const pa_shape &s, const float *partials, int64_t G, const float **combined, hipStream_t st) {
  const int64_t stride = s.B * s.H * s.S * (s.D + 1);
  *combined = partials;
  if (G <= 1) return PA_OK;
  float *total = const_cast<float *>(partials) + G * stride;
  const int n_out = (int)(s.S * (s.D + 1));
  hipLaunchKernelGGL(combine_partials_kernel, dim3((unsigned)((n_out + 63) / 64), (unsigned)(s.B * s.H)), dim3(256), 0, st,
                     partials, (int)G, stride, total, n_out);
  *combined = total;
  return launch_status();
}

int combine_attention(const pa_shape &s, const pa_params &p, const float *partials, int64_t G, float *slice_token,
                      float *slice_norm, float *out_token, hipStream_t st) {
  size_t lds = combine_attn_lds_bytes(s);
  const size_t wq_bytes = (size_t)3 * s.D * (s.D + 1) * 4;
  const int stage_w = lds + wq_bytes <= 96 * 1024 ? 1 : 0;  // qkv weight rows in LDS when they fit comfortably
  if (stage_w) lds += wq_bytes;
  int rc = allow_dynamic_lds(slice_combine_attn_kernel, lds);
  if (rc) return rc;
  const int64_t stride = s.B * s.H * s.S * (s.D + 1);
  const float *src = partials;
  int g_in = (int)G;  // a few partials are summed by the attention kernel itself, in index order
  if (G > 8) {
    if ((rc = combine_partials(s, partials, G, &src, st))) return rc;
    g_in = 1;
  }
  hipLaunchKernelGGL(slice_combine_attn_kernel, dim3((unsigned)(s.B * s.H)), dim3(kAttnThreads), lds, st, src, g_in, stride,
                     p.qkv_project_weight, slice_token, slice_norm, out_token, (int)s.D, (int)s.S, stage_w);
  return launch_status();
}

int slice_partial(int dtype, const pa_shape &s, const void *w, const void *fx_mid, float *partials, hipStream_t st) {
  return dtype == PA_F32 ? slice_partial_t<float>(s, w, fx_mid, partials, st)
                         : slice_partial_t<bf16>(s, w, fx_mid, partials, st);
}

template <typename T>
static int deslice_t(const pa_shape &s, const void *w, const float *out_token, void *out_x, hipStream_t st) {
  int R = 128;  // rows per workgroup: the head's token table (S x D floats) is loaded once per tile
  while (R > 8 && (size_t)(s.S * s.D + R * (s.S + 1)) * 4 > 48 * 1024) R >>= 1;
  size_t lds = (size_t)(s.S * s.D + R * (s.S + 1)) * 4;
  int rc = allow_dynamic_lds(deslice_kernel<T>, lds);
  if (rc) return rc;
  const int tiles = (int)((s.N + R - 1) / R);
  dim3 grid((unsigned)(tiles * s.B), (unsigned)s.H);
  hipLaunchKernelGGL((deslice_kernel<T>), grid, dim3(256), lds, st, static_cast<const T *>(w), out_token,
                     static_cast<T *>(out_x), s.N, (int)s.H, (int)s.D, (int)s.S, R, tiles);
  return launch_status();
}

int deslice(int dtype, const pa_shape &s, const void *w, const float *out_token, void *out_x, hipStream_t st) {
  return dtype == PA_F32 ? deslice_t<float>(s, w, out_token, out_x, st) : deslice_t<bf16>(s, w, out_token, out_x, st);
}

template <typename T>
static int residual_ln_t(const pa_shape &s, void *y, const pa_block_tail &tail, hipStream_t st) {
  const int64_t M = s.B * s.N;
  const int C = (int)s.C;
  constexpr int UE = 16 / sizeof(T);
  dim3 grid((unsigned)((M + 3) / 4));
  const dim3 vgrid((unsigned)std::min<int64_t>((M + 3) / 4, 256 * 16));  // the vector kernel's waves walk the rows
  T *yp = static_cast<T *>(y), *lo = static_cast<T *>(tail.ln_out);
  const T *res = static_cast<const T *>(tail.residual);
  const bool vec = C % UE == 0 && aligned16(y) && aligned16(tail.residual) && aligned16(tail.ln_out);
  const int upl = (C / UE + 63) / 64;
  if (vec && upl <= 1)
    hipLaunchKernelGGL((residual_ln_vec_kernel<T, 1>), vgrid, dim3(256), 0, st, yp, res, tail.ln_gamma, tail.ln_beta,
                       tail.ln_eps, lo, M, C);
  else if (vec && upl <= 2)
    hipLaunchKernelGGL((residual_ln_vec_kernel<T, 2>), vgrid, dim3(256), 0, st, yp, res, tail.ln_gamma, tail.ln_beta,
                       tail.ln_eps, lo, M, C);
  else if (vec && upl <= 4)
    hipLaunchKernelGGL((residual_ln_vec_kernel<T, 4>), vgrid, dim3(256), 0, st, yp, res, tail.ln_gamma, tail.ln_beta,
                       tail.ln_eps, lo, M, C);
  else
    hipLaunchKernelGGL((residual_ln_kernel<T>), grid, dim3(256), 0, st, yp, res, tail.ln_gamma, tail.ln_beta,
                       tail.ln_eps, lo, M, C);
  return launch_status();
}

int64_t layernorm_backward_groups(int64_t rows) { return std::min<int64_t>((rows + 3) / 4, 256 * 8); }

template <typename T>
static int layernorm_backward_t(int64_t rows, int C, const void *x, const void *dy, const float *gamma, float eps, void *dx,
                                float *partials, hipStream_t st) {
  constexpr int UE = 16 / sizeof(T);
  if (C % UE != 0) return PA_ERR_UNSUPPORTED;
  const int upl = (C / UE + 63) / 64;
  const dim3 grid((unsigned)layernorm_backward_groups(rows));
  const size_t lds = (size_t)8 * C * 4;
  const T *xp = static_cast<const T *>(x), *dp = static_cast<const T *>(dy);
  T *op = static_cast<T *>(dx);
  if (upl <= 1)
    hipLaunchKernelGGL((layernorm_backward_kernel<T, 1>), grid, dim3(256), lds, st, xp, dp, gamma, eps, op, partials, rows, C);
  else if (upl <= 2)
    hipLaunchKernelGGL((layernorm_backward_kernel<T, 2>), grid, dim3(256), lds, st, xp, dp, gamma, eps, op, partials, rows, C);
  else if (upl <= 4)
    hipLaunchKernelGGL((layernorm_backward_kernel<T, 4>), grid, dim3(256), lds, st, xp, dp, gamma, eps, op, partials, rows, C);
  else
    return PA_ERR_UNSUPPORTED;
  return launch_status();
}

int layernorm_backward(int dtype, int64_t rows, int64_t C, const void *x, const void *dy, const float *gamma, float eps,
                       void *dx, float *partials, hipStream_t st) {
  return dtype == PA_F32 ? layernorm_backward_t<float>(rows, (int)C, x, dy, gamma, eps, dx, partials, st)
                         : layernorm_backward_t<bf16>(rows, (int)C, x, dy, gamma, eps, dx, partials, st);
}

int residual_ln(int dtype, const pa_shape &s, void *y, const pa_block_tail &tail, hipStream_t st) {
  return dtype == PA_F32 ? residual_ln_t<float>(s, y, tail, st) : residual_ln_t<bf16>(s, y, tail, st);
}

}  // namespace general
}  // namespace pa
