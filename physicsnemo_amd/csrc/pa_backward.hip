// Backward pass of the PhysicsAttention layer: the per-point and per-slice kernels (fp32 arithmetic on the
// vector ALUs, fp32 or bf16 storage, natural layouts) of the general kernel family.  The weight gradients, plain
// d out^T . in products over the point axis, are computed by cols_gemm_kernel (pa_gemm.hip) or the caller's GEMM
// library; the bf16 MFMA versions of these kernels are in pa_mfma_bwd.hip.
//
// Forward (PA.py:501-558), per batch b and head h, with T = clamp(temperature_h, .5, 5):
//   z[n,s]   = x_mid[n,:] . Ws[s,:] + bs[s];  w[n,:] = softmax_s(z[n,:] / T)
//   num[s,:] = sum_n w[n,s] fx_mid[n,:];  nrm[s] = sum_n w[n,s] + 1e-2;  tok = num / nrm
//   tok'     = softmax(q k^T / sqrt D) v with q|k|v = tok Wqkv^T
//   out_x[n,:] = sum_s w[n,s] tok'[s,:]
// Backward, given g = d out_x:
//   d tok'[s,:] = sum_n w[n,s] g[n,:]                    (slice_partial_kernel + combine, same as the forward sum)
//   d tok       = attention backward                      (slice_attention_backward_kernel)
//   d num = d tok / nrm;  d nrm[s] = -(d tok[s,:] . tok[s,:]) / nrm[s]
//   d w[n,s]  = g[n,:] . tok'[s,:] + fx_mid[n,:] . d num[s,:] + d nrm[s]      (slice_softmax_backward_kernel)
//   d fx_mid[n,:] = sum_s w[n,s] d num[s,:]
//   d l[n,s]  = w[n,s] (d w[n,s] - sum_s' w[n,s'] d w[n,s']);  d z = d l / T;  d T = -sum_{n,s} d l (z/T) / T
//   d x_mid[n,:] = sum_s d z[n,s] Ws[s,:]
#include "pa_common.h"
#include "pa_host.h"

namespace pa {
namespace backward {

constexpr int kAttnBwdThreads = 512;

// ------------------------------------------------------------------------------------------------
// slice_attention_backward_kernel: one workgroup per (b, h).  Recomputes q, k, v and the S x S attention
// matrix P from the saved slice tokens, then
//   dP = dO v^T;  dSc = P * (dP - rowsum(P * dP)) / sqrt(D);  dq = dSc k;  dk = dSc^T q;  dv = P^T dO
//   d tok = dq Wq + dk Wk + dv Wv;   dWq = dq^T tok, dWk = dk^T tok, dWv = dv^T tok   (this (b, h)'s share)
// P and dSc live in a caller-provided scratch of 2*S*S floats per (b, h) (cache resident); the S x D operands in LDS.
// `slice_norm` != nullptr: the outputs are d num = d tok / nrm and d nrm (gradients of the un-normalised sums);
// nullptr: d_num receives d tok itself and d_norm is not written.
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kAttnBwdThreads) void slice_attention_backward_kernel(
    const float *__restrict__ slice_token, const float *__restrict__ slice_norm, const float *__restrict__ w_qkv,
    const float *__restrict__ d_out_token, float *__restrict__ scratch, float *__restrict__ d_num,
    float *__restrict__ d_norm, float *__restrict__ d_wqkv_part, int D, int S) {
  extern __shared__ float lds[];
  const int D1 = D + 1;
  float *tok = lds;             // S * D1
  float *q = tok + S * D1;      // later: d tok
  float *k = q + S * D1;
  float *v = k + S * D1;
  float *dq = v + S * D1;
  float *dk = dq + S * D1;
  float *dv = dk + S * D1;
  float *rows = dv + S * D1;    // per wave: p[S], ds[S]
  const int t = threadIdx.x;
  const int bh = blockIdx.x;
  const int wave = t >> 6, lane = t & 63;
  constexpr int kWaves = kAttnBwdThreads / 64;
  const float *tk = slice_token + (int64_t)bh * S * D;
  const float *dO = d_out_token + (int64_t)bh * S * D;
  float *P = scratch + (int64_t)bh * 2 * S * S;
  float *dSc = P + (int64_t)S * S;

  for (int i = t; i < S * D; i += kAttnBwdThreads) tok[(i / D) * D1 + (i % D)] = tk[i];
  __syncthreads();
  for (int i = t; i < S * 3 * D; i += kAttnBwdThreads) {
    const int s = i / (3 * D), e = i - s * 3 * D;
    const float *wr = w_qkv + (int64_t)e * D;
    const float *tr = tok + s * D1;
    float acc = 0.f;
    for (int d = 0; d < D; ++d) acc = fmaf(tr[d], wr[d], acc);
    float *dst = e < D ? q : (e < 2 * D ? k : v);
    dst[s * D1 + (e % D)] = acc;
  }
  __syncthreads();

  const float scale = rsqrtf((float)D);
  float *pr = rows + wave * 2 * S;
  float *dr = pr + S;
  for (int s = wave; s < S; s += kWaves) {
    const float *qs = q + s * D1;
    const float *dos = dO + (int64_t)s * D;
    float mx = -INFINITY;
    for (int u = lane; u < S; u += 64) {
      const float *ku = k + u * D1;
      const float *vu = v + u * D1;
      float acc = 0.f, dp = 0.f;
      for (int e = 0; e < D; ++e) {
        acc = fmaf(qs[e], ku[e], acc);
        dp = fmaf(dos[e], vu[e], dp);
      }
      acc *= scale;
      pr[u] = acc;
      dr[u] = dp;
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
    const float inv = 1.f / sum;
    float delta = 0.f;
    for (int u = lane; u < S; u += 64) {
      const float p = pr[u] * inv;
      pr[u] = p;
      delta = fmaf(p, dr[u], delta);
    }
    delta = wave_sum(delta);
    for (int u = lane; u < S; u += 64) {
      const float ds = pr[u] * (dr[u] - delta) * scale;
      dr[u] = ds;
      P[(int64_t)s * S + u] = pr[u];
      dSc[(int64_t)s * S + u] = ds;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    for (int e = lane; e < D; e += 64) {
      float acc = 0.f;
      for (int u = 0; u < S; ++u) acc = fmaf(dr[u], k[u * D1 + e], acc);
      dq[s * D1 + e] = acc;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
  __syncthreads();  // P, dSc (global, this workgroup's own) and dq are complete

  for (int i = t; i < S * D; i += kAttnBwdThreads) {
    const int u = i / D, e = i - u * D;
    float ak = 0.f, av = 0.f;
    for (int s = 0; s < S; ++s) {
      ak = fmaf(dSc[(int64_t)s * S + u], q[s * D1 + e], ak);
      av = fmaf(P[(int64_t)s * S + u], dO[(int64_t)s * D + e], av);
    }
    dk[u * D1 + e] = ak;
    dv[u * D1 + e] = av;
  }
  __syncthreads();

  float *dtok = q;  // q is no longer needed
  for (int i = t; i < S * D; i += kAttnBwdThreads) {
    const int s = i / D, d = i - s * D;
    const float *wq = w_qkv + d, *wk = wq + (int64_t)D * D, *wv = wk + (int64_t)D * D;
    float acc = 0.f;
    for (int e = 0; e < D; ++e) {
      acc = fmaf(dq[s * D1 + e], wq[(int64_t)e * D], acc);
      acc = fmaf(dk[s * D1 + e], wk[(int64_t)e * D], acc);
      acc = fmaf(dv[s * D1 + e], wv[(int64_t)e * D], acc);
    }
    dtok[s * D1 + d] = acc;
    const float scale_out = slice_norm ? 1.f / slice_norm[(int64_t)bh * S + s] : 1.f;
    d_num[(int64_t)bh * S * D + i] = acc * scale_out;
  }
  for (int i = t; i < 3 * D * D; i += kAttnBwdThreads) {
    const int which = i / (D * D), rem = i - which * D * D;
    const int e = rem / D, d = rem - e * D;
    const float *src = which == 0 ? dq : (which == 1 ? dk : dv);
    float acc = 0.f;
    for (int s = 0; s < S; ++s) acc = fmaf(src[s * D1 + e], tok[s * D1 + d], acc);
    d_wqkv_part[(int64_t)bh * 3 * D * D + i] = acc;
  }
  if (!slice_norm) return;
  __syncthreads();
  for (int s = t; s < S; s += kAttnBwdThreads) {
    float acc = 0.f;
    for (int d = 0; d < D; ++d) acc = fmaf(dtok[s * D1 + d], tok[s * D1 + d], acc);
    d_norm[(int64_t)bh * S + s] = -acc / slice_norm[(int64_t)bh * S + s];
  }
}

// ------------------------------------------------------------------------------------------------
// slice_softmax_backward_kernel: grid (row tiles of R points per batch, H).  See the file header for the formulas.
// LDS: the head's tables tok', d num, Ws (row stride D+1), d nrm, bs; the tile's rows of x_mid, fx_mid, g (row stride
// D+1) and three R x (S+1) arrays (w, d w -> d z, logits).  R is a power of two <= 32, 256 / R threads share a row
// in the row reductions.
// Outputs: d_proj (B, N, 2*H*D) = [d x_mid | d fx_mid], d_z (B, N, H, S), dT_part[tile, h] (summed by the caller).
//
// PLUS (Transolver++, PA.py:166-170, :530-532): one projection (fx_mid is x_mid; d_proj is (B, N, H*D) and holds the
// sum of both gradients), the softmax argument is (logits + Gumbel noise) / temp with the per-point
//   temp = max(temperature[h] + gelu(a2), 0.01),  a2 = b2 + sum_s w2[s] gelu(a1[s]),  a1 = b1 + W1 x_mid[n,h,:]
// so  d temp = -sum_s d l[s] (logits + noise)[s] / temp^2, which flows (where temp was not clamped) into temperature[h]
// (dT_part, no mask left for the caller) and through the small MLP:  d a2 = d temp gelu'(a2)  (d_a2 (B, N, H) float32),
// d a1[s] = d a2 w2[s] gelu'(a1[s])  (d_a1 (B, N, H, S)),  d x_mid += d a1 . W1.
// ------------------------------------------------------------------------------------------------
struct PlusArgs {
  const void *uniform;   // (B, N, H, S) activation type
  const float *w1, *b1, *w2, *b2;
  void *d_a1;            // (B, N, H, S) activation type
  float *d_a2;           // (B, N, H)
};

template <typename T, bool PLUS>
__global__ __launch_bounds__(256) void slice_softmax_backward_kernel(
    const T *__restrict__ x_mid, const T *__restrict__ fx_mid, const T *__restrict__ w, const T *__restrict__ d_out_x,
    const float *__restrict__ out_token, const float *__restrict__ d_num, const float *__restrict__ d_norm,
    const float *__restrict__ w_slice, const float *__restrict__ b_slice, const float *__restrict__ temperature,
    T *__restrict__ d_proj, T *__restrict__ d_z, float *__restrict__ dT_part, int64_t N, int H, int D, int S, int R,
    int tiles_per_batch, PlusArgs plus) {
  extern __shared__ float lds[];
  const int D1 = D + 1, S1 = S + 1;
  float *to = lds;               // S * D1
  float *dn = to + S * D1;       // S * D1
  float *ws = dn + S * D1;       // S * D1
  float *dnr = ws + S * D1;      // S
  float *bs = dnr + S;           // S
  float *xm = bs + S;            // R * D1
  float *fm = xm + R * D1;       // R * D1
  float *go = fm + R * D1;       // R * D1
  float *wl = go + R * D1;       // R * S1
  float *dwl = wl + R * S1;      // R * S1
  float *lgl = dwl + R * S1;     // R * S1
  float *w1 = lgl + R * S1;      // PLUS only: S * D1
  float *b1 = w1 + S * D1;       // S
  float *w2 = b1 + S;            // S
  float *a1l = w2 + S;           // R * S1
  __shared__ float red[4];
  const int t = threadIdx.x;
  const int h = blockIdx.y;
  const int b = blockIdx.x / tiles_per_batch;
  const int64_t n0 = (int64_t)(blockIdx.x % tiles_per_batch) * R;
  const int rows = (int)min((int64_t)R, N - n0);
  const int64_t m0 = (int64_t)b * N + n0;
  const int HD = H * D, HS = H * S;
  const float temp_h = PLUS ? temperature[h] : clamp_temperature(temperature[h]);
  const float inv_temp_h = 1.f / temp_h;

  const int64_t bh = (int64_t)b * H + h;
  for (int i = t; i < S * D; i += 256) {
    const int s = i / D, d = i - s * D;
    to[s * D1 + d] = out_token[bh * S * D + i];
    dn[s * D1 + d] = d_num[bh * S * D + i];
    ws[s * D1 + d] = w_slice[i];
    if constexpr (PLUS) w1[s * D1 + d] = plus.w1[i];
  }
  for (int i = t; i < S; i += 256) {
    dnr[i] = d_norm[bh * S + i];
    bs[i] = b_slice[i];
    if constexpr (PLUS) {
      b1[i] = plus.b1[i];
      w2[i] = plus.w2[i];
    }
  }
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  constexpr int UE = 16 / sizeof(T);
  // rows that are whole numbers of 16-byte units move with 16-byte accesses
  const bool vec_d = D % UE == 0 && (reinterpret_cast<uintptr_t>(x_mid) | reinterpret_cast<uintptr_t>(fx_mid) |
                                     reinterpret_cast<uintptr_t>(d_out_x) | reinterpret_cast<uintptr_t>(d_proj)) % 16 == 0;
  const bool vec_s = S % UE == 0 && (reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(d_z) |
                                     (PLUS ? reinterpret_cast<uintptr_t>(plus.d_a1) : 0)) % 16 == 0;
  if (vec_d) {
    const int units = D / UE;
    for (int i = t; i < R * units; i += 256) {
      const int r = i / units, u = i - r * units;
      u32x4 rx = {0u, 0u, 0u, 0u}, rf = rx, rg = rx;
      if (r < rows) {
        const int64_t off = (m0 + r) * HD + h * D + u * UE;
        rx = *reinterpret_cast<const u32x4 *>(x_mid + off);
        rf = *reinterpret_cast<const u32x4 *>(fx_mid + off);
        rg = *reinterpret_cast<const u32x4 *>(d_out_x + off);
      }
      const T *ex = reinterpret_cast<const T *>(&rx), *ef = reinterpret_cast<const T *>(&rf),
              *eg = reinterpret_cast<const T *>(&rg);
#pragma unroll
      for (int j = 0; j < UE; ++j) {
        xm[r * D1 + u * UE + j] = load_as_f32(ex + j);
        fm[r * D1 + u * UE + j] = load_as_f32(ef + j);
        go[r * D1 + u * UE + j] = load_as_f32(eg + j);
      }
    }
  } else {
    for (int i = t; i < R * D; i += 256) {
      const int r = i / D, d = i - r * D;
      const bool ok = r < rows;
      const int64_t off = (m0 + r) * HD + h * D + d;
      xm[r * D1 + d] = ok ? load_as_f32(x_mid + off) : 0.f;
      fm[r * D1 + d] = ok ? load_as_f32(fx_mid + off) : 0.f;
      go[r * D1 + d] = ok ? load_as_f32(d_out_x + off) : 0.f;
    }
  }
  if (vec_s) {
    const int units = S / UE;
    for (int i = t; i < R * units; i += 256) {
      const int r = i / units, u = i - r * units;
      u32x4 rw = {0u, 0u, 0u, 0u};
      if (r < rows) rw = *reinterpret_cast<const u32x4 *>(w + (m0 + r) * HS + h * S + u * UE);
      const T *ew = reinterpret_cast<const T *>(&rw);
#pragma unroll
      for (int j = 0; j < UE; ++j) wl[r * S1 + u * UE + j] = load_as_f32(ew + j);
    }
  } else {
    for (int i = t; i < R * S; i += 256) {
      const int r = i / S, s = i - r * S;
      wl[r * S1 + s] = r < rows ? load_as_f32(w + (m0 + r) * HS + h * S + s) : 0.f;
    }
  }
  __syncthreads();

  // d w and the logits: a thread owns 2 rows x 4 slices (slices sq, sq + SQ, ...: neighbouring lanes read
  // neighbouring table rows, whose odd stride spreads them over the banks; the row operands are wave-wide broadcasts),
  // 18 LDS reads feed 24 multiply-adds
  {
    const int SQ = (S + 3) >> 2;
    for (int tile = t; tile < (R >> 1) * SQ; tile += 256) {
      const int rp = tile / SQ, sq = tile - rp * SQ, r0 = 2 * rp;
      int so[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) so[k] = min(sq + k * SQ, S - 1) * D1;
      const float *x0 = xm + r0 * D1, *f0 = fm + r0 * D1, *g0 = go + r0 * D1;
      float z[2][4], dw[2][4], a[2][4];
#pragma unroll
      for (int jj = 0; jj < 2; ++jj)
#pragma unroll
        for (int k = 0; k < 4; ++k) z[jj][k] = dw[jj][k] = a[jj][k] = 0.f;
      for (int d = 0; d < D; ++d) {
        const float xa = x0[d], xb = x0[D1 + d], fa = f0[d], fb = f0[D1 + d], ga = g0[d], gb = g0[D1 + d];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const float tv = to[so[k] + d], nv = dn[so[k] + d], wv = ws[so[k] + d];
          z[0][k] = fmaf(xa, wv, z[0][k]);
          z[1][k] = fmaf(xb, wv, z[1][k]);
          dw[0][k] = fmaf(fa, nv, fmaf(ga, tv, dw[0][k]));
          dw[1][k] = fmaf(fb, nv, fmaf(gb, tv, dw[1][k]));
          if constexpr (PLUS) {
            const float v1 = w1[so[k] + d];
            a[0][k] = fmaf(xa, v1, a[0][k]);
            a[1][k] = fmaf(xb, v1, a[1][k]);
          }
        }
      }
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int sl = sq + k * SQ;
        if (sl >= S) continue;
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
          const int r = r0 + jj;
          dwl[r * S1 + sl] = dw[jj][k] + dnr[sl];
          if constexpr (PLUS) {
            a1l[r * S1 + sl] = a[jj][k] + b1[sl];
            const float u = r < rows ? load_as_f32(static_cast<const T *>(plus.uniform) + (m0 + r) * HS + h * S + sl) : 0.5f;
            lgl[r * S1 + sl] = round_to(x_mid, z[jj][k] + bs[sl]) - logf(-logf(u + 1e-8f) + 1e-8f);  // divided by temp below
          } else {
            lgl[r * S1 + sl] = round_to(x_mid, z[jj][k] + bs[sl]) * inv_temp_h;  // the forward divides the stored Linear output
          }
        }
      }
    }
  }
  __syncthreads();

  // softmax backward per row; 256 / R threads per row
  const int tpr = 256 / R;
  const int r_own = t / tpr, j_own = t - r_own * tpr;
  float inv_temp = inv_temp_h, traw = 0.f, a2 = 0.f;
  if constexpr (PLUS) {
    a2 = 0.f;
    for (int s = j_own; s < S; s += tpr) a2 = fmaf(w2[s], gelu_erf(a1l[r_own * S1 + s]), a2);
    for (int off = tpr >> 1; off > 0; off >>= 1) a2 += __shfl_xor(a2, off, 64);
    a2 += plus.b2[0];
    traw = temp_h + gelu_erf(a2);
    inv_temp = 1.f / round_to(x_mid, fmaxf(traw, 0.01f));
  }
  // The softmax is formed again in float32 for its own backward: its rows then sum to one, which the identity
  // sum_s d l[s] = 0 behind d temperature needs (with weights rounded to bf16 the defect, times the common offset of
  // the logits, would swamp it).  The stored weights still serve the aggregation and deslice terms.
  const float yscale = PLUS ? inv_temp : 1.f;  // lgl holds the softmax argument itself when not PLUS
  float mx = -INFINITY;
  for (int s = j_own; s < S; s += tpr) mx = fmaxf(mx, lgl[r_own * S1 + s] * yscale);
  for (int off = tpr >> 1; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
  float sum = 0.f;
  for (int s = j_own; s < S; s += tpr) sum += expf(lgl[r_own * S1 + s] * yscale - mx);
  for (int off = tpr >> 1; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
  const float inv_sum = 1.f / sum;
  auto weight = [&](int s) { return r_own < rows ? expf(lgl[r_own * S1 + s] * yscale - mx) * inv_sum : 0.f; };
  float dot = 0.f;
  for (int s = j_own; s < S; s += tpr) dot = fmaf(weight(s), dwl[r_own * S1 + s], dot);
  for (int off = tpr >> 1; off > 0; off >>= 1) dot += __shfl_xor(dot, off, 64);
  float tsum = 0.f;
  for (int s = j_own; s < S; s += tpr) {
    const float dl = weight(s) * (dwl[r_own * S1 + s] - dot);
    tsum = fmaf(dl, lgl[r_own * S1 + s], tsum);
    dwl[r_own * S1 + s] = dl * inv_temp;
  }
  if constexpr (PLUS) {
    for (int off = tpr >> 1; off > 0; off >>= 1) tsum += __shfl_xor(tsum, off, 64);
    const float d_temp = traw >= 0.01f ? -tsum * inv_temp * inv_temp : 0.f;  // clamp(min): gradient where not clamped
    const float d_a2 = d_temp * gelu_erf_grad(a2);
    for (int s = j_own; s < S; s += tpr) a1l[r_own * S1 + s] = d_a2 * w2[s] * gelu_erf_grad(a1l[r_own * S1 + s]);
    if (j_own == 0 && r_own < rows) plus.d_a2[(m0 + r_own) * H + h] = d_a2;
    tsum = j_own == 0 ? d_temp : 0.f;  // summed over the tile's rows below
  }
  tsum = wave_sum(tsum);
  if ((t & 63) == 0) red[t >> 6] = tsum;
  __syncthreads();
  if (t == 0) {
    const float total = ((red[0] + red[1]) + red[2]) + red[3];
    dT_part[(int64_t)blockIdx.x * H + h] = PLUS ? total : -total * inv_temp_h;
  }

  if (vec_s) {
    const int units = S / UE;
    for (int i = t; i < rows * units; i += 256) {
      const int r = i / units, u = i - r * units;
      alignas(16) T o[UE];
#pragma unroll
      for (int j = 0; j < UE; ++j) store_from_f32(o + j, dwl[r * S1 + u * UE + j]);
      *reinterpret_cast<u32x4 *>(d_z + (m0 + r) * HS + h * S + u * UE) = *reinterpret_cast<const u32x4 *>(o);
      if constexpr (PLUS) {
#pragma unroll
        for (int j = 0; j < UE; ++j) store_from_f32(o + j, a1l[r * S1 + u * UE + j]);
        *reinterpret_cast<u32x4 *>(static_cast<T *>(plus.d_a1) + (m0 + r) * HS + h * S + u * UE) =
            *reinterpret_cast<const u32x4 *>(o);
      }
    }
  } else {
    for (int i = t; i < rows * S; i += 256) {
      const int r = i / S, s = i - r * S;
      store_from_f32(d_z + (m0 + r) * HS + h * S + s, dwl[r * S1 + s]);
      if constexpr (PLUS)
        store_from_f32(static_cast<T *>(plus.d_a1) + (m0 + r) * HS + h * S + s, a1l[r * S1 + s]);
    }
  }
  // d x_mid and d fx_mid: a thread owns 2 rows x 2 features (features dq and dq + DQ), 8 LDS reads per 8 multiply-adds
  const int DQ = (D + 1) >> 1;
  for (int tile = t; tile < (R >> 1) * DQ; tile += 256) {
    const int rp = tile / DQ, dq = tile - rp * DQ, r0 = 2 * rp;
    const int d0 = dq, d1 = min(dq + DQ, D - 1);
    const float *wr = wl + r0 * S1, *zr = dwl + r0 * S1;
    float dx[2][2] = {{0.f, 0.f}, {0.f, 0.f}}, df[2][2] = {{0.f, 0.f}, {0.f, 0.f}};
    for (int sl = 0; sl < S; ++sl) {
      const float za = zr[sl], zb = zr[S1 + sl], wa = wr[sl], wb = wr[S1 + sl];
      const float w0 = ws[sl * D1 + d0], w1v = ws[sl * D1 + d1], n0 = dn[sl * D1 + d0], n1 = dn[sl * D1 + d1];
      dx[0][0] = fmaf(za, w0, dx[0][0]);
      dx[0][1] = fmaf(za, w1v, dx[0][1]);
      dx[1][0] = fmaf(zb, w0, dx[1][0]);
      dx[1][1] = fmaf(zb, w1v, dx[1][1]);
      df[0][0] = fmaf(wa, n0, df[0][0]);
      df[0][1] = fmaf(wa, n1, df[0][1]);
      df[1][0] = fmaf(wb, n0, df[1][0]);
      df[1][1] = fmaf(wb, n1, df[1][1]);
    }
    if constexpr (PLUS) {
      const float *ar = a1l + r0 * S1;
      for (int sl = 0; sl < S; ++sl) {
        const float aa = ar[sl], ab = ar[S1 + sl], v0 = w1[sl * D1 + d0], v1 = w1[sl * D1 + d1];
        dx[0][0] = fmaf(aa, v0, dx[0][0]);
        dx[0][1] = fmaf(aa, v1, dx[0][1]);
        dx[1][0] = fmaf(ab, v0, dx[1][0]);
        dx[1][1] = fmaf(ab, v1, dx[1][1]);
      }
    }
#pragma unroll
    for (int jj = 0; jj < 2; ++jj) {
      const int r = r0 + jj;
      if (r >= rows) continue;
#pragma unroll
      for (int k = 0; k < 2; ++k) {
        const int d = dq + k * DQ;
        if (d >= D) continue;
        if (vec_d) {  // xm / fm are free since the first phase: the results leave through them as 16-byte stores
          xm[r * D1 + d] = PLUS ? dx[jj][k] + df[jj][k] : dx[jj][k];
          fm[r * D1 + d] = df[jj][k];
        } else if constexpr (PLUS) {
          store_from_f32(d_proj + (m0 + r) * HD + h * D + d, dx[jj][k] + df[jj][k]);
        } else {
          store_from_f32(d_proj + (m0 + r) * 2 * HD + h * D + d, dx[jj][k]);
          store_from_f32(d_proj + (m0 + r) * 2 * HD + HD + h * D + d, df[jj][k]);
        }
      }
    }
  }
  if (vec_d) {
    __syncthreads();
    const int units = D / UE;
    for (int i = t; i < rows * units; i += 256) {
      const int r = i / units, u = i - r * units;
      alignas(16) T o[UE];
#pragma unroll
      for (int j = 0; j < UE; ++j) store_from_f32(o + j, xm[r * D1 + u * UE + j]);
      T *dst = d_proj + (m0 + r) * (PLUS ? HD : 2 * HD) + h * D + u * UE;
      *reinterpret_cast<u32x4 *>(dst) = *reinterpret_cast<const u32x4 *>(o);
      if constexpr (!PLUS) {
#pragma unroll
        for (int j = 0; j < UE; ++j) store_from_f32(o + j, fm[r * D1 + u * UE + j]);
        *reinterpret_cast<u32x4 *>(dst + HD) = *reinterpret_cast<const u32x4 *>(o);
      }
    }
  }
}

// ================================================================================================
// host launchers
// ================================================================================================
size_t attention_lds_bytes(const pa_shape &s) {
  return (size_t)(7 * s.S * (s.D + 1) + (kAttnBwdThreads / 64) * 2 * s.S) * 4;
}

int slice_attention(const pa_shape &s, const pa_params &p, const float *slice_token, const float *slice_norm,
                    const float *d_out_token, float *scratch, float *d_num, float *d_norm, float *d_wqkv_part,
                    hipStream_t st) {
  const size_t lds = attention_lds_bytes(s);
  int rc = allow_dynamic_lds(slice_attention_backward_kernel, lds);
  if (rc) return rc;
  hipLaunchKernelGGL(slice_attention_backward_kernel, dim3((unsigned)(s.B * s.H)), dim3(kAttnBwdThreads), lds, st,
                     slice_token, slice_norm, p.qkv_project_weight, d_out_token, scratch, d_num, d_norm, d_wqkv_part,
                     (int)s.D, (int)s.S);
  return launch_status();
}

// Rows per tile of slice_softmax_backward_kernel: the largest power of two <= 32 whose LDS footprint fits; 0 = none.
static size_t point_tile_lds(const pa_shape &s, int R, bool plus) {
  size_t words = (size_t)(3 * s.S * (s.D + 1) + 2 * s.S) + (size_t)R * (3 * (s.D + 1) + 3 * (s.S + 1));
  if (plus) words += (size_t)(s.S * (s.D + 1) + 2 * s.S) + (size_t)R * (s.S + 1);
  return words * 4;
}

int point_tile_rows(const pa_shape &s, bool plus) {
  for (int R = 32; R >= 4; R >>= 1)
    if (point_tile_lds(s, R, plus) <= 120 * 1024) return R;
  return 0;
}

int64_t point_tiles(const pa_shape &s, bool plus) {
  const int R = point_tile_rows(s, plus);
  return R == 0 ? 0 : s.B * ((s.N + R - 1) / R);
}

template <typename T, bool PLUS>
static int slice_softmax_t(const pa_shape &s, const pa_params &p, const void *x_mid, const void *fx_mid, const void *w,
                           const void *d_out_x, const float *out_token, const float *d_num, const float *d_norm,
                           void *d_proj, void *d_z, float *dT_part, const PlusArgs &plus, hipStream_t st) {
  const int R = point_tile_rows(s, PLUS);
  if (R == 0) return PA_ERR_UNSUPPORTED;
  const size_t lds = point_tile_lds(s, R, PLUS);
  int rc = allow_dynamic_lds(slice_softmax_backward_kernel<T, PLUS>, lds);
  if (rc) return rc;
  const int tiles = (int)((s.N + R - 1) / R);
  dim3 grid((unsigned)(tiles * s.B), (unsigned)s.H);
  hipLaunchKernelGGL((slice_softmax_backward_kernel<T, PLUS>), grid, dim3(256), lds, st, static_cast<const T *>(x_mid),
                     static_cast<const T *>(fx_mid), static_cast<const T *>(w), static_cast<const T *>(d_out_x),
                     out_token, d_num, d_norm, p.in_project_slice_weight, p.in_project_slice_bias, p.temperature,
                     static_cast<T *>(d_proj), static_cast<T *>(d_z), dT_part, s.N, (int)s.H, (int)s.D, (int)s.S, R,
                     tiles, plus);
  return launch_status();
}

int slice_softmax(int dtype, const pa_shape &s, const pa_params &p, const void *x_mid, const void *fx_mid,
                  const void *w, const void *d_out_x, const float *out_token, const float *d_num, const float *d_norm,
                  void *d_proj, void *d_z, float *dT_part, hipStream_t st) {
  const PlusArgs none{};
  return dtype == PA_F32 ? slice_softmax_t<float, false>(s, p, x_mid, fx_mid, w, d_out_x, out_token, d_num, d_norm,
                                                         d_proj, d_z, dT_part, none, st)
                         : slice_softmax_t<bf16, false>(s, p, x_mid, fx_mid, w, d_out_x, out_token, d_num, d_norm,
                                                        d_proj, d_z, dT_part, none, st);
}

int slice_softmax_plus(int dtype, const pa_shape &s, const pa_params &p, const pa_plus_params &pp, const void *x_mid,
                       const void *uniform, const void *w, const void *d_out_x, const float *out_token,
                       const float *d_num, const float *d_norm, void *d_x_mid, void *d_z, void *d_a1, float *d_a2,
                       float *dT_part, hipStream_t st) {
  const PlusArgs plus{uniform, pp.proj_temperature_0_weight, pp.proj_temperature_0_bias, pp.proj_temperature_2_weight,
                      pp.proj_temperature_2_bias, d_a1, d_a2};
  return dtype == PA_F32 ? slice_softmax_t<float, true>(s, p, x_mid, x_mid, w, d_out_x, out_token, d_num, d_norm,
                                                        d_x_mid, d_z, dT_part, plus, st)
                         : slice_softmax_t<bf16, true>(s, p, x_mid, x_mid, w, d_out_x, out_token, d_num, d_norm,
                                                       d_x_mid, d_z, dT_part, plus, st);
}

}  // namespace backward
}  // namespace pa
