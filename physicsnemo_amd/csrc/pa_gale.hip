// GALE (geometry-aware latent embeddings) slice-token stage: cross-attention of the slice tokens to a context and
// the blend with the slice self-attention output (physicsnemo/nn/module/gale.py:87-145 and :43-84).  Everything else of a GALE
// layer (projections, slice softmax, aggregation, slice self-attention, deslice + out_linear) is the PhysicsAttention
// layer's own kernels; this stage sits between the slice self-attention and the deslice.
//
// Workgroups (batch * head, blocks of 16 slice tokens), operands and weights in LDS (every workgroup forms k and v of
// its (batch, head) itself); fp32 arithmetic on the vector ALUs (the stage is S x D work, independent of the
// number of points):
//   q = tok Wq^T + bq (S x D);  k = ctx Wk^T + bk,  v = ctx Wv^T + bv (Sc x D)
//   cross = softmax(q k^T / sqrt(D)) v
//   weighted:        out = sigmoid(m) self + (1 - sigmoid(m)) cross
//   concat_project:  out = gelu([self | cross] Wc^T + bc)
// The result goes out as float32 (B,H,S,D) and, optionally, as the bf16 operands of the MFMA deslice kernel.
#include "pa_common.h"
#include "pa_host.h"

namespace pa {
namespace gale {

constexpr int kThreads = 256;
constexpr int kQueryBlock = 16;  // slice tokens per workgroup: grid.y = ceil(S / 16) workgroups share a (batch, head)

__global__ __launch_bounds__(kThreads) void slice_cross_mix_kernel(
    const float *__restrict__ slice_token, const float *__restrict__ self_token, const float *__restrict__ context,
    pa_gale_params gp, float *__restrict__ out_token, uint16_t *__restrict__ tokp, int S, int D, int Sc, int Dc) {
  extern __shared__ float lds[];
  const int D1 = D + 1, Dc1 = Dc + 1;
  float *tok = lds;               // S * D1, later: cross
  float *ctx = tok + S * D1;      // Sc * Dc1
  float *q = ctx + Sc * Dc1;      // S * D1
  float *k = q + S * D1;          // Sc * D1
  float *v = k + Sc * D1;         // Sc * D1
  float *prow = v + Sc * D1;      // (kThreads / 64) * Sc
  float *wq = prow + (kThreads / 64) * Sc;  // D * D1   cross_q weight rows
  float *wk = wq + D * D1;                  // D * Dc1  cross_k weight rows
  float *wv = wk + D * Dc1;                 // D * Dc1  cross_v weight rows
  float *wc = wv + D * Dc1;                 // D * (2D + 1)  concat_project weight rows (that blend mode only)
  const int t = threadIdx.x, wave = t >> 6, lane = t & 63;
  const int64_t bh = blockIdx.x;
  const int s0 = blockIdx.y * kQueryBlock, s1 = min(S, s0 + kQueryBlock);  // this workgroup's slice tokens
  const float *tk = slice_token + bh * S * D;
  const float *cx = context + bh * Sc * Dc;

  for (int i = t; i < S * D; i += kThreads) tok[(i / D) * D1 + (i % D)] = tk[i];
  for (int i = t; i < Sc * Dc; i += kThreads) ctx[(i / Dc) * Dc1 + (i % Dc)] = cx[i];
  // the three weights go through LDS: read from global memory inside the dot products, every term waits for its load
  for (int i = t; i < D * D; i += kThreads) wq[(i / D) * D1 + (i % D)] = gp.cross_q_weight[i];
  for (int i = t; i < D * Dc; i += kThreads) {
    wk[(i / Dc) * Dc1 + (i % Dc)] = gp.cross_k_weight[i];
    wv[(i / Dc) * Dc1 + (i % Dc)] = gp.cross_v_weight[i];
  }
  if (!gp.state_mixing)
    for (int i = t; i < D * 2 * D; i += kThreads) wc[(i / (2 * D)) * (2 * D + 1) + (i % (2 * D))] = gp.concat_project_weight[i];
  __syncthreads();
  for (int i = s0 * D + t; i < s1 * D; i += kThreads) {
    const int s = i / D, e = i - s * D;
    const float *wr = wq + e * D1;
    float acc = gp.cross_q_bias[e];
    for (int d = 0; d < D; ++d) acc = fmaf(tok[s * D1 + d], wr[d], acc);
    q[s * D1 + e] = acc;
  }
  for (int i = t; i < Sc * D; i += kThreads) {
    const int u = i / D, e = i - u * D;
    const float *wkr = wk + e * Dc1, *wvr = wv + e * Dc1;
    float ak = gp.cross_k_bias[e], av = gp.cross_v_bias[e];
    for (int c = 0; c < Dc; ++c) {
      ak = fmaf(ctx[u * Dc1 + c], wkr[c], ak);
      av = fmaf(ctx[u * Dc1 + c], wvr[c], av);
    }
    k[u * D1 + e] = ak;
    v[u * D1 + e] = av;
  }
  __syncthreads();  // tok is dead from here on: its rows receive the cross-attention output

  const float scale = rsqrtf((float)D);
  float *pr = prow + wave * Sc;
  for (int s = s0 + wave; s < s1; s += kThreads / 64) {
    const float *qs = q + s * D1;
    float mx = -INFINITY;
    for (int u = lane; u < Sc; u += 64) {
      float acc = 0.f;
      for (int e = 0; e < D; ++e) acc = fmaf(qs[e], k[u * D1 + e], acc);
      acc *= scale;
      pr[u] = acc;
      mx = fmaxf(mx, acc);
    }
    mx = wave_max(mx);
    float sum = 0.f;
    for (int u = lane; u < Sc; u += 64) {
      const float e = expf(pr[u] - mx);
      pr[u] = e;
      sum += e;
    }
    sum = wave_sum(sum);
    const float inv = 1.f / sum;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    for (int e = lane; e < D; e += 64) {
      float acc = 0.f;
      for (int u = 0; u < Sc; ++u) acc = fmaf(pr[u], v[u * D1 + e], acc);
      tok[s * D1 + e] = acc * inv;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
  __syncthreads();

  const float *sf = self_token + bh * S * D;
  float mixw = 0.f;
  if (gp.state_mixing) mixw = 1.f / (1.f + expf(-gp.state_mixing[0]));
  const int NCH = S / 16;
  for (int i = s0 * D + t; i < s1 * D; i += kThreads) {
    const int s = i / D, e = i - s * D;
    float o;
    if (gp.state_mixing) {
      o = mixw * sf[i] + (1.f - mixw) * tok[s * D1 + e];
    } else {
      const float *wr = wc + e * (2 * D + 1);
      float acc = gp.concat_project_bias[e];
      for (int d = 0; d < D; ++d) acc = fmaf(sf[s * D + d], wr[d], acc);
      for (int d = 0; d < D; ++d) acc = fmaf(tok[s * D1 + d], wr[D + d], acc);
      o = gelu_erf(acc);
    }
    out_token[bh * S * D + i] = o;
    if (tokp) {  // operand order of the MFMA deslice product (D = 32): chunk of 16 slices, lane = 32 g' + d, element j
      const int cq = s >> 4, ss = s & 15, gq = (ss >> 2) & 1, j = 4 * (ss >> 3) + (ss & 3);
      tokp[(((bh * NCH + cq) * 64 + 32 * gq + e) * 8) + j] = f32_to_bf16_bits(o);
    }
  }
}

// out_token (B,H,S,32) float32 -> the bf16 operands of the MFMA deslice kernel (same order as above)
__global__ __launch_bounds__(kThreads) void pack_tokens_kernel(const float *__restrict__ out_token,
                                                               uint16_t *__restrict__ tokp, int S) {
  const int64_t bh = blockIdx.x;
  const int NCH = S / 16;
  for (int i = threadIdx.x; i < S * 32; i += kThreads) {
    const int s = i >> 5, e = i & 31;
    const int cq = s >> 4, ss = s & 15, gq = (ss >> 2) & 1, j = 4 * (ss >> 3) + (ss & 3);
    tokp[(((bh * NCH + cq) * 64 + 32 * gq + e) * 8) + j] = f32_to_bf16_bits(out_token[bh * S * 32 + i]);
  }
}

int pack_tokens(const pa_shape &s, const float *out_token, void *tokp, hipStream_t st) {
  hipLaunchKernelGGL(pack_tokens_kernel, dim3((unsigned)(s.B * s.H)), dim3(kThreads), 0, st, out_token,
                     static_cast<uint16_t *>(tokp), (int)s.S);
  return launch_status();
}

size_t lds_bytes(const pa_shape &s, int64_t Sc, int64_t Dc) {
  return (size_t)(2 * s.S * (s.D + 1) + Sc * (Dc + 1) + 2 * Sc * (s.D + 1) + (kThreads / 64) * Sc +
                  s.D * (s.D + 1) + 2 * s.D * (Dc + 1) + s.D * (2 * s.D + 1)) * 4;
}

int slice_cross_mix(const pa_shape &s, const pa_gale_params &gp, int64_t Sc, int64_t Dc, const float *slice_token,
                    const float *self_token, const float *context, float *out_token, void *tokp, hipStream_t st) {
  const size_t lds = lds_bytes(s, Sc, Dc);
  int rc = allow_dynamic_lds(slice_cross_mix_kernel, lds);
  if (rc) return rc;
  hipLaunchKernelGGL(slice_cross_mix_kernel, dim3((unsigned)(s.B * s.H), (unsigned)((s.S + kQueryBlock - 1) / kQueryBlock)),
                     dim3(kThreads), lds, st, slice_token,
                     self_token, context, gp, out_token, static_cast<uint16_t *>(tokp), (int)s.S, (int)s.D, (int)Sc,
                     (int)Dc);
  return launch_status();
}

}  // namespace gale
}  // namespace pa
