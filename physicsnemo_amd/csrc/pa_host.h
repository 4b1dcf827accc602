// Host-side declarations shared by the kernel translation units and the C ABI.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/physattn.h"

namespace pa {

constexpr size_t kMaxLdsBytes = 160 * 1024;  // LDS per workgroup on gfx950

// result of the launch just enqueued, as a C-ABI return code
inline int launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? PA_OK : (int)e;
}

// opt a kernel in to more than the default 48 KiB of dynamic LDS
// (the attribute is per kernel and per device: remembered for the device it was last set on, so the steady state of a
// process that stays on one GPU makes no runtime call here)
template <typename F>
inline int allow_dynamic_lds(F kernel, size_t bytes) {
  if (bytes > kMaxLdsBytes) return PA_ERR_UNSUPPORTED;
  if (bytes > 48 * 1024) {
    static thread_local const void *last_kernel = nullptr;
    static thread_local size_t last_bytes = 0;
    static thread_local int last_dev = -1;
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess) dev = -1;
    const void *k = reinterpret_cast<const void *>(kernel);
    if (k == last_kernel && bytes <= last_bytes && dev == last_dev && dev >= 0) return PA_OK;
    hipError_t e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e != hipSuccess) return (int)e;
    last_kernel = k;
    last_bytes = bytes;
    last_dev = dev;
  }
  return PA_OK;
}

// Arguments of the row GEMMs: out[m, o] = bias[o] + sum_k A(m, k) * W[o, k]
//   linear: A(m, k) = in[m*K + k]
//   conv  : K = taps*C, k = tap*C + c; 2-D: taps = ks^2, tap = u*ks + v, A(m,k) = in[b, (i+u-p)*gw + (j+v-p), c];
//           3-D: taps = ks^3, tap = (u*ks + v)*ks + z, A(m,k) = in[b, ((i+u-p)*gw + (j+v-p))*gd + (l+z-p), c];
//           0 outside the grid; the PyTorch weight element is W[o, c, u, v(, z)] = W[o*K + c*taps + tap].
// Up to two (W, bias, out) sets share the same input (x_mid and fx_mid), selected by blockIdx.z.
struct GemmArgs {
  const void *in;
  const void *w[2];
  const float *bias[2];
  void *out[2];
  int64_t M;   // rows = B*N
  int K, O;    // reduction length, output columns
  int C, N, gh, gw, ks;  // conv geometry (ks = 0: linear)
  int gd;                // depth of a 3-D grid (0: 2-D)
  int w_tap_major;       // conv weights as (O, taps, C) (= the reduction order k = tap * C + c) instead of (O, C, taps)
  // MFMA kernel only, bf16, Linear, O = 32 * pack_heads: pack_tpb > 0 walks the rows batch by batch in tiles of 32
  // points (pack_tpb tiles per batch, the last one padded) and also writes each (tile, head) block of the result in
  // the packed operand layout of the MFMA slice kernels (fx_pack).  out[z] may then be NULL.
  void *out_pack[2];
  int pack_tpb, pack_heads;
  int act;  // applied to out (not to out_pack): 0 none, 1 GELU in its erf form (torch.nn.GELU default)
};

namespace gemm {
// MFMA row GEMM (fp32: v_mfma_f32_32x32x2_f32, bf16: v_mfma_f32_32x32x16_bf16); `serves` tells whether the shape and
// the pointers meet its 16-byte granularity, otherwise the scalar kernel of the general family runs.
bool serves(const GemmArgs &a, int nsets, size_t elem_bytes);
int launch(const GemmArgs &a, int nsets, int dtype, hipStream_t st);
// weight-gradient products over the row axis: partials[g][oa][ob] = sum over chunk g of A[m][oa] * B[m][ob] (bf16 in)
int64_t cols_gemm_chunks(int64_t M, int64_t OA, int num_cu);
int cols_gemm(const void *A, int64_t lda, int64_t OA, const void *B, int64_t ldb, int64_t OB, int64_t M,
              float *partials, float *col_sums, int num_cu, hipStream_t st);
// the same for float32 operands (fp32 MFMA)
int64_t cols_gemm_f32_chunks(int64_t M, int64_t OA, int64_t OB, int num_cu);
int cols_gemm_f32(const void *A, int64_t lda, int64_t OA, const void *B, int64_t ldb, int64_t OB, int64_t M,
                  float *partials, float *col_sums, int num_cu, hipStream_t st);
}  // namespace gemm

namespace general {
int dequant_e4m3(const void *in, const float *scale, void *out, int64_t rows, int64_t cols, hipStream_t st);
int project_inputs(int dtype, const pa_shape &s, const pa_params &p, const void *x, void *x_mid, void *fx_mid,
                   hipStream_t st);
int out_linear(int dtype, const pa_shape &s, const pa_params &p, const void *out_x, void *y, hipStream_t st);
int rows_gemm(int dtype, const pa_shape &grid, int64_t c_in, int64_t c_out, const void *in, const void *weight,
              const float *bias, int act, void *out, hipStream_t st);
int rows_gemm_packed(const pa_shape &s, int64_t c_in, const void *in, const void *weight, const float *bias, void *out,
                     void *out_pack, hipStream_t st);
int slice_softmax(int dtype, const pa_shape &s, const pa_params &p, const void *x_mid, void *w, hipStream_t st);
int slice_softmax_plus(int dtype, const pa_shape &s, const pa_params &p, const pa_plus_params &pp, const void *x_mid,
                       const void *uniform, void *w, void *scratch, hipStream_t st);
int64_t partial_count(const pa_shape &s);
size_t combine_attn_lds_bytes(const pa_shape &s);
int slice_partial(int dtype, const pa_shape &s, const void *w, const void *fx_mid, float *partials, hipStream_t st);
int combine_partials(const pa_shape &s, const float *partials, int64_t G, const float **combined, hipStream_t st);
int combine_attention(const pa_shape &s, const pa_params &p, const float *partials, int64_t G, float *slice_token,
                      float *slice_norm, float *out_token, hipStream_t st);
int deslice(int dtype, const pa_shape &s, const void *w, const float *out_token, void *out_x, hipStream_t st);
int residual_ln(int dtype, const pa_shape &s, void *y, const pa_block_tail &tail, hipStream_t st);
int64_t layernorm_backward_groups(int64_t rows);
int layernorm_backward(int dtype, int64_t rows, int64_t C, const void *x, const void *dy, const float *gamma, float eps,
                       void *dx, float *partials, hipStream_t st);
}  // namespace general

namespace conv {
// float32 structured 2-D front end (C = 128, 8 heads of 16, 32 slices): both convolutions on split-bf16 MFMA products,
// slice softmax and partial token sums in one launch.  `w`: (B, N, H, S) float32; `partials`: groups(s) partials of
// B * H * S * (D + 1) floats each, in the layout the general combine kernels read.
bool supported(int dtype, const pa_shape &s);
int64_t groups(const pa_shape &s);
int64_t blob_bytes(const pa_shape &s);
// blob_out (may be NULL): f32rows::backend_blob_bytes() that receive out_linear's weight in the form f32rows::backend
// reads, cut by the same launch that cuts the convolution weights
// (with mlp: f32rows::block_blob_bytes(mlp->F), and the block MLP's weights behind it, as f32rows::block_tail reads)
int front(const pa_shape &s, const pa_params &p, const void *x, void *blob, void *w, float *partials, void *blob_out,
          const pa_block_mlp *mlp, hipStream_t st);
}  // namespace conv

namespace f32rows {
// float32 per-point kernels of a 128-wide block on split-bf16 products.  backend: out_x = w . out_token per head
// (8 heads of 16, 32 slices; w (B, N, H, S), out_token (B, H, S, D)), y = out_x W_out^T + b_out and the tail, one
// launch; blob: backend_blob_bytes() of scratch for the repacked W_out.  mlp_*: Mlp(128 -> F -> 128), F a multiple of
// 128, with the same tail; blob: mlp_blob_bytes(F) written by mlp_pack.
bool backend_supported(int dtype, const pa_shape &s);
int64_t backend_blob_bytes();
int backend(const pa_shape &s, const pa_params &p, const void *w, const float *out_token, void *y,
            const pa_block_tail *tail, void *blob, bool blob_ready, hipStream_t st);
bool mlp_supported(int dtype, int64_t rows, int64_t C, int64_t F);
int64_t mlp_blob_bytes(int64_t F);
int mlp_pack(int64_t F, const void *w1, const void *w2, void *blob, hipStream_t st);
int mlp_forward(int64_t rows, int64_t F, const void *blob, const float *b1, const float *b2, const void *u, void *y,
                const pa_block_tail *tail, hipStream_t st);
// the whole per-point tail of a block in one launch: hand-back, out_linear, + fx_in, LayerNorm, Mlp, + residual, next
// LayerNorm (see pa_block_forward); blob: block_blob_bytes(F) of scratch
bool block_supported(int dtype, const pa_shape &s, int64_t F);
int64_t block_blob_bytes(int64_t F);
int block_tail(const pa_shape &s, const pa_params &p, const pa_block_mlp &m, const void *w, const float *out_token,
               const void *fx_in, void *fx_out, const pa_block_tail *next, const pa_block_head *head, void *blob,
               bool blob_ready, hipStream_t st);
// the model's preprocess Mlp, Linear(c_in -> F) -> GELU -> Linear(F -> 128), c_in <= 8, with the tail (the first
// LayerNorm); blob: premlp_blob_bytes(F) of scratch
bool premlp_supported(int dtype, int64_t rows, int64_t c_in, int64_t F, int64_t C);
int64_t premlp_blob_bytes(int64_t F);
int premlp_forward(int64_t rows, int64_t c_in, int64_t F, const void *w1, const float *b1, const void *w2,
                   const float *b2, const void *u, void *y, const pa_block_tail *tail, void *blob, hipStream_t st);
}  // namespace f32rows

namespace backward {
size_t attention_lds_bytes(const pa_shape &s);
int slice_attention(const pa_shape &s, const pa_params &p, const float *slice_token, const float *slice_norm,
                    const float *d_out_token, float *scratch, float *d_num, float *d_norm, float *d_wqkv_part,
                    hipStream_t st);
int point_tile_rows(const pa_shape &s, bool plus = false);  // plus: the Transolver++ form of the per-point kernel
int64_t point_tiles(const pa_shape &s, bool plus = false);
int slice_softmax(int dtype, const pa_shape &s, const pa_params &p, const void *x_mid, const void *fx_mid,
                  const void *w, const void *d_out_x, const float *out_token, const float *d_num, const float *d_norm,
                  void *d_proj, void *d_z, float *dT_part, hipStream_t st);
int slice_softmax_plus(int dtype, const pa_shape &s, const pa_params &p, const pa_plus_params &pp, const void *x_mid,
                       const void *uniform, const void *w, const void *d_out_x, const float *out_token,
                       const float *d_num, const float *d_norm, void *d_x_mid, void *d_z, void *d_a1, float *d_a2,
                       float *dT_part, hipStream_t st);
}  // namespace backward

namespace flare {
int64_t column_max_chunks(const pa_shape &s);
int column_weights(int dtype, const pa_shape &s, const void *a, float *partial, float *colmax, void *wc,
                   hipStream_t st);
// temperature: NULL, or (H) float32 -- the entries are then divided by clamp(temperature[head], 0.5, 5) first
int softmax_rows(int dtype, const pa_shape &s, void *a, const float *temperature, hipStream_t st);
int column_max(int dtype, const pa_shape &s, const void *a, float *partial, float *colmax, hipStream_t st);
// bf16 scores (B,N,H,S) -> exp(A - column max) and softmax_s(A) in the packed layout of the MFMA slice kernels
int pack_weights(const pa_shape &s, const void *scores, const float *colmax, void *wc_pack, void *wr_pack, int num_cu,
                 hipStream_t st);
int normalise(const pa_shape &s, const float *sums, float *z, hipStream_t st);
int backward_tile_rows(const pa_shape &s);
int backward_points(int dtype, const pa_shape &s, const void *wr, const void *wc, const void *v, const void *g,
                    const float *z, const float *d_num, const float *d_den, void *d_a, void *d_v, hipStream_t st);
}  // namespace flare

namespace gale {
size_t lds_bytes(const pa_shape &s, int64_t Sc, int64_t Dc);
int pack_tokens(const pa_shape &s, const float *out_token, void *tokp, hipStream_t st);
int slice_cross_mix(const pa_shape &s, const pa_gale_params &gp, int64_t Sc, int64_t Dc, const float *slice_token,
                    const float *self_token, const float *context, float *out_token, void *tokp, hipStream_t st);
}  // namespace gale

namespace ballquery {
int ball_query(int64_t B, int64_t Np, int64_t Nq, int64_t K, float radius, const float *points, const float *queries,
               int64_t *indices, float *out_points, float *out_dists, int32_t *counts, hipStream_t st);
int ball_query_cells(int64_t B, int64_t Np, int64_t Nq, int64_t K, float radius, int64_t G, const float *grid,
                     const float *sorted_points, const int32_t *sorted_index, const int32_t *cell_start,
                     const float *queries, const int32_t *query_order, int64_t *indices, float *out_points,
                     float *out_dists, int32_t *counts, hipStream_t st);
}  // namespace ballquery

namespace mfma {
bool staged_supported(int dtype, const pa_shape &s);
int slice_softmax_pack_plus(const pa_shape &s, const pa_params &p, const pa_plus_params &pp, const void *x_mid,
                            const void *uniform, void *w_pack, int num_cu, hipStream_t st);
int slice_softmax_pack(const pa_shape &s, const pa_params &p, const void *x_mid, void *w_pack, int num_cu,
                       hipStream_t st);
// the same weights recomputed where they are used, never stored: token sums (softmax_reduce_groups partials) and
// the hand-back to the points (out_x may be x_mid)
int64_t softmax_reduce_groups(const pa_shape &s, int num_cu);
// packed_x: x_mid (and out_x) are packed operand tiles [tile][head][2][64 lanes] of 16 bytes instead of rows
int slice_softmax_reduce(const pa_shape &s, const pa_params &p, const void *x_mid, bool packed_x, const void *fx_pack,
                         float *partials, int num_cu, hipStream_t st);
int deslice_recompute(const pa_shape &s, const pa_params &p, const void *x_mid, bool packed_x, const void *tokp,
                      void *out_x, int num_cu, hipStream_t st);
bool backward_supported(const pa_shape &s);
int64_t backward_groups(const pa_shape &s, int num_cu);
int64_t backward_tables_bytes(const pa_shape &s);
int deslice_natural(const pa_shape &s, const void *w_pack, const void *tokp, void *out_x, int num_cu, hipStream_t st);
int slice_softmax_backward(const pa_shape &s, const pa_params &p, const void *x_mid, const void *fx_mid,
                           const void *d_out_x, const void *w_pack, const float *out_token, const float *d_num,
                           const float *d_norm, void *tables, void *d_proj, void *d_z, float *dT_part, int num_cu,
                           hipStream_t st);
bool supported(int dtype, const pa_shape &s);
int64_t tiles_per_batch(const pa_shape &s);
int64_t reduce_groups(const pa_shape &s);
int64_t blob_bytes(const pa_shape &s);
int64_t fx_pack_bytes(const pa_shape &s);
int64_t w_pack_bytes(const pa_shape &s);
int64_t tokp_bytes(const pa_shape &s);
int pack_params(const pa_shape &s, const pa_params &p, void *blob, hipStream_t st);
int pack_out_linear(const pa_shape &s, const void *w_out, const float *w_scale, const float *b_out, void *blob,
                    hipStream_t st);
int64_t project_groups(const pa_shape &s, int num_cu, bool fused);
bool fuse_reduce(const pa_shape &s);
int project_softmax(const pa_shape &s, const void *blob, const void *x, void *fx_pack, void *w_pack, float *partials,
                    int num_cu, hipStream_t st);
// the fused form with the shader clock of one of its workgroups reported (C = 256, S <= 64): clock_out[0] = shader
// cycles, clock_out[1] = ticks of the 100 MHz wall clock
int project_softmax_clocked(const pa_shape &s, const void *blob, const void *x, void *w_pack, float *partials,
                            uint64_t *clock_out, int num_cu, hipStream_t st);
int slice_reduce(const pa_shape &s, const void *w_pack, const void *fx_pack, float *partials, hipStream_t st);
int combine_attention(const pa_shape &s, const pa_params &p, const float *fx_bias, const float *partials, int64_t G,
                      float *slice_token, float *slice_norm, float *out_token, void *tokp, hipStream_t st);
int deslice_project(const pa_shape &s, const void *blob, const void *w_pack, const void *tokp, void *y,
                    const pa_block_tail *tail, int num_cu, hipStream_t st);
// kernel (d) fed with x_mid tiles: the slice weights are recomputed per tile and never stored (S = 128)
bool deslice_recompute_project_supported(const pa_shape &s);
int deslice_recompute_project(const pa_shape &s, const pa_params &p, const void *blob, const void *xm_pack,
                              const void *tokp, void *y, const pa_block_tail *tail, int num_cu, hipStream_t st);
}  // namespace mfma

namespace mlp {
bool supported(int dtype, int64_t rows, int64_t C, int64_t F);
int64_t blob_bytes(int64_t C, int64_t F);
// w*_scale: nullptr for bf16 weights; else the weight is fp8-e4m3 bytes with one float32 scale per output row
int pack(int64_t C, int64_t F, const void *w1, const float *w1_scale, const void *w2, const float *w2_scale, void *blob,
         hipStream_t st);
// LayerNorm applied to the input rows on their way into the first product (gamma == nullptr: none)
struct InputLn {
  const float *gamma = nullptr, *beta = nullptr;
  float eps = 0.f;
};
bool input_ln_supported(int dtype, int64_t rows, int64_t C, int64_t F);
int forward(int64_t rows, int64_t C, int64_t F, const void *blob, const float *b1, const float *b2, const void *u,
            void *y, const pa_block_tail *tail, const InputLn &in, int num_cu, hipStream_t st);
// the preprocess MLP (c_in <= 16 inputs -> F -> C in {256, 512}) with the hidden layer kept on chip; bf16 rows and weights
bool premlp_supported(int dtype, int64_t rows, int64_t c_in, int64_t F, int64_t C);
int64_t premlp_blob_bytes(int64_t F, int64_t C);
int premlp(int64_t rows, int64_t c_in, int64_t F, int64_t C, const void *w1, const float *b1, const void *w2,
           const float *b2, const void *u, void *y, const float *ln_gamma, const float *ln_beta, float ln_eps,
           void *ln_out, void *blob, int num_cu, hipStream_t st);
// y = W x + bias [+ residual] [-> LayerNorm] for bf16 rows, W (C x C) bf16 row-major; blob: linear_blob_bytes(C) of scratch
bool linear_supported(int dtype, int64_t rows, int64_t C);
int64_t linear_blob_bytes(int64_t C);
int linear(int64_t rows, int64_t C, const void *w, const float *w_scale, const float *bias, const void *x, void *y,
           const pa_block_tail *tail, void *blob, int num_cu, hipStream_t st);
// the same with x as packed operand tiles [B tpb][C / 32][2][64 lanes] (k order kperm within a head)
int linear_packed(int64_t B, int64_t N, int64_t C, const void *w, const float *w_scale, const float *bias,
                  const void *x_pack, void *y, const pa_block_tail *tail, void *blob, int num_cu, hipStream_t st);
// the layer's two Linear input projections as packed operand tiles; blob: 2 linear_blob_bytes(C) of scratch
int project_packed(int64_t B, int64_t N, int64_t C, const void *w_x, const float *s_x, const float *b_x, const void *w_fx,
                   const float *s_fx, const float *b_fx, const void *x, void *xm_pack, void *fx_pack, void *blob,
                   int num_cu, hipStream_t st);
// the same for the k x k (x k) grid convolutions of the structured layers, as an implicit GEMM over taps x channels;
// blob: conv_project_blob_bytes(C, taps) of scratch
bool conv_project_supported(int dtype, int64_t B, int64_t N, int64_t C);
int64_t conv_project_blob_bytes(int64_t C, int64_t taps);
int conv_project_packed(int64_t B, int64_t N, int64_t C, int64_t gh, int64_t gw, int64_t gd, int64_t k, int tap_major,
                        const void *w_x, const float *b_x, const void *w_fx, const float *b_fx, const void *x,
                        void *xm_pack, void *fx_pack, void *blob, int num_cu, hipStream_t st);
}  // namespace mlp

}  // namespace pa
