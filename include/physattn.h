/*
 * physattn.h -- C ABI of libphysattn.so: the forward pass of Transolver's PhysicsAttention layer on
 * AMD MI355X (gfx950), hand-written HIP kernels.
 *
 * The reference implementation is pure Python (PyTorch ATen ops) and has no native interface; every
 * entry point below cites the reference code it replaces (paths relative to the reference checkout,
 * physicsnemo/nn/module/physics_attention.py is abbreviated PA.py, physicsnemo/models/transolver/
 * transolver.py is abbreviated TR.py).
 *
 * Conventions
 *   - Plain pointers and sizes only.  All tensor pointers are DEVICE pointers, 16-byte aligned,
 *     contiguous row-major (last index fastest) in the shapes stated.
 *   - Symbols: B batch, N points per batch, C = layer width `dim`, H heads, D dim_head, S slice_num.
 *   - `dtype` selects the ACTIVATION element type (x, intermediates, y) and the element type of the
 *     three large weights (in_project_x, in_project_fx, out_linear): PA_F32 or PA_BF16; PA_BF16_W8 = bf16
 *     activations with fp8-e4m3 large weights (see below).
 *     Small parameters are ALWAYS float32: every bias, temperature (H), in_project_slice weight (S,D)
 *     and bias (S), qkv_project weight (3D,D), LayerNorm gamma/beta.
 *     Slice tokens, slice norms and reduction partials are ALWAYS float32.
 *   - Ownership: the caller allocates every input, output and workspace.  The library never
 *     allocates, frees or keeps a pointer after the call returns.
 *   - Every call only enqueues work on `stream` (a hipStream_t passed as void*; NULL = the default
 *     stream); it never synchronises the host.  Calls are re-entrant.
 *   - Return value: 0 = success; negative = argument error (see PA_ERR_*), nothing was enqueued;
 *     positive = hipError_t reported by a launch.  Nothing throws or aborts across this boundary.
 */
#ifndef PHYSATTN_H
#define PHYSATTN_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PA_F32 0
#define PA_BF16 1
/* bf16 activations; the three large weights are fp8 e4m3 (OCP "fn": bias 7, no infinities, 0x7f/0xff = NaN) bytes
 * with one float32 scale per OUTPUT channel: W[o, :] = scale[o] * decode(byte[o, :]).  Irregular variant only.
 * On the MFMA paths the kernels that repack the weights into operand fragments read the e4m3 bytes themselves
 * (pa_mfma_pack_params, pa_mlp_pack_e4m3, the per-call repack of the 512-wide layers), so a call does the same
 * launches as with bf16 weights; other shapes expand the weights to bf16 in the workspace first.
 * No reference counterpart (the reference's only fp8 is Transformer Engine delayed scaling). */
#define PA_BF16_W8 2

#define PA_OK 0
#define PA_ERR_NULL (-1)        /* a required pointer is NULL */
#define PA_ERR_DIMS (-2)        /* a dimension is <= 0 or inconsistent */
#define PA_ERR_UNSUPPORTED (-3) /* shape/dtype outside what the kernels serve */
#define PA_ERR_ALIGN (-4)       /* a pointer is not 16-byte aligned */
#define PA_ERR_WORKSPACE (-5)   /* workspace too small */
#define PA_ERR_SCRATCH (-6)     /* the problem needs more than PA_STATIC_SCRATCH_BYTES of the library's static scratch */

/* Limits of the general kernels (PA_ERR_UNSUPPORTED beyond them). */
#define PA_MAX_D 128
#define PA_MAX_S 256
#define PA_MAX_N 2147483647ll /* points per batch element */
/* Limits of the entry points that take plain row / column counts instead of a shape struct, the column GEMMs
 * (PA_ERR_UNSUPPORTED beyond them): sizes are refused before any product of them is formed. */
#define PA_MAX_ROWS (1ll << 40)
#define PA_MAX_COLS (1ll << 24)

/* Library version (major*10000 + minor*100 + patch). No reference counterpart. */
int pa_version(void);

/* Measurement knob, no reference counterpart: the persistent kernels (one workgroup per compute unit walking the
 * tiles) size their grids by the device's compute-unit count; n > 0 makes them use n workgroups' worth instead, i.e.
 * run on n compute units with the rest of the chip idle; 0 restores the device's count.  Process-wide; set it before
 * sizing any workspace (partial-sum counts follow it).  bench.py uses it to show how the shader clock the chip holds
 * under a kernel depends on how much of the chip that kernel keeps busy. */
int pa_set_compute_units(int n);

/* 1 when marker ranges are on: the process environment held PA_ROCTX=1 when the library first looked and a roctx
 * library (librocprofiler-sdk-roctx / libroctx64) could be opened at run time; 0 otherwise.  With ranges on, the
 * layer-, block- and MLP-level entry points push a range named after themselves, and the fused layer brackets its
 * three stages with "_compute_slices_from_projections", "_compute_slice_attention_sdpa" and
 * "_project_attention_outputs" — the names of the reference's stages and of its record_function ranges
 * (physicsnemo/nn/module/physics_attention.py:358,445,490) — for `rocprofv3 --marker-trace`. */
int pa_markers_enabled(void);

/* Static text for a PA_ERR_* code (or "hip error" for positive codes). No reference counterpart. */
const char *pa_status_string(int code);

/* Dimensions of one layer call.  `conv_k` = 0 selects the irregular-mesh variant (nn.Linear
 * projections, PA.py:625-627); conv_k = k > 0 selects a structured variant (k x k Conv2d or k x k x k Conv3d,
 * stride 1, zero padding k/2, PA.py:740-742, :865-867): grid_d = 0 is the 2-D grid, N = grid_h*grid_w, token
 * n = i*grid_w + j (PA.py:772-783); grid_d > 0 the 3-D grid, N = grid_h*grid_w*grid_d, token
 * n = (i*grid_w + j)*grid_d + l (PA.py:896-907). */
typedef struct pa_shape {
  int64_t B, N, C, H, D, S;
  int64_t grid_h, grid_w, conv_k;
  int64_t grid_d;
  /* layout of convolution weights: 0 = as torch holds them, (c_out, c_in, k, k[, k]); 1 = tap-major,
   * (c_out, k, k[, k], c_in) -- the order of the implicit GEMM's reduction index, which lets the kernels fetch
   * weights with full-width loads (several times faster; the Python modules repack once per parameter set) */
  int64_t conv_tap_major;
} pa_shape;

/* Parameters of one layer, named as the reference state_dict keys (PA.py:285-327, :625-627, :740-742). */
typedef struct pa_params {
  const void *in_project_x_weight;   /* dtype, (H*D, C), (H*D, C, k, k) or (H*D, C, k, k, k) */
  const float *in_project_x_bias;    /* (H*D) */
  const void *in_project_fx_weight;  /* dtype, same shape */
  const float *in_project_fx_bias;   /* (H*D) */
  const float *in_project_slice_weight; /* (S, D), shared by all heads (PA.py:301,537) */
  const float *in_project_slice_bias;   /* (S) */
  const float *temperature;          /* (H); clamped to [0.5, 5] inside (PA.py:173) */
  const float *qkv_project_weight;   /* (3D, D), rows [q | k | v], no bias (PA.py:309,450) */
  const void *out_linear_weight;     /* dtype, (C, H*D) */
  const float *out_linear_bias;      /* (C) */
  /* PA_BF16_W8 only (NULL otherwise): per-output-channel scales of the fp8 weights */
  const float *in_project_x_scale;   /* (H*D) */
  const float *in_project_fx_scale;  /* (H*D) */
  const float *out_linear_scale;     /* (C) */
} pa_params;

/* Optional fused tail of the caller TransolverBlock.forward (TR.py:300-303):
 *   fx_new = y + residual;  ln_out = LayerNorm(fx_new; gamma, beta, eps)
 * All-NULL / zero = plain layer output. */
typedef struct pa_block_tail {
  const void *residual; /* dtype, (B, N, C) or NULL */
  const float *ln_gamma; /* (C) or NULL */
  const float *ln_beta;  /* (C) or NULL */
  float ln_eps;          /* torch default 1e-5 */
  void *ln_out;          /* dtype, (B, N, C) or NULL */
} pa_block_tail;

/* Bytes of caller-provided workspace pa_layer_forward needs for this shape. Negative = error code. */
int64_t pa_workspace_bytes(int dtype, const pa_shape *shape);

/* Which kernel family pa_layer_forward runs for this shape: 0 = general kernels, 1 = fused bf16 MFMA kernels
 * (C in {128, 256}), 2 = staged bf16 MFMA kernels (the same arithmetic as separate launches; adds C = 512, needs
 * B*N >= 4096).  The pa_mfma_* stage entry points serve the shapes with answer 1.  Negative = error code.
 * No reference counterpart. */
int pa_query_path(int dtype, const pa_shape *shape);

/* ---- stage-level entry points (natural layouts; general kernels) ------------------------------ */

/* Stage (a1): input projections, replaces project_input_onto_slices (PA.py:629-660 irregular,
 * :744-783 structured 2D) -> x_mid, fx_mid as (B, N, H*D) with channel c = h*D + d.  fx_mid == NULL: only x_mid is
 * computed and in_project_fx_* are not read (the single projection of plus=True, PA.py:652). */
int pa_project_inputs(int dtype, const pa_shape *shape, const pa_params *p, const void *x,
                      void *x_mid, void *fx_mid, void *stream);

/* Stage (a2): slice logits + temperature softmax, replaces in_project_slice (PA.py:537) and the
 * softmax half of _compute_slices_from_projections (PA.py:172-181): w (B, N, H, S), rows sum to 1. */
int pa_slice_softmax(int dtype, const pa_shape *shape, const pa_params *p, const void *x_mid, void *w,
                     void *stream);

/* Transolver++ (plus=True, PA.py:166-170, :287-295, :530-532): one projection (fx_mid = x_mid: call
 * pa_project_inputs with in_project_fx_* and fx_mid NULL and pass x_mid as fx_mid to the later stages), a learned
 * per-point temperature  max(temperature[h] + proj_temperature(x_mid[n,h,:]), 0.01)  with
 * proj_temperature = Linear(D,S) -> GELU -> Linear(S,1) -> GELU, and Gumbel noise added to the slice logits before
 * the division (physicsnemo/nn/module/gumbel_softmax.py:49-57).  All four tensors float32. */
typedef struct pa_plus_params {
  const float *proj_temperature_0_weight; /* (S, D) */
  const float *proj_temperature_0_bias;   /* (S) */
  const float *proj_temperature_2_weight; /* (1, S) */
  const float *proj_temperature_2_bias;   /* (1) */
} pa_plus_params;

/* Stage (a2) of Transolver++: replaces in_project_slice (PA.py:537) and the plus branch of
 * _compute_slices_from_projections (PA.py:166-170).  `uniform` (B,N,H,S), activation dtype: the U[0,1) samples the
 * reference draws with torch.rand_like(logits); the kernel forms the noise -log(-log(u + 1e-8) + 1e-8) itself.
 * `scratch`: NULL, or B*N*H*S elements of the activation dtype; with it the two Linears over the (point, head) rows run
 * on the row GEMM kernels (several times faster) and only the per-row part is left to a row kernel. */
int pa_slice_softmax_plus(int dtype, const pa_shape *shape, const pa_params *p, const pa_plus_params *plus,
                          const void *x_mid, const void *uniform, void *w, void *scratch, void *stream);

/* Stage (b): slice-token aggregation, replaces PA.py:185-203.
 *   partials: float32 scratch of pa_reduce_partial_count(shape) * B*H*S*(D+1) elements (per-chunk sums
 *             plus one slot for their total)
 *   slice_token (B,H,S,D) = (sum_n w fx_mid) / (sum_n w + 1e-2);  slice_norm (B,H,S) = sum_n w + 1e-2.
 * Two passes: per-chunk partial sums, then a fixed-order combine (bit-reproducible, no atomics). */
int64_t pa_reduce_partial_count(const pa_shape *shape);
int pa_slice_reduce(int dtype, const pa_shape *shape, const void *w, const void *fx_mid, float *partials,
                    float *slice_token, float *slice_norm, void *stream);

/* Stage (b) without any device allocation and without a workspace argument.  No counterpart in the reference: it is
 * for callers that cannot allocate device memory -- code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc.  Same kernels, same arguments and bit-identical results as pa_slice_reduce; the per-chunk
 * partial sums live in a static device array of PA_STATIC_SCRATCH_BYTES that every GPU the library runs on holds
 * until the process ends.  PA_ERR_SCRATCH if (pa_reduce_partial_count(shape) + 1) * B*H*S*(D+1) * 4 bytes exceed it
 * (one slot per chunk and one for their fixed-order total).
 * Calls on one GPU share that GPU's array: calls that overlap in time on the same GPU race on it (calls on one
 * stream, or otherwise ordered, are safe).  Only `shape`'s B, N, H, D, S are read. */
#define PA_STATIC_SCRATCH_BYTES (64ll << 20)
int64_t pa_static_scratch_bytes(void);
int pa_slice_reduce_static(int dtype, const pa_shape *shape, const void *w, const void *fx_mid, float *slice_token,
                           float *slice_norm, void *stream);

/* Stage (c): self-attention among the S slice tokens of each (batch, head), replaces
 * _compute_slice_attention_sdpa (PA.py:429-465): softmax(q k^T / sqrt(D)) v, float32, LDS resident. */
int pa_slice_attention(const pa_shape *shape, const pa_params *p, const float *slice_token,
                       float *out_slice_token, void *stream);

/* Stage (d): deslice + out_linear (+ optional residual / LayerNorm tail), replaces
 * _project_attention_outputs (PA.py:467-499) and TR.py:300-303.
 *   scratch: dtype, (B, N, H*D) caller-provided. tail may be NULL. */
int pa_deslice_project(int dtype, const pa_shape *shape, const pa_params *p, const void *w,
                       const float *out_slice_token, void *scratch, void *y, const pa_block_tail *tail,
                       void *stream);
/* The deslice alone (PA.py:492-495): out_x (B,N,H*D) = sum_s w[n,h,s] out_slice_token[h,s,:], heads merged; used where
 * something other than out_linear follows (GALE_FA blends two such results first, gale.py:735-760). */
int pa_deslice(int dtype, const pa_shape *shape, const void *w, const float *out_slice_token, void *out_x,
               void *stream);

/* ---- backward pass (general kernels; fp32 arithmetic, fp32 or bf16 storage) -------------------------
 * The reference has no backward code of its own: gradients come from autograd over PA.py:501-558
 * (exercised by test/nn/module/test_physics_attention.py:185-226, :364-387).  The entry points below are the
 * layer-specific parts of that gradient; the weight gradients, which are plain GEMMs over the point axis
 * (d W = d out^T . in), are left to the caller's GEMM library.  With g = d out_x (B,N,H*D):
 *   1. pa_rows_gemm            g = d y . W_out                  (and, last, d x = [d x_mid | d fx_mid] . [W_x ; W_fx])
 *   2. pa_slice_weighted_sum   d tok'[s,:] = sum_n w[n,s] g[n,:]                      (adjoint of PA.py:480-481)
 *   3. pa_slice_attention_backward   d tok' -> gradients of the un-normalised slice sums  (PA.py:429-465, :185-203)
 *   4. pa_slice_softmax_backward     per point: d x_mid, d fx_mid, d z (slice logits before the temperature),
 *                                    d temperature                                    (PA.py:172-203, :480-481, :537)
 */

/* out[m, o] = bias[o] + sum_k A(m, k) weight[o, k] over the B*N rows of `in` (B, N, c_in); bias may be NULL.
 * grid->conv_k == 0: A(m, k) = in[m, k], weight (c_out, c_in).  conv_k = k > 0: the stride-1 zero-padded
 * convolution over the point grid (grid_h, grid_w[, grid_d]) with weight (c_out, c_in, k, k[, k]) as torch lays
 * it out.  Only B, N, grid_* and conv_k of `grid` are read.  `weight` has the activation dtype. */
int pa_rows_gemm(int dtype, const pa_shape *grid, int64_t c_in, int64_t c_out, const void *in, const void *weight,
                 const float *bias, void *out, void *stream);
/* The same followed by an activation: act = 0 none, 1 = GELU in its erf form.  With act = 1 and a second call this is
 * the preprocess Mlp of the model, Linear -> GELU -> Linear (TR.py:519-525, mlp_layers.py:139-173); with act = 0 and
 * c_out = out_dim the output head ln_mlp2[1] (TR.py:305-307). */
int pa_rows_gemm_act(int dtype, const pa_shape *grid, int64_t c_in, int64_t c_out, const void *in, const void *weight,
                     const float *bias, int act, void *out, void *stream);

/* sums[b,h,s,d] = sum_n w[b,n,h,s] v[b,n,h*D+d] for d < D, sums[b,h,s,D] = sum_n w[b,n,h,s]; float32
 * (B,H,S,D+1).  `partials` as for pa_slice_reduce.  Two passes, fixed order. */
int pa_slice_weighted_sum(int dtype, const pa_shape *shape, const void *w, const void *v, float *partials,
                          float *sums, void *stream);

/* 1 if the backward entry points serve this shape (their LDS footprints fit), 0 if not, negative = error. */
int pa_backward_query(int dtype, const pa_shape *shape);

/* Backward of the slice attention and of the normalisation tok = num / nrm (nrm = slice_norm = sum_n w + 1e-2).
 *   d_out_slice_token (B,H,S,D): gradient w.r.t. the attended tokens.
 *   scratch: float32, B*H*2*S*S elements.
 *   d_num (B,H,S,D), d_norm (B,H,S): gradients w.r.t. num and nrm.  slice_norm == NULL: d_num receives the
 *   gradient w.r.t. slice_token itself and d_norm is not written (plain backward of pa_slice_attention).
 *   d_qkv_partials (B*H, 3D, D): each (b,h)'s share of d qkv_project_weight; the caller adds them up. */
int pa_slice_attention_backward(const pa_shape *shape, const pa_params *p, const float *slice_token,
                                const float *slice_norm, const float *d_out_slice_token, float *scratch,
                                float *d_num, float *d_norm, float *d_qkv_partials, void *stream);

/* Per-point part of the backward pass.  Inputs as saved by the forward stages (x_mid, fx_mid (B,N,H*D), w (B,N,H,S),
 * out_slice_token (B,H,S,D)), d_out_x (B,N,H*D) and the d_num / d_norm of pa_slice_attention_backward.  Outputs:
 *   d_proj (B,N,2*H*D) = [d x_mid | d fx_mid];  d_z (B,N,H,S) = gradient of the in_project_slice output;
 *   d_temperature_partials: float32, pa_backward_point_tiles(shape) * H elements; d clamp(temperature)[h] is the
 *   sum over the first index (the caller masks it with 0.5 <= temperature <= 5, the clamp's own gradient). */
int64_t pa_backward_point_tiles(const pa_shape *shape);
int pa_slice_softmax_backward(int dtype, const pa_shape *shape, const pa_params *p, const void *x_mid,
                              const void *fx_mid, const void *w, const void *d_out_x, const float *out_slice_token,
                              const float *d_num, const float *d_norm, void *d_proj, void *d_z,
                              float *d_temperature_partials, void *stream);

/* The same for Transolver++ (plus = True; PA.py:166-170, :530-532, gumbel_softmax.py:49-57): one projection
 * (fx_mid is x_mid), `uniform` the samples given to pa_slice_softmax_plus, w its output.  Outputs:
 *   d_x_mid (B,N,H*D): the whole gradient of the projection (slice logits, aggregation and proj_temperature paths);
 *   d_z (B,N,H,S) as above;  d_a1 (B,N,H,S), activation dtype: gradient of the proj_temperature[0] output;
 *   d_a2 (B,N,H) float32: gradient of the proj_temperature[2] output;
 *   d_temperature_partials: pa_backward_point_tiles_plus(shape) * H float32; d temperature[h] is the sum over the
 *   first index (the lower clamp at 0.01 is already applied per point). */
int64_t pa_backward_point_tiles_plus(const pa_shape *shape);
int pa_slice_softmax_plus_backward(int dtype, const pa_shape *shape, const pa_params *p, const pa_plus_params *plus,
                                   const void *x_mid, const void *uniform, const void *w, const void *d_out_x,
                                   const float *out_slice_token, const float *d_num, const float *d_norm,
                                   void *d_x_mid, void *d_z, void *d_a1, float *d_a2, float *d_temperature_partials,
                                   void *stream);

/* ---- GALE: cross-attention of the slice tokens to a context (physicsnemo/nn/module/gale.py) ------
 * A GALE layer (gale.py:242-478) is a PhysicsAttention layer whose slice-token stage also attends to a context
 * (B,H,Sc,Dc) and blends the two results (gale.py:87-145 _gale_compute_slice_attention_cross, :43-84
 * _mix_self_and_cross); every other stage is the entry points above.  All tensors float32. */
typedef struct pa_gale_params {
  const float *cross_q_weight; /* (D, D)  */
  const float *cross_q_bias;   /* (D)     */
  const float *cross_k_weight; /* (D, Dc) */
  const float *cross_k_bias;   /* (D)     */
  const float *cross_v_weight; /* (D, Dc) */
  const float *cross_v_bias;   /* (D)     */
  const float *state_mixing;   /* scalar; state_mixing_mode "weighted": out = sigmoid(m) self + (1 - sigmoid(m)) cross */
  const float *concat_project_weight; /* (D, 2D) concat_project[0]; mode "concat_project":                          */
  const float *concat_project_bias;   /* (D)      out = gelu([self | cross] W^T + b).  Exactly one mode is non-NULL. */
} pa_gale_params;
/* out_slice_token (B,H,S,D) = blend(self_out_slice_token, softmax(q k^T / sqrt(D)) v) with q from slice_token and
 * k, v from context (B,H,context_slices,context_dim).  tokp: NULL, or the PA_BUF_TOKP buffer of the MFMA kernels,
 * which then receives the result as operands of pa_mfma_deslice_project (shapes with pa_query_path() == 1 only). */
int pa_slice_cross_attention_mix(const pa_shape *shape, const pa_gale_params *gale, int64_t context_slices,
                                 int64_t context_dim, const float *slice_token, const float *self_out_slice_token,
                                 const float *context, float *out_slice_token, void *tokp, void *stream);

/* ---- Ball query (physicsnemo/nn/module/ball_query.py:32-140, BQWarp.forward with neighbors_in_radius set; the order
 * of physicsnemo/nn/functional/neighbors/radius_search/_torch_impl.py:59-160) --------------------------------------
 * For every query the up to max_neighbors (<= 64) nearest points with distance <= radius, ascending by distance (equal
 * distances: lower index first).  points (batch, n_points, 3), queries (batch, n_queries, 3) float32;
 * indices (batch, n_queries, max_neighbors) int64, 0 in unused slots; optional outputs (NULL to skip):
 * neighbor_points (batch, n_queries, max_neighbors, 3) float32, zeros in unused slots; neighbor_dists
 * (batch, n_queries, max_neighbors) float32; counts (batch, n_queries) int32 = used slots.  Used by the local
 * features of GeoTransolver (physicsnemo/models/geotransolver/context_projector.py:491-606). */
int pa_ball_query(int64_t batch, int64_t n_points, int64_t n_queries, int64_t max_neighbors, float radius,
                  const float *points, const float *queries, int64_t *indices, float *neighbor_points,
                  float *neighbor_dists, int32_t *counts, void *stream);

/* The same search over a cell list the caller has built (for large clouds; pa_ball_query looks at every pair):
 * the points of each batch binned into cells_per_axis^3 cells whose edge along every axis is >= radius * 1.0001,
 *   grid (batch, 6) float32 = origin x, y, z and 1 / edge x, y, z;  cell of a point = floor((p - origin) / edge) per
 *   axis clamped to the grid, cell index (ix * G + iy) * G + iz;
 *   sorted_points (batch * n_points, 3): the points ordered by (batch, cell index); sorted_index (batch * n_points)
 *   int32: each one's index within its batch; cell_start (batch * G^3 + 1) int32: offset of every cell's first point in
 *   that order;  query_order (batch, n_queries) int32 or NULL: a processing order of each batch's queries (a
 *   permutation; spatially sorted queries read the same cells in neighbouring lanes).
 * Same outputs as pa_ball_query, identical results. */
int pa_ball_query_cells(int64_t batch, int64_t n_points, int64_t n_queries, int64_t max_neighbors, float radius,
                        int64_t cells_per_axis, const float *grid, const float *sorted_points,
                        const int32_t *sorted_index, const int32_t *cell_start, const float *queries,
                        const int32_t *query_order, int64_t *indices, float *neighbor_points, float *neighbor_dists,
                        int32_t *counts, void *stream);

/* ---- FLARE attention (physicsnemo/nn/module/flare_attention.py:38-72, :195-255) ------------------
 * y = softmax_s(A) (softmax_n(A)^T v) with the scores A[b,n,h,s] = k[b,n,h,:] . q_global[h,s,:], S = number of global
 * queries.  A (B,N,H,S) and v (B,N,H*D) come from pa_rows_gemm (the caller folds in_project_x, self_k / self_v and
 * q_global into two weight matrices); then
 *   pa_flare_column_weights  weights = exp(A - max_n A)          (column_max (B,H,S) float32 is an output as well;
 *                            partials: pa_flare_column_max_chunks(shape) * B*H*S float32 of scratch)
 *   pa_slice_reduce(weights, v)  ->  z = slice_token * slice_norm / (slice_norm - 1e-2)     (the first attention pass)
 *   pa_flare_softmax_rows    A <- softmax_s(A) in place
 *   pa_deslice_project(A, z) ->  out_linear(y)                                              (the second pass) */
int64_t pa_flare_column_max_chunks(const pa_shape *shape);
int pa_flare_column_weights(int dtype, const pa_shape *shape, const void *scores, float *partials, float *column_max,
                            void *weights, void *stream);
int pa_flare_softmax_rows(int dtype, const pa_shape *shape, void *scores, void *stream);
/* The whole FLARE layer forward on the bf16 MFMA kernels (flare_attention.py:222-255 with the weights composed as
 * above): scores and values by the weights-stationary row GEMM (values straight into the packed operand layout),
 * column maxima, one kernel that writes both normalisations of the scores as packed operands, the MFMA aggregation and
 * deslice kernels of the PhysicsAttention layer, out_linear (+ optional residual / LayerNorm tail).  bf16, D = 32,
 * C = H*32 in {128, 256}, S in {16, 32, 64, 128}, B*N >= 4096 (pa_flare_forward_mfma_supported() == 1).
 * scores_weight (H*S, C) bf16, values_weight (H*32, C) bf16, out_linear_weight (C, H*32) bf16, biases float32.
 * out_linear_weight NULL (tail NULL as well): y receives the attention output (B, N, H*32) itself, for callers that
 * blend it with something else before the output projection (GALE_FA, gale.py:735-760). */
int pa_flare_forward_mfma_supported(const pa_shape *shape);
int64_t pa_flare_forward_mfma_workspace_bytes(const pa_shape *shape);
int pa_flare_forward_mfma(const pa_shape *shape, const void *scores_weight, const float *scores_bias,
                          const void *values_weight, const float *values_bias, const void *out_linear_weight,
                          const float *out_linear_bias, const void *x, void *y, const pa_block_tail *tail,
                          void *workspace, int64_t workspace_bytes, void *stream);
/* Per-point part of the FLARE backward pass (the reference differentiates flare_attention.py:38-72 with autograd).
 * row_weights = softmax_s(A), column_weights = exp(A - max_n A), values v, d_out_x = gradient of the hand-back result
 * (B,N,H*D), z (B,H,S,D) float32, and d_num / d_den = gradients of the un-normalised gather sums (z = num / den):
 *   d_scores (B,N,H,S) = row softmax backward of d_out_x . z^T  +  column_weights * (v . d_num^T + d_den)
 *   d_values (B,N,H*D) = column_weights . d_num
 * The rest of the backward is the entry points above: pa_rows_gemm (d out_x from d y; d x from d_scores | d_values),
 * pa_slice_weighted_sum (d z), weight gradients as products over the point axis. */
int pa_flare_backward_points(int dtype, const pa_shape *shape, const void *row_weights, const void *column_weights,
                             const void *values, const void *d_out_x, const float *z, const float *d_num,
                             const float *d_den, void *d_scores, void *d_values, void *stream);

/* Attended slice tokens (B,H,S,32) float32 computed by the caller (e.g. a GALE token stage under autograd) -> the
 * PA_BUF_TOKP operands of pa_mfma_deslice_project, which pa_mfma_combine_attention otherwise writes
 * (shapes with pa_query_path() == 1). */
int pa_mfma_pack_tokens(const pa_shape *shape, const float *out_slice_token, void *tokp, void *stream);

/* ---- stage-level entry points of the bf16 MFMA kernels (shapes with pa_query_path() == 1) ------
 * Intermediates use an internal register-order ("packed") layout; buffers are opaque to the caller and
 * sized by pa_mfma_buffer_bytes(shape, which):
 *   PA_BUF_BLOB     repacked parameters        PA_BUF_FX_PACK  fx_mid        PA_BUF_W_PACK  slice weights
 *   PA_BUF_PARTIALS float32 reduction partials PA_BUF_TOKP     attended slice tokens as bf16 MFMA operands
 * They replace the same reference lines as the natural-layout stages above. */
#define PA_BUF_BLOB 0
#define PA_BUF_FX_PACK 1
#define PA_BUF_W_PACK 2
#define PA_BUF_PARTIALS 3
#define PA_BUF_TOKP 4
int64_t pa_mfma_buffer_bytes(const pa_shape *shape, int which);
/* Repack the layer parameters for the MFMA kernels; run once per parameter set.  The three large weights are bf16
 * (all three p->*_scale NULL) or fp8-e4m3 bytes with per-output-channel scales (all three non-NULL, as PA_BF16_W8):
 * the repacking kernel reads the e4m3 bytes itself, so a parameter set kept in fp8 is expanded once, here, and
 * pa_mfma_layer_forward then runs exactly the bf16 launches. */
int pa_mfma_pack_params(const pa_shape *shape, const pa_params *p, void *blob, void *stream);
/* Kernel (a): projections + slice logits + temperature softmax (PA.py:529-537, :172-181). x is bf16 (B,N,C).
 * fx_pack receives fx_mid WITHOUT the in_project_fx bias: pa_mfma_combine_attention adds bias * (sum of the weights)
 * to the summed values, which is the same sum. */
int pa_mfma_project_softmax(const pa_shape *shape, const void *blob, const void *x, void *fx_pack, void *w_pack,
                            void *stream);
/* Kernel (b): first pass of the slice aggregation (PA.py:185-203) -> partials. */
int pa_mfma_slice_reduce(const pa_shape *shape, const void *w_pack, const void *fx_pack, float *partials,
                         void *stream);
/* Kernels (a)+(b) in one launch (S <= 64): projections, slice softmax and the first pass of the slice aggregation
 * (PA.py:529-537, :172-181, :185-203); fx_mid never leaves the chip. Writes w_pack and partials. This is what
 * pa_layer_forward runs when it applies; PA_ERR_UNSUPPORTED otherwise. */
int pa_mfma_project_softmax_reduce(const pa_shape *shape, const void *blob, const void *x, void *w_pack,
                                   float *partials, void *stream);
/* pa_mfma_project_softmax_reduce with a clock reading: the same kernel (bit-identical w_pack and partials) whose
 * workgroup in the middle of the grid also stores how long it ran -- clock_out[0] in shader cycles, clock_out[1] in
 * ticks of the 100 MHz wall clock (device memory, 16 bytes, 16-byte aligned).  cycles / (10 * ticks) GHz is the shader
 * clock the chip held under this kernel, which is what its roofline fractions should be read against (the published
 * peaks assume the top clock).  Served for C = 256, S <= 64; PA_ERR_UNSUPPORTED otherwise.  No reference counterpart
 * (a measurement aid for bench.py). */
int pa_mfma_project_softmax_reduce_clocked(const pa_shape *shape, const void *blob, const void *x, void *w_pack,
                                           float *partials, uint64_t *clock_out, void *stream);
/* Number of partial sums a first pass leaves in `partials`: fused = 1 for pa_mfma_project_softmax_reduce (or
 * PA_ERR_UNSUPPORTED where it does not apply), 0 for pa_mfma_slice_reduce. Pass it to pa_mfma_combine_attention. */
int64_t pa_mfma_partial_groups(const pa_shape *shape, int fused);
/* Second pass + kernel (c): fixed-order combine, normalisation, slice attention (PA.py:185-203, :429-465).
 * groups = pa_mfma_partial_groups() of the producer. slice_token / slice_norm may be NULL. Writes out_slice_token (B,H,S,D) float32 and its packed copy tokp.
 * Reads p->qkv_project_weight and p->in_project_fx_bias (the bias the producers above leave out of their sums). */
int pa_mfma_combine_attention(const pa_shape *shape, const pa_params *p, const float *partials, int64_t groups,
                              float *slice_token, float *slice_norm, float *out_slice_token, void *tokp,
                              void *stream);
/* Kernel (d): deslice + out_linear + optional residual / LayerNorm tail (PA.py:467-499, TR.py:300-303). */
int pa_mfma_deslice_project(const pa_shape *shape, const void *blob, const void *w_pack, const void *tokp, void *y,
                            const pa_block_tail *tail, void *stream);

/* ---- backward pass on the bf16 MFMA kernels (pa_mfma_backward_query() == 1: MFMA shapes with S <= 64) -------
 * Same gradient as the general backward entry points above, for callers that ran the forward through the pa_mfma_*
 * stages and kept w_pack, the slice tokens and tokp.  No reference counterpart beyond autograd over PA.py:501-558. */
int pa_mfma_backward_query(const pa_shape *shape);
/* Weight-gradient product over the row axis (d W = d out^T . in, the adjoint of a Linear): for bf16 matrices a
 * (rows, lda) and b (rows, ldb) in natural layout,  P[i][j] = sum_m a[m][i] * b[m][j]  for i < cols_a, j < cols_b.
 * cols_a, cols_b multiples of 32 (cols_b in {32, 64, 128, 256}; cols_a <= 256 or a multiple of 256); lda, ldb multiples
 * of 8.  The kernel leaves pa_cols_gemm_chunks(rows, cols_a) partial results, partials (chunks, cols_a, cols_b) float32; the
 * caller adds them up over the first index (fixed order: deterministic).  col_sum_partials (chunks, cols_a) float32,
 * optional (NULL to skip): the column sums of a, i.e. the bias gradient that goes with the weight gradient. */
int64_t pa_cols_gemm_chunks(int64_t rows, int64_t cols_a);
int pa_cols_gemm(int64_t rows, const void *a, int64_t lda, int64_t cols_a, const void *b, int64_t ldb, int64_t cols_b,
                 float *partials, float *col_sum_partials, void *stream);
/* The same for float32 operands (fp32 MFMA, natural row-major operands; cols_a, cols_b, lda, ldb multiples of 4):
 * partials pa_cols_gemm_f32_chunks(rows, cols_a, cols_b) * cols_a * cols_b float32, col_sum_partials chunks * cols_a
 * or NULL. */
int64_t pa_cols_gemm_f32_chunks(int64_t rows, int64_t cols_a, int64_t cols_b);
int pa_cols_gemm_f32(int64_t rows, const void *a, int64_t lda, int64_t cols_a, const void *b, int64_t ldb,
                     int64_t cols_b, float *partials, float *col_sum_partials, void *stream);
/* bf16 Linear over the rows of `in` (B, N, c_in) -> H*32 columns, weight (H*32, c_in) bf16, bias float32 or NULL:
 * `out` natural (B, N, H*32) and/or `out_pack` in the packed layout of PA_BUF_FX_PACK (either may be NULL). */
int pa_rows_gemm_packed(const pa_shape *shape, int64_t c_in, const void *in, const void *weight, const float *bias,
                        void *out, void *out_pack, void *stream);
/* sums (B,H,S,D+1) float32 = sum_n w[n,s] [v[n,:], 1] from the packed operands (adjoint of the deslice when v = d out_x);
 * `partials` sized as PA_BUF_PARTIALS. */
int pa_mfma_slice_weighted_sum(const pa_shape *shape, const void *w_pack, const void *v_pack, float *partials,
                               float *sums, void *stream);
/* out_x (B, N, H*32) bf16 = deslice of the attended tokens (PA.py:492-495), the input of d W_out = dy^T out_x. */
int pa_mfma_deslice(const pa_shape *shape, const void *w_pack, const void *tokp, void *out_x, void *stream);
/* Per-point part of the backward pass, as pa_slice_softmax_backward but with the slice weights taken from w_pack.
 * tables: scratch of pa_mfma_backward_tables_bytes(shape) bytes; d_temperature_partials: float32,
 * pa_mfma_backward_groups(shape) * H elements (sum over the first index). */
int64_t pa_mfma_backward_tables_bytes(const pa_shape *shape);
int64_t pa_mfma_backward_groups(const pa_shape *shape);
int pa_mfma_slice_softmax_backward(const pa_shape *shape, const pa_params *p, const void *x_mid, const void *fx_mid,
                                   const void *d_out_x, const void *w_pack, const float *out_slice_token,
                                   const float *d_num, const float *d_norm, void *tables, void *d_proj, void *d_z,
                                   float *d_temperature_partials, void *stream);

/* ---- block MLP ---------------------------------------------------------------------------------- */

/* Parameters of Mlp(C -> F -> C) with GELU (physicsnemo/nn/module/mlp_layers.py:139-173): torch layouts,
 * w1 (F,C) and w2 (C,F) in the activation dtype, biases float32. */
typedef struct pa_mlp_params {
  const void *w1;
  const float *b1;
  const void *w2;
  const float *b2;
} pa_mlp_params;

/* 1 if pa_mlp_forward serves (dtype, rows, C, F) [bf16, C in {128, 256, 512}, F a multiple of 64 up to 8192 / 6912 /
 * 5632 for the three widths (what the kernel's LDS holds)], else 0. */
int pa_mlp_query(int dtype, int64_t rows, int64_t C, int64_t F);
/* Bytes of workspace pa_mlp_forward needs (the repacked weights), or a negative error code. */
int64_t pa_mlp_workspace_bytes(int dtype, int64_t rows, int64_t C, int64_t F);
/* y = w2 . gelu_erf(w1 . u + b1) + b2 for `rows` rows of u (rows, C); with a tail: y = that + tail->residual and
 * tail->ln_out = LayerNorm(y). Replaces `self.ln_mlp1[1](ln) + fx` of TransolverBlock.forward (TR.py:301-303) and
 * produces the LayerNorm the next consumer starts with (TR.py:300 of the next block, or :305-307). */
int pa_mlp_forward(int dtype, int64_t rows, int64_t C, int64_t F, const pa_mlp_params *p, const void *u, void *y,
                   const pa_block_tail *tail, void *workspace, int64_t workspace_bytes, void *stream);

/* The same in two steps, for callers that keep the repacked weights between calls (one pa_mlp_pack per parameter set):
 * pa_mlp_pack writes pa_mlp_workspace_bytes() bytes into `packed`; pa_mlp_forward_packed is pa_mlp_forward with
 * p->w1 / p->w2 replaced by that buffer (p->b1, p->b2 are still read).  No reference counterpart (the reference's
 * Linear layers keep their weights in the layout the GEMM library wants). */
int pa_mlp_pack(int dtype, int64_t C, int64_t F, const pa_mlp_params *p, void *packed, int64_t packed_bytes, void *stream);
int pa_mlp_forward_packed(int dtype, int64_t rows, int64_t C, int64_t F, const void *packed, const float *b1,
                          const float *b2, const void *u, void *y, const pa_block_tail *tail, void *stream);
/* pa_mlp_forward_packed for rows that still lack the LayerNorm in front of the Mlp: the kernel applies
 * LayerNorm(in_ln) to the rows of u as it turns them into operands, so `ln_mlp1[0]` of TransolverBlock (TR.py:303) costs
 * no pass over memory and its producer (the attention layer's tail) need not write a normalised copy.  With
 * tail->residual == u this is TR.py:303 whole: y = u + Mlp(LayerNorm(u)).  bf16, C in {256, 512}
 * (pa_mlp_input_ln_query() == 1). */
typedef struct pa_input_ln {
  const float *gamma; /* (C) */
  const float *beta;  /* (C) */
  float eps;
} pa_input_ln;
int pa_mlp_input_ln_query(int dtype, int64_t rows, int64_t C, int64_t F);
int pa_mlp_forward_packed_ln(int dtype, int64_t rows, int64_t C, int64_t F, const void *packed, const float *b1,
                             const float *b2, const pa_input_ln *in_ln, const void *u, void *y, const pa_block_tail *tail,
                             void *stream);
/* pa_mlp_pack for weights held as fp8-e4m3 bytes (layout as PA_BF16_W8: w1 (F,C), w2 (C,F) row-major bytes, 8-byte
 * aligned, one float32 scale per output row): the repacking kernel reads the bytes and scales itself and writes the
 * bf16 operand fragments pa_mlp_forward_packed(PA_BF16, ...) takes, bit-identical to pa_mlp_pack over the weights
 * bf16(scale * e4m3).  No reference counterpart (the reference's only fp8 is Transformer Engine autocast). */
int pa_mlp_pack_e4m3(int64_t C, int64_t F, const void *w1, const float *w1_scale, const void *w2, const float *w2_scale,
                     void *packed, int64_t packed_bytes, void *stream);

/* ---- whole block ------------------------------------------------------------------------------ */

/* The rest of TransolverBlock.forward behind the attention layer (TR.py:300-303): LayerNorm ln_mlp1[0] and
 * Mlp ln_mlp1[1] (C -> F -> C, GELU erf); torch layouts, weights in the activation dtype. */
typedef struct pa_block_mlp {
  const float *ln_gamma; /* (C) */
  const float *ln_beta;  /* (C) */
  float ln_eps;
  const void *w1;        /* (F, C) */
  const float *b1;       /* (F) */
  const void *w2;        /* (C, F) */
  const float *b2;       /* (C) */
  int64_t F;
} pa_block_mlp;

/* The last block's output head ln_mlp2[1] (TR.py:305-307), a Linear(C -> O) over next->ln_out with O <= 4 outputs. */
typedef struct pa_block_head {
  const void *weight; /* (O, C), activation dtype */
  const float *bias;  /* (O) or NULL */
  int64_t O;
  void *out;          /* (B, N, O), activation dtype */
} pa_block_head;

/* Replaces TransolverBlock.forward (TR.py:296-307): for a block that is not the last one head is NULL; for the last
 * block next is ln_mlp2[0] and head its Linear (next->ln_out may then be NULL: the LayerNorm is not stored):
 *   fx1 = Attn(x) + fx_in;  fx_out = Mlp(LayerNorm(fx1)) + fx1;  next->ln_out = LayerNorm_next(fx_out)
 * x (B,N,C) is LayerNorm_1(fx_in), which the caller has from the block before (or pa_preprocess_forward);
 * next: ln_gamma / ln_beta / ln_eps / ln_out of the LayerNorm that follows (ln_1 of the next block, or ln_mlp2[0]),
 * residual must be NULL; next may be NULL.  fx1 and its LayerNorm are never stored.
 * Served where pa_block_query() is 1: float32, C = 128, 8 heads of 16, 32 slices, F a multiple of 128 (up to 1024).
 * workspace: pa_block_workspace_bytes(). */
int pa_block_query(int dtype, const pa_shape *shape, int64_t F);
int64_t pa_block_workspace_bytes(int dtype, const pa_shape *shape, int64_t F);
int pa_block_forward(int dtype, const pa_shape *shape, const pa_params *p, const pa_block_mlp *mlp, const void *x,
                     const void *fx_in, void *fx_out, const pa_block_tail *next, const pa_block_head *head,
                     void *workspace, int64_t workspace_bytes, void *stream);

/* The model's preprocess Mlp (TR.py:519-525 with mlp_layers.py:139-173): Linear(c_in -> F) -> GELU(erf) -> Linear(F -> C)
 * over `rows` rows of u (rows, c_in), c_in = coordinates + fields per point; with a tail, tail->ln_out is the first
 * block's LayerNorm of the result (TR.py:300).  Served for float32, C = 128, c_in <= 8, F a multiple of 128
 * (pa_preprocess_query); p: w1 (F, c_in), w2 (C, F) float32.  workspace: pa_preprocess_workspace_bytes(). */
int pa_preprocess_query(int dtype, int64_t rows, int64_t c_in, int64_t F, int64_t C);
int64_t pa_preprocess_workspace_bytes(int dtype, int64_t rows, int64_t c_in, int64_t F, int64_t C);
int pa_preprocess_forward(int dtype, int64_t rows, int64_t c_in, int64_t F, int64_t C, const pa_mlp_params *p,
                          const void *u, void *y, const pa_block_tail *tail, void *workspace, int64_t workspace_bytes,
                          void *stream);

/* The block tail on its own (TR.py:300-303, :305-307): y (rows, C) <- y + tail->residual (if given), then
 * tail->ln_out = LayerNorm(y) (if given).  For callers whose producer of y is not one of the fused kernels. */
int pa_residual_layernorm(int dtype, int64_t rows, int64_t C, void *y, const pa_block_tail *tail, void *stream);

/* Backward of LayerNorm over the last axis (TR.py:210, :300-307; the reference relies on autograd): x, dy, dx (rows, C)
 * in the activation dtype, C a multiple of 4 (float32) / 8 (bf16) and <= 1024; the statistics are recomputed from x.
 * partials: float32 (pa_layernorm_backward_groups(rows), 2, C): [g][0][:] = that group's share of d gamma,
 * [g][1][:] of d beta; the caller adds them up over g. */
int64_t pa_layernorm_backward_groups(int64_t rows);
int pa_layernorm_backward(int dtype, int64_t rows, int64_t C, const void *x, const void *dy, const float *gamma,
                          float eps, void *dx, float *partials, void *stream);

/* ---- whole layer ------------------------------------------------------------------------------ */

/* Replaces PhysicsAttentionBase.forward (PA.py:501-558), plus=False, use_te=False, dropout off.
 *   x (B,N,C) -> y (B,N,C) [= out_linear output; with a tail: y = fx_new, tail->ln_out = LN(fx_new)].
 *   slice_token_out: optional float32 (B,H,S,D) copy of the aggregated slice tokens (may be NULL).
 * Dispatches to the bf16 MFMA kernels when pa_query_path() == 1, else to the general kernels. */
int pa_layer_forward(int dtype, const pa_shape *shape, const pa_params *p, const void *x, void *y,
                     const pa_block_tail *tail, float *slice_token_out, void *workspace,
                     int64_t workspace_bytes, void *stream);

/* The Transolver++ layer (plus = True: PA.py:166-170, :530-537; one projection, per-point temperature, Gumbel noise
 * from the caller's samples `uniform` (B,N,H,S) bf16) on the staged bf16 MFMA kernels: dtype PA_BF16, D = 32,
 * C in {128, 256, 512}, S in {16, 32, 64, 128}, Linear projections (pa_layer_forward_plus_supported() == 1; other
 * shapes run the stage sequence on the general kernels).  Workspace: pa_layer_forward_plus_workspace_bytes(). */
int pa_layer_forward_plus_supported(int dtype, const pa_shape *shape);
int64_t pa_layer_forward_plus_workspace_bytes(int dtype, const pa_shape *shape);
int pa_layer_forward_plus(int dtype, const pa_shape *shape, const pa_params *p, const pa_plus_params *plus,
                          const void *x, const void *uniform, void *y, const pa_block_tail *tail,
                          float *slice_token_out, void *workspace, int64_t workspace_bytes, void *stream);

/* pa_layer_forward for the fused MFMA shapes (pa_query_path() == 1) with the parameters already repacked by
 * pa_mfma_pack_params into `blob` (PA_BUF_BLOB bytes): callers that run many forwards with unchanged weights keep
 * the blob and skip the repack.  For S <= 64 only qkv_project_weight and in_project_fx_bias of `p` are read (both
 * required: PA_ERR_NULL otherwise -- the kernels sum fx_mid without its bias and the combine step adds it); for
 * S = 128 the call runs the packed-tile kernels of the staged family, which take every parameter from `p` (bf16
 * weights, or e4m3 bytes when the three scales are set) and leave `blob` unused.  Workspace as for
 * pa_layer_forward.  No reference counterpart. */
int pa_mfma_layer_forward(const pa_shape *shape, const pa_params *p, const void *blob, const void *x, void *y,
                          const pa_block_tail *tail, float *slice_token_out, void *workspace,
                          int64_t workspace_bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* PHYSATTN_H */
