// C ABI of libphysattn.so: argument validation, workspace carving and dispatch.  No kernels here.
#include <dlfcn.h>
#include <stdlib.h>

#include "pa_common.h"
#include "pa_host.h"

#include <atomic>

namespace {

using pa::aligned16;

// Optional marker ranges for rocprofv3 --marker-trace, in place of the reference's record_function brackets around its
// stages ("_compute_slice_attention_sdpa", "_project_attention_outputs": physics_attention.py:445,490).  Off unless
// the environment holds PA_ROCTX=1 when the first entry point runs; the marker library is looked up at run time, so
// the library has no link-time dependency on it and runs without it.  A range covers the host-side enqueue of its
// stage (the kernels themselves are asynchronous), as the reference's ranges do.
struct Markers {
  int (*push)(const char *);
  int (*pop)();
};

const Markers &markers() {
  static const Markers m = [] {
    Markers r{nullptr, nullptr};
    const char *e = getenv("PA_ROCTX");
    if (!e || e[0] == '\0' || e[0] == '0') return r;
    const char *names[] = {"librocprofiler-sdk-roctx.so.1", "librocprofiler-sdk-roctx.so", "libroctx64.so.4", "libroctx64.so",
                           "/opt/rocm/lib/librocprofiler-sdk-roctx.so", "/opt/rocm/lib/libroctx64.so"};
    for (const char *n : names) {
      void *h = dlopen(n, RTLD_NOW | RTLD_GLOBAL);
      if (!h) continue;
      r.push = reinterpret_cast<int (*)(const char *)>(dlsym(h, "roctxRangePushA"));
      r.pop = reinterpret_cast<int (*)()>(dlsym(h, "roctxRangePop"));
      if (r.push && r.pop) return r;
      r = Markers{nullptr, nullptr};
    }
    return r;
  }();
  return m;
}

struct Range {
  bool on;
  explicit Range(const char *name) : on(markers().push != nullptr) {
    if (on) markers().push(name);
  }
  ~Range() {
    if (on) markers().pop();
  }
  Range(const Range &) = delete;
  Range &operator=(const Range &) = delete;
};

int check_shape(int dtype, const pa_shape *s) {
  if (!s) return PA_ERR_NULL;
  if (dtype != PA_F32 && dtype != PA_BF16 && dtype != PA_BF16_W8) return PA_ERR_UNSUPPORTED;
  if (dtype == PA_BF16_W8 && s->conv_k != 0) return PA_ERR_UNSUPPORTED;
  if (s->B <= 0 || s->N <= 0 || s->C <= 0 || s->H <= 0 || s->D <= 0 || s->S <= 0) return PA_ERR_DIMS;
  if (s->conv_k < 0 || (s->conv_k == 0 && s->grid_d != 0)) return PA_ERR_DIMS;
  if (s->conv_tap_major != 0 && s->conv_tap_major != 1) return PA_ERR_DIMS;
  // the range of every single field first: none of the products below, here or in the workspace plans, can overflow
  if (s->D > PA_MAX_D || s->S > PA_MAX_S) return PA_ERR_UNSUPPORTED;
  if (s->C > (1 << 16) || s->H > 1024) return PA_ERR_UNSUPPORTED;
  if (s->N > PA_MAX_N || s->B > (1 << 20)) return PA_ERR_UNSUPPORTED;  // kernels hold N in an int
  if (s->B * s->H > 65535) return PA_ERR_UNSUPPORTED;  // grid.y of the reduction
  if (s->conv_k > 0) {
    if (s->grid_h <= 0 || s->grid_w <= 0 || s->grid_d < 0) return PA_ERR_DIMS;
    if (s->grid_h > s->N || s->grid_w > s->N || s->grid_d > s->N) return PA_ERR_DIMS;
    const int64_t plane = s->grid_h * s->grid_w;  // at most 2^62
    if (plane > s->N || plane * (s->grid_d > 0 ? s->grid_d : 1) != s->N) return PA_ERR_DIMS;
    if (s->conv_k > 1024) return PA_ERR_UNSUPPORTED;
    const int64_t taps = s->conv_k * s->conv_k * (s->grid_d > 0 ? s->conv_k : 1);
    if (taps * s->C > (int64_t)1 << 30) return PA_ERR_UNSUPPORTED;
    if (s->conv_k % 2 == 0) return PA_ERR_UNSUPPORTED;  // even kernels change the output size in the reference
  }
  if (pa::general::combine_attn_lds_bytes(*s) > pa::kMaxLdsBytes) return PA_ERR_UNSUPPORTED;
  return PA_OK;
}

int64_t round_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

// Limits of the row-count / column-count entry points (those without a pa_shape): sizes beyond them are refused
// before any product of them is formed.
constexpr int64_t kMaxRows = PA_MAX_ROWS, kMaxCols = PA_MAX_COLS;
bool rows_ok(int64_t rows) { return rows <= kMaxRows; }
bool cols_ok(int64_t cols) { return cols <= kMaxCols; }

int64_t elem_bytes(int dtype) { return dtype == PA_F32 ? 4 : 2; }

// bf16 copies of the three fp8 weights (PA_BF16_W8), placed at the end of the workspace
int64_t dequant_bytes(int dtype, const pa_shape &s) {
  return dtype == PA_BF16_W8 ? 3 * round_up(s.H * s.D * s.C * 2, 256) : 0;
}

// Workspace plan of the general path.
struct GeneralPlan {
  int64_t off_x_mid, off_fx_mid, off_w, off_partials, off_tok, off_norm, off_tok_out, off_blob, total;
  int64_t G;
  bool conv_front;  // float32 structured 2-D layer of the fused front end's shape class
  bool rows_back;   // float32 layer whose hand-back, out_linear and tail run in the row kernel
  int64_t off_blob_out;
};

GeneralPlan plan_general(int dtype, const pa_shape &s) {
  GeneralPlan p{};
  const int64_t e = elem_bytes(dtype), M = s.B * s.N, HD = s.H * s.D;
  p.conv_front = pa::conv::supported(dtype, s);
  p.G = p.conv_front ? pa::conv::groups(s) : pa::general::partial_count(s);
  int64_t off = 0;
  p.off_x_mid = off;  // reused for out_x once the slice weights exist
  off += round_up(M * HD * e, 256);
  p.off_fx_mid = off;
  off += round_up(M * HD * e, 256);
  p.off_w = off;
  off += round_up(M * s.H * s.S * e, 256);
  p.off_partials = off;
  off += round_up((p.G + 1) * s.B * s.H * s.S * (s.D + 1) * 4, 256);  // G partials + their total
  p.off_tok = off;
  off += round_up(s.B * s.H * s.S * s.D * 4, 256);
  p.off_norm = off;
  off += round_up(s.B * s.H * s.S * 4, 256);
  p.off_tok_out = off;
  off += round_up(s.B * s.H * s.S * s.D * 4, 256);
  p.off_blob = off;  // the convolution weights cut into bf16 pieces, in fragment order
  if (p.conv_front) off += round_up(pa::conv::blob_bytes(s), 256);
  p.rows_back = pa::f32rows::backend_supported(dtype, s);
  p.off_blob_out = off;  // out_linear's weight in the same form
  if (p.rows_back) off += round_up(pa::f32rows::backend_blob_bytes(), 256);
  p.total = off;
  return p;
}

// Workspace plan of the MFMA path.
struct MfmaPlan {
  int64_t off_blob, off_fx, off_w, off_partials, off_tok, off_norm, off_tok_out, off_tokp, total;
  int64_t G;
};

int compute_units();

// partial slice-token sums the first reduction pass leaves: one per workgroup of the fused kernel (a), or one per
// point group of kernel (b)
int64_t mfma_groups(const pa_shape &s, bool fused) {
  return fused ? pa::mfma::project_groups(s, compute_units(), true) : pa::mfma::reduce_groups(s);
}

// S = 128 (the slice-token sums do not fit beside the weights of the fused kernel): the layer call runs the packed-tile
// sequence of the staged path instead of kernels (a), (b), (d), where its row kernels serve the width
bool mfma_layer_on_tiles(const pa_shape &s) {
  return !pa::mfma::fuse_reduce(s) && pa::mlp::linear_supported(PA_BF16, s.B * s.N, s.C);
}

int64_t mfma_partials_bytes(const pa_shape &s) {
  int64_t g = mfma_groups(s, false);
  if (pa::mfma::fuse_reduce(s)) g = std::max(g, mfma_groups(s, true));
  if (mfma_layer_on_tiles(s)) g = std::max(g, pa::mfma::softmax_reduce_groups(s, compute_units()));
  return (g + 1) * s.B * s.H * s.S * (s.D + 1) * 4;  // G partials + their total
}

MfmaPlan plan_mfma(const pa_shape &s) {
  MfmaPlan p{};
  p.G = mfma_groups(s, pa::mfma::fuse_reduce(s));
  int64_t off = 0;
  p.off_blob = off;  // the repacked parameters; on the packed-tile sequence the three projections in fragment order
  off += round_up(std::max(pa::mfma::blob_bytes(s), 3 * pa::mlp::linear_blob_bytes(s.C)), 256);
  p.off_fx = off;
  off += round_up(pa::mfma::fx_pack_bytes(s), 256);
  p.off_w = off;
  off += round_up(pa::mfma::w_pack_bytes(s), 256);
  p.off_partials = off;
  off += round_up(mfma_partials_bytes(s), 256);
  p.off_tok = off;
  off += round_up(s.B * s.H * s.S * s.D * 4, 256);
  p.off_norm = off;
  off += round_up(s.B * s.H * s.S * 4, 256);
  p.off_tok_out = off;
  off += round_up(s.B * s.H * s.S * s.D * 4, 256);
  p.off_tokp = off;
  off += round_up(pa::mfma::tokp_bytes(s), 256);
  p.total = off;
  return p;
}

// Workspace plan of the staged MFMA path.  The slice weights are never stored: the token sums and the hand-back to
// the points each recompute them from x_mid.
struct StagedPlan {
  int64_t off_x_mid, off_fx, off_partials, off_tok, off_norm, off_tok_out, off_tokp, off_wout, total;
  int64_t G;
};

int64_t conv_taps(const pa_shape &s) { return s.conv_k * s.conv_k * (s.grid_d > 0 ? s.conv_k : 1); }

// grid convolutions whose projections run on the implicit-GEMM kernel that writes packed tiles
bool staged_conv_on_tiles(const pa_shape &s) {
  return s.conv_k > 0 && pa::mlp::conv_project_supported(PA_BF16, s.B, s.N, s.C) &&
         pa::mlp::linear_supported(PA_BF16, s.B * s.N, s.C);
}

StagedPlan plan_staged(const pa_shape &s) {
  StagedPlan p{};
  p.G = pa::mfma::softmax_reduce_groups(s, compute_units());
  const int64_t tiles = s.B * pa::mfma::tiles_per_batch(s);
  int64_t off = 0;
  // x_mid as rows (B, N, H*32) or as packed tiles (whole tiles per batch); overwritten by out_x, one point and head
  // at a time, as the weights are recomputed
  p.off_x_mid = off;
  off += round_up(tiles * 32 * s.H * 32 * 2, 256);
  p.off_fx = off;
  off += round_up(tiles * s.H * 2 * 1024, 256);
  p.off_partials = off;
  off += round_up((p.G + 1) * s.B * s.H * s.S * (s.D + 1) * 4, 256);
  p.off_tok = off;
  off += round_up(s.B * s.H * s.S * s.D * 4, 256);
  p.off_norm = off;
  off += round_up(s.B * s.H * s.S * 4, 256);
  p.off_tok_out = off;
  off += round_up(s.B * s.H * s.S * s.D * 4, 256);
  p.off_tokp = off;
  off += round_up(s.B * s.H * (s.S / 16) * 1024, 256);
  p.off_wout = off;  // the three projections' weights in fragment order, where the row-owning kernels serve them
  if (staged_conv_on_tiles(s))
    off += round_up(pa::mlp::conv_project_blob_bytes(s.C, conv_taps(s)), 256) + round_up(pa::mlp::linear_blob_bytes(s.C), 256);
  else if (pa::mlp::linear_supported(PA_BF16, s.B * s.N, s.C)) off += round_up(3 * pa::mlp::linear_blob_bytes(s.C), 256);
  p.total = off;
  return p;
}

// Workspace plan of the Transolver++ layer: the staged kernels with the slice weights stored (their Gumbel noise
// comes from the caller's samples, which are read once).
struct PlusPlan {
  int64_t off_x_mid, off_fx, off_w, off_partials, off_tok, off_norm, off_tok_out, off_tokp, off_blob, total;
  int64_t G;
};

PlusPlan plan_plus(const pa_shape &s) {
  PlusPlan p{};
  p.G = mfma_groups(s, false);
  const int64_t tiles = s.B * pa::mfma::tiles_per_batch(s);
  int64_t off = 0;
  p.off_x_mid = off;  // natural (B, N, H*32); reused for out_x once the slice weights exist
  off += round_up(s.B * s.N * s.H * 32 * 2, 256);
  p.off_fx = off;
  off += round_up(tiles * s.H * 2 * 1024, 256);
  p.off_w = off;
  off += round_up(tiles * s.H * (s.S / 16) * 1024, 256);
  p.off_partials = off;
  off += round_up((p.G + 1) * s.B * s.H * s.S * (s.D + 1) * 4, 256);
  p.off_tok = off;
  off += round_up(s.B * s.H * s.S * s.D * 4, 256);
  p.off_norm = off;
  off += round_up(s.B * s.H * s.S * 4, 256);
  p.off_tok_out = off;
  off += round_up(s.B * s.H * s.S * s.D * 4, 256);
  p.off_tokp = off;
  off += round_up(s.B * s.H * (s.S / 16) * 1024, 256);
  p.off_blob = off;  // the parameter blob of kernel (d), where that kernel serves the shape
  if (pa::mfma::supported(PA_BF16, s)) off += round_up(pa::mfma::blob_bytes(s), 256);
  p.total = off;
  return p;
}

// 0 general kernels, 1 fused MFMA kernels, 2 staged MFMA kernels
int kernel_path(int dtype, const pa_shape &s) {
  if (pa::mfma::supported(dtype, s)) return 1;
  if (pa::mfma::staged_supported(dtype, s)) return 2;
  return 0;
}

int64_t body_bytes(int dtype, const pa_shape &s) {
  switch (kernel_path(dtype, s)) {
    case 1: return plan_mfma(s).total;
    case 2: return plan_staged(s).total;
    default: return plan_general(dtype, s).total;
  }
}

static std::atomic<int> g_compute_units_limit{0};

int compute_units() {
  const int limit = g_compute_units_limit.load(std::memory_order_relaxed);
  if (limit > 0) return limit;
  static int cached[64];  // per device; 0 = not yet asked (racing first calls write the same value)
  int dev = 0, n = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 256;
  if (dev >= 0 && dev < 64 && cached[dev] > 0) return cached[dev];
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 256;
  if (dev >= 0 && dev < 64) cached[dev] = n;
  return n;
}

int check_params(const pa_params *p) {
  if (!p) return PA_ERR_NULL;
  if (!p->in_project_x_weight || !p->in_project_x_bias || !p->in_project_fx_weight || !p->in_project_fx_bias ||
      !p->in_project_slice_weight || !p->in_project_slice_bias || !p->temperature || !p->qkv_project_weight ||
      !p->out_linear_weight || !p->out_linear_bias)
    return PA_ERR_NULL;
  if (!aligned16(p->in_project_x_weight) || !aligned16(p->in_project_fx_weight) || !aligned16(p->out_linear_weight))
    return PA_ERR_ALIGN;
  return PA_OK;
}

int check_tail(const pa_block_tail *t) {
  if (!t) return PA_OK;
  if (t->ln_out && (!t->ln_gamma || !t->ln_beta)) return PA_ERR_NULL;
  if (!aligned16(t->residual) || !aligned16(t->ln_out)) return PA_ERR_ALIGN;
  return PA_OK;
}

bool tail_active(const pa_block_tail *t) { return t && (t->residual || t->ln_out); }

// the fused MFMA kernels of one layer call, parameters already repacked into `blob`
int mfma_layer(const pa_shape &s, const pa_params &p, const void *blob, const void *x, void *y, const pa_block_tail *tail,
               float *slice_token_out, char *ws, const MfmaPlan &mp, hipStream_t st) {
  void *fxp = ws + mp.off_fx, *wp = ws + mp.off_w, *tokp = ws + mp.off_tokp;
  float *partials = reinterpret_cast<float *>(ws + mp.off_partials);
  float *tok = slice_token_out ? slice_token_out : reinterpret_cast<float *>(ws + mp.off_tok);
  float *norm = reinterpret_cast<float *>(ws + mp.off_norm);
  float *tok_out = reinterpret_cast<float *>(ws + mp.off_tok_out);
  int rc;
  if (mfma_layer_on_tiles(s)) {
    // slice weights recomputed where they are used, never stored; every intermediate a packed tile of 32 points.
    // x_mid / out_x take the room of the slice weights, the projections' fragments that of the parameter blob.
    char *wts = ws + mp.off_blob;
    const int64_t G = pa::mfma::softmax_reduce_groups(s, compute_units());
    if ((rc = pa::mlp::project_packed(s.B, s.N, s.C, p.in_project_x_weight, p.in_project_x_scale, p.in_project_x_bias,
                                      p.in_project_fx_weight, p.in_project_fx_scale, p.in_project_fx_bias, x, wp, fxp,
                                      wts, compute_units(), st)))
      return rc;
    if ((rc = pa::mfma::slice_softmax_reduce(s, p, wp, true, fxp, partials, compute_units(), st))) return rc;
    if ((rc = pa::mfma::combine_attention(s, p, nullptr, partials, G, tok, norm, tok_out, tokp, st))) return rc;
    // hand-back, out_linear and the tail in kernel (d) with the slice weights recomputed from the x_mid tiles (the
    // out_linear part of the parameter blob lies behind the room the projections' fragments took)
    if (pa::mfma::deslice_recompute_project_supported(s))
      return pa::mfma::deslice_recompute_project(s, p, blob, wp, tokp, y, tail_active(tail) ? tail : nullptr,
                                                 compute_units(), st);
    if ((rc = pa::mfma::deslice_recompute(s, p, wp, true, tokp, wp, compute_units(), st))) return rc;
    return pa::mlp::linear_packed(s.B, s.N, s.C, p.out_linear_weight, p.out_linear_scale, p.out_linear_bias, wp, y,
                                  tail_active(tail) ? tail : nullptr, wts + 2 * pa::mlp::linear_blob_bytes(s.C),
                                  compute_units(), st);
  }
  {
    Range r("_compute_slices_from_projections");
    if (pa::mfma::fuse_reduce(s)) {  // kernel (a) also leaves the partial slice-token sums
      if ((rc = pa::mfma::project_softmax(s, blob, x, nullptr, wp, partials, compute_units(), st))) return rc;
    } else {
      if ((rc = pa::mfma::project_softmax(s, blob, x, fxp, wp, nullptr, compute_units(), st))) return rc;
      if ((rc = pa::mfma::slice_reduce(s, wp, fxp, partials, st))) return rc;
    }
  }
  {
    Range r("_compute_slice_attention_sdpa");
    if ((rc = pa::mfma::combine_attention(s, p, p.in_project_fx_bias, partials, mp.G, tok, norm, tok_out, tokp, st)))
      return rc;
  }
  Range r("_project_attention_outputs");
  return pa::mfma::deslice_project(s, blob, wp, tokp, y, tail_active(tail) ? tail : nullptr, compute_units(), st);
}

}  // namespace

extern "C" {

int pa_version(void) { return 111; }

int pa_set_compute_units(int n) {
  if (n < 0 || n > 4096) return PA_ERR_DIMS;
  g_compute_units_limit.store(n, std::memory_order_relaxed);
  return PA_OK;
}

int pa_markers_enabled(void) { return markers().push != nullptr ? 1 : 0; }

const char *pa_status_string(int code) {
  switch (code) {
    case PA_OK: return "ok";
    case PA_ERR_NULL: return "a required pointer is NULL";
    case PA_ERR_DIMS: return "a dimension is non-positive or inconsistent";
    case PA_ERR_UNSUPPORTED: return "shape or dtype outside the supported range";
    case PA_ERR_ALIGN: return "a pointer is not 16-byte aligned";
    case PA_ERR_WORKSPACE: return "workspace too small";
    case PA_ERR_SCRATCH: return "problem too large for the library's static scratch buffer";
    default: return code > 0 ? "hip error" : "unknown error";
  }
}

int pa_query_path(int dtype, const pa_shape *shape) {
  int rc = check_shape(dtype, shape);
  if (rc) return rc;
  return kernel_path(dtype == PA_BF16_W8 ? PA_BF16 : dtype, *shape);
}

int64_t pa_workspace_bytes(int dtype, const pa_shape *shape) {
  int rc = check_shape(dtype, shape);
  if (rc) return rc;
  const int act = dtype == PA_BF16_W8 ? PA_BF16 : dtype;
  return body_bytes(act, *shape) + dequant_bytes(dtype, *shape);
}

int pa_project_inputs(int dtype, const pa_shape *shape, const pa_params *p, const void *x, void *x_mid, void *fx_mid,
                      void *stream) {
  int rc = check_shape(dtype, shape);
  if (rc) return rc;
  if (dtype == PA_BF16_W8) return PA_ERR_UNSUPPORTED;  // fp8 weights: whole-layer entry point only
  if (!p || !p->in_project_x_weight || !p->in_project_x_bias) return PA_ERR_NULL;
  if (fx_mid && (!p->in_project_fx_weight || !p->in_project_fx_bias)) return PA_ERR_NULL;
  if (!x || !x_mid) return PA_ERR_NULL;
  if (!aligned16(x) || !aligned16(x_mid) || !aligned16(fx_mid) || !aligned16(p->in_project_x_weight) ||
      !aligned16(p->in_project_fx_weight))
    return PA_ERR_ALIGN;
  return pa::general::project_inputs(dtype, *shape, *p, x, x_mid, fx_mid, static_cast<hipStream_t>(stream));
}

int pa_slice_softmax_plus(int dtype, const pa_shape *shape, const pa_params *p, const pa_plus_params *plus,
                          const void *x_mid, const void *uniform, void *w, void *scratch, void *stream) {
  int rc = check_shape(dtype, shape);
  if (rc) return rc;
  if (dtype == PA_BF16_W8) return PA_ERR_UNSUPPORTED;
  if (!p || !p->in_project_slice_weight || !p->in_project_slice_bias || !p->temperature) return PA_ERR_NULL;
  if (!plus || !plus->proj_temperature_0_weight || !plus->proj_temperature_0_bias || !plus->proj_temperature_2_weight ||
      !plus->proj_temperature_2_bias)
    return PA_ERR_NULL;
  if (!x_mid || !uniform || !w) return PA_ERR_NULL;
  if (!aligned16(x_mid) || !aligned16(uniform) || !aligned16(w) || !aligned16(scratch)) return PA_ERR_ALIGN;
  return pa::general::slice_softmax_plus(dtype, *shape, *p, *plus, x_mid, uniform, w, scratch,
                                         static_cast<hipStream_t>(stream));
}

int pa_slice_softmax(int dtype, const pa_shape *shape, const pa_params *p, const void *x_mid, void *w, void *stream) {
  int rc = check_shape(dtype, shape);
  if (rc) return rc;
  if (dtype == PA_BF16_W8) return PA_ERR_UNSUPPORTED;  // fp8 weights: whole-layer entry point only
  if (!p || !p->in_project_slice_weight || !p->in_project_slice_bias || !p->temperature || !x_mid || !w) return PA_ERR_NULL;
  if (!aligned16(x_mid) || !aligned16(w)) return PA_ERR_ALIGN;
  return pa::general::slice_softmax(dtype, *shape, *p, x_mid, w, static_cast<hipStream_t>(stream));
}

int64_t pa_reduce_partial_count(const pa_shape *shape) {
  int rc = check_shape(PA_F32, shape);
  if (rc) return rc;
  return pa::general::partial_count(*shape) + 1;  // G partial sums + one slot for their total
}

int pa_slice_reduce(int dtype, const pa_shape *shape, const void *w, const void *fx_mid, float *partials,
                    float *slice_token, float *slice_norm, void *stream) {
  int rc = check_shape(dtype, shape);
  if (rc) return rc;
  if (dtype == PA_BF16_W8) return PA_ERR_UNSUPPORTED;  // fp8 weights: whole-layer entry point only
  if (!w || !fx_mid || !partials || !slice_token || !slice_norm) return PA_ERR_NULL;
  if (!aligned16(w) || !aligned16(fx_mid) || !aligned16(partials)) return PA_ERR_ALIGN;
  hipStream_t st = static_cast<hipStream_t>(stream);
  rc = pa::general::slice_partial(dtype, *shape, w, fx_mid, partials, st);
  if (rc) return rc;
  // the combine kernel also runs the slice attention; here only its token/norm outputs are wanted
  pa_params none{};
  return pa::general::combine_attention(*shape, none, partials, pa::general::partial_count(*shape), slice_token,
                                        slice_norm, nullptr, st);
}

int pa_slice_attention(const pa_shape *shape, const pa_params *p, const float *slice_token, float *out_slice_token,
                       void *stream) {
  int rc = check_shape(PA_F32, shape);
  if (rc) return rc;
  if (!p || !p->qkv_project_weight || !slice_token || !out_slice_token) return PA_ERR_NULL;
  // tokens enter as a single already-normalised "partial": the numerators with a zero count column
  // are not available here, so this entry point uses the dedicated token-input mode (G = 0).
  return pa::general::combine_attention(*shape, *p, slice_token, 0, nullptr, nullptr, out_slice_token,
                                        static_cast<hipStream_t>(stream));
}

int pa_deslice_project(int dtype, const pa_shape *shape, const pa_params *p, const void *w, const float *out_slice_token,
                       void *scratch, void *y, const pa_block_tail *tail, void *stream) {
  int rc = check_shape(dtype, shape);
  if (rc) return rc;
  if (dtype == PA_BF16_W8) return PA_ERR_UNSUPPORTED;  // fp8 weights: whole-layer entry point only
  if (!p || !p->out_linear_weight || !p->out_linear_bias || !w || !out_slice_token || !scratch || !y) return PA_ERR_NULL;
  if (!aligned16(w) || !aligned16(scratch) || !aligned16(y) || !aligned16(p->out_linear_weight)) return PA_ERR_ALIGN;
  if ((rc = check_tail(tail))) return rc;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if ((rc = pa::general::deslice(dtype, *shape, w, out_slice_token, scratch, st))) return rc;
  if ((rc = pa::general::out_linear(dtype, *shape, *p, scratch, y, st))) return rc;
  if (tail_active(tail)) rc = pa::general::residual_ln(dtype, *shape, y, *tail, st);
  return rc;
}

int pa_deslice(int dtype, const pa_shape *shape, const void *w, const float *out_slice_token, void *out_x,
               void *stream) {
  int rc = check_shape(dtype, shape);
  if (rc) return rc;
  if (dtype == PA_BF16_W8) return PA_ERR_UNSUPPORTED;
  if (!w || !out_slice_token || !out_x) return PA_ERR_NULL;
  if (!aligned16(w) || !aligned16(out_x)) return PA_ERR_ALIGN;
  return pa::general::deslice(dtype, *shape, w, out_slice_token, out_x, static_cast<hipStream_t>(stream));
}

int pa_rows_gemm(int dtype, const pa_shape *grid, int64_t c_in, int64_t c_out, const void *in, const void *weight,
                 const float *bias, void *out, void *stream) {
  return pa_rows_gemm_act(dtype, grid, c_in, c_out, in, weight, bias, 0, out, stream);
}

int pa_rows_gemm_act(int dtype, const pa_shape *grid, int64_t c_in, int64_t c_out, const void *in, const void *weight,
                     const float *bias, int act, void *out, void *stream) {
  if (!grid) return PA_ERR_NULL;
  if (act != 0 && act != 1) return PA_ERR_UNSUPPORTED;
  if (dtype != PA_F32 && dtype != PA_BF16) return PA_ERR_UNSUPPORTED;
  if (grid->B <= 0 || grid->N <= 0 || c_in <= 0 || c_out <= 0 || grid->conv_k < 0) return PA_ERR_DIMS;
  if (c_in > (1 << 16) || c_out > (1 << 16) || grid->N > PA_MAX_N) return PA_ERR_UNSUPPORTED;
  if (grid->conv_k > 0) {
    if (grid->grid_h <= 0 || grid->grid_w <= 0 || grid->grid_d < 0) return PA_ERR_DIMS;
    // every extent is at most N (itself at most PA_MAX_N) before any product is formed: no product can overflow
    if (grid->grid_h > grid->N || grid->grid_w > grid->N || grid->grid_d > grid->N) return PA_ERR_DIMS;
    if (grid->grid_h * grid->grid_w > grid->N) return PA_ERR_DIMS;
    if (grid->grid_h * grid->grid_w * (grid->grid_d > 0 ? grid->grid_d : 1) != grid->N) return PA_ERR_DIMS;
    if (grid->conv_k % 2 == 0 || grid->conv_k > 1024) return PA_ERR_UNSUPPORTED;
    const int64_t taps = grid->conv_k * grid->conv_k * (grid->grid_d > 0 ? grid->conv_k : 1);
    if (taps * c_in > (int64_t)1 << 30) return PA_ERR_UNSUPPORTED;
  } else if (grid->grid_d != 0) {
    return PA_ERR_DIMS;
  }
  if (!in || !weight || !out) return PA_ERR_NULL;
  if (!aligned16(in) || !aligned16(weight) || !aligned16(out)) return PA_ERR_ALIGN;
  return pa::general::rows_gemm(dtype, *grid, c_in, c_out, in, weight, bias, act, out, static_cast<hipStream_t>(stream));
}

int pa_slice_weighted_sum(int dtype, const pa_shape *shape, const void *w, const void *v, float *partials, float *sums,
                          void *stream) {
  int rc = check_shape(dtype, shape);
  if (rc) return rc;
  if (dtype == PA_BF16_W8) return PA_ERR_UNSUPPORTED;
  if (!w || !v || !partials || !sums) return PA_ERR_NULL;
  if (!aligned16(w) || !aligned16(v) || !aligned16(partials) || !aligned16(sums)) return PA_ERR_ALIGN;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if ((rc = pa::general::slice_partial(dtype, *shape, w, v, partials, st))) return rc;
  const float *total = nullptr;
  if ((rc = pa::general::combine_partials(*shape, partials, pa::general::partial_count(*shape), &total, st))) return rc;
  const size_t bytes = (size_t)(shape->B * shape->H * shape->S * (shape->D + 1)) * 4;
  hipError_t e = hipMemcpyAsync(sums, total, bytes, hipMemcpyDeviceToDevice, st);
  return e == hipSuccess ? PA_OK : (int)e;
}

static int check_backward_shape(int dtype, const pa_shape *shape) {
  int rc = check_shape(dtype, shape);
  if (rc) return rc;
  if (dtype == PA_BF16_W8) return PA_ERR_UNSUPPORTED;
  if (pa::backward::attention_lds_bytes(*shape) > pa::kMaxLdsBytes) return PA_ERR_UNSUPPORTED;
  if (pa::backward::point_tile_rows(*shape) == 0) return PA_ERR_UNSUPPORTED;
  return PA_OK;
}

int pa_backward_query(int dtype, const pa_shape *shape) {
  int rc = check_backward_shape(dtype, shape);
  return rc == PA_OK ? 1 : (rc == PA_ERR_UNSUPPORTED ? 0 : rc);
}

int64_t pa_backward_point_tiles(const pa_shape *shape) {
  int rc = check_backward_shape(PA_F32, shape);
  if (rc) return rc;
  return pa::backward::point_tiles(*shape);
}

int pa_slice_attention_backward(const pa_shape *shape, const pa_params *p, const float *slice_token,
                                const float *slice_norm, const float *d_out_slice_token, float *scratch,
                                float *d_num, float *d_norm, float *d_qkv_partials, void *stream) {
  int rc = check_backward_shape(PA_F32, shape);
  if (rc) return rc;
  if (!p || !p->qkv_project_weight || !slice_token || !d_out_slice_token || !scratch || !d_num || !d_qkv_partials)
    return PA_ERR_NULL;
  if (slice_norm && !d_norm) return PA_ERR_NULL;
  return pa::backward::slice_attention(*shape, *p, slice_token, slice_norm, d_out_slice_token, scratch, d_num, d_norm,
                                       d_qkv_partials, static_cast<hipStream_t>(stream));
}

int pa_slice_softmax_backward(int dtype, const pa_shape *shape, const pa_params *p, const void *x_mid,
                              const void *fx_mid, const void *w, const void *d_out_x, const float *out_slice_token,
                              const float *d_num, const float *d_norm, void *d_proj, void *d_z,
                              float *d_temperature_partials, void *stream) {
  int rc = check_backward_shape(dtype, shape);
  if (rc) return rc;
  if (!p || !p->in_project_slice_weight || !p->in_project_slice_bias || !p->temperature) return PA_ERR_NULL;
  if (!x_mid || !fx_mid || !w || !d_out_x || !out_slice_token || !d_num || !d_norm || !d_proj || !d_z ||
      !d_temperature_partials)
    return PA_ERR_NULL;
  if (!aligned16(x_mid) || !aligned16(fx_mid) || !aligned16(w) || !aligned16(d_out_x) || !aligned16(d_proj) ||
      !aligned16(d_z))
    return PA_ERR_ALIGN;
  return pa::backward::slice_softmax(dtype, *shape, *p, x_mid, fx_mid, w, d_out_x, out_slice_token, d_num, d_norm,
                                     d_proj, d_z, d_temperature_partials, static_cast<hipStream_t>(stream));
}

int64_t pa_backward_point_tiles_plus(const pa_shape *shape) {
  int rc = check_backward_shape(PA_F32, shape);
  if (rc) return rc;
  const int64_t tiles = pa::backward::point_tiles(*shape, true);
  return tiles == 0 ? (int64_t)PA_ERR_UNSUPPORTED : tiles;
}

int pa_slice_softmax_plus_backward(int dtype, const pa_shape *shape, const pa_params *p, const pa_plus_params *plus,
                                   const void *x_mid, const void *uniform, const void *w, const void *d_out_x,
                                   const float *out_slice_token, const float *d_num, const float *d_norm,
                                   void *d_x_mid, void *d_z, void *d_a1, float *d_a2, float *d_temperature_partials,
                                   void *stream) {
  int rc = check_backward_shape(dtype, shape);
  if (rc) return rc;
  if (pa::backward::point_tile_rows(*shape, true) == 0) return PA_ERR_UNSUPPORTED;
  if (!p || !p->in_project_slice_weight || !p->in_project_slice_bias || !p->temperature) return PA_ERR_NULL;
  if (!plus || !plus->proj_temperature_0_weight || !plus->proj_temperature_0_bias || !plus->proj_temperature_2_weight ||
      !plus->proj_temperature_2_bias)
    return PA_ERR_NULL;
  if (!x_mid || !uniform || !w || !d_out_x || !out_slice_token || !d_num || !d_norm || !d_x_mid || !d_z || !d_a1 ||
      !d_a2 || !d_temperature_partials)
    return PA_ERR_NULL;
  if (!aligned16(x_mid) || !aligned16(uniform) || !aligned16(w) || !aligned16(d_out_x) || !aligned16(d_x_mid) ||
      !aligned16(d_z) || !aligned16(d_a1))
    return PA_ERR_ALIGN;
  return pa::backward::slice_softmax_plus(dtype, *shape, *p, *plus, x_mid, uniform, w, d_out_x, out_slice_token, d_num,
                                          d_norm, d_x_mid, d_z, d_a1, d_a2, d_temperature_partials,
                                          static_cast<hipStream_t>(stream));
}

int pa_slice_cross_attention_mix(const pa_shape *shape, const pa_gale_params *gale, int64_t context_slices,
                                 int64_t context_dim, const float *slice_token, const float *self_out_slice_token,
                                 const float *context, float *out_slice_token, void *tokp, void *stream) {
  int rc = check_shape(PA_F32, shape);
  if (rc) return rc;
  if (context_slices <= 0 || context_dim <= 0 || context_slices > (1 << 16) || context_dim > (1 << 16))
    return PA_ERR_DIMS;
  if (!gale || !gale->cross_q_weight || !gale->cross_q_bias || !gale->cross_k_weight || !gale->cross_k_bias ||
      !gale->cross_v_weight || !gale->cross_v_bias)
    return PA_ERR_NULL;
  const bool weighted = gale->state_mixing != nullptr;
  const bool concat = gale->concat_project_weight != nullptr && gale->concat_project_bias != nullptr;
  if (weighted == concat) return PA_ERR_NULL;  // exactly one blend mode
  if (!slice_token || !self_out_slice_token || !context || !out_slice_token) return PA_ERR_NULL;
  if (tokp && !pa::mfma::supported(PA_BF16, *shape)) return PA_ERR_UNSUPPORTED;
  if (pa::gale::lds_bytes(*shape, context_slices, context_dim) > pa::kMaxLdsBytes) return PA_ERR_UNSUPPORTED;
  return pa::gale::slice_cross_mix(*shape, *gale, context_slices, context_dim, slice_token, self_out_slice_token,
                                   context, out_slice_token, tokp, static_cast<hipStream_t>(stream));
}

int64_t pa_flare_column_max_chunks(const pa_shape *shape) {
  int rc = check_shape(PA_F32, shape);
  if (rc) return rc;
  return pa::flare::column_max_chunks(*shape);
}

int pa_flare_column_weights(int dtype, const pa_shape *shape, const void *scores, float *partials, float *column_max,
                            void *weights, void *stream) {
  int rc = check_shape(dtype, shape);
  if (rc) return rc;
  if (dtype == PA_BF16_W8) return PA_ERR_UNSUPPORTED;
  if (!scores || !partials || !column_max || !weights) return PA_ERR_NULL;
  if (shape->B > 65535) return PA_ERR_UNSUPPORTED;
  return pa::flare::column_weights(dtype, *shape, scores, partials, column_max, weights,
                                   static_cast<hipStream_t>(stream));
}

int pa_flare_softmax_rows(int dtype, const pa_shape *shape, void *scores, void *stream) {
  int rc = check_shape(dtype, shape);
  if (rc) return rc;
  if (dtype == PA_BF16_W8) return PA_ERR_UNSUPPORTED;
  if (!scores) return PA_ERR_NULL;
  return pa::flare::softmax_rows(dtype, *shape, scores, nullptr, static_cast<hipStream_t>(stream));
}

int pa_flare_backward_points(int dtype, const pa_shape *shape, const void *row_weights, const void *column_weights,
                             const void *values, const void *d_out_x, const float *z, const float *d_num,
                             const float *d_den, void *d_scores, void *d_values, void *stream) {
  int rc = check_shape(dtype, shape);
  if (rc) return rc;
  if (dtype == PA_BF16_W8) return PA_ERR_UNSUPPORTED;
  if (pa::flare::backward_tile_rows(*shape) == 0) return PA_ERR_UNSUPPORTED;
  if (!row_weights || !column_weights || !values || !d_out_x || !z || !d_num || !d_den || !d_scores || !d_values)
    return PA_ERR_NULL;
  return pa::flare::backward_points(dtype, *shape, row_weights, column_weights, values, d_out_x, z, d_num, d_den,
                                    d_scores, d_values, static_cast<hipStream_t>(stream));
}

int pa_mfma_pack_tokens(const pa_shape *shape, const float *out_slice_token, void *tokp, void *stream) {
  int rc = check_shape(PA_BF16, shape);
  if (rc) return rc;
  if (!pa::mfma::supported(PA_BF16, *shape)) return PA_ERR_UNSUPPORTED;
  if (!out_slice_token || !tokp) return PA_ERR_NULL;
  return pa::gale::pack_tokens(*shape, out_slice_token, tokp, static_cast<hipStream_t>(stream));
}

int pa_residual_layernorm(int dtype, int64_t rows, int64_t C, void *y, const pa_block_tail *tail, void *stream) {
  if (dtype != PA_F32 && dtype != PA_BF16) return PA_ERR_UNSUPPORTED;
  if (rows <= 0 || C <= 0 || C > (1 << 16)) return PA_ERR_DIMS;
  if (!y || !tail || (!tail->residual && !tail->ln_out)) return PA_ERR_NULL;
  int rc = check_tail(tail);
  if (rc) return rc;
  pa_shape s{};
  s.B = 1;
  s.N = rows;
  s.C = C;
  return pa::general::residual_ln(dtype, s, y, *tail, static_cast<hipStream_t>(stream));
}

int64_t pa_layernorm_backward_groups(int64_t rows) {
  if (rows <= 0) return PA_ERR_DIMS;
  return pa::general::layernorm_backward_groups(rows);
}

int pa_layernorm_backward(int dtype, int64_t rows, int64_t C, const void *x, const void *dy, const float *gamma, float eps,
                          void *dx, float *partials, void *stream) {
  if (dtype != PA_F32 && dtype != PA_BF16) return PA_ERR_UNSUPPORTED;
  if (rows <= 0 || C <= 0 || C > 1024) return PA_ERR_DIMS;
  if (!x || !dy || !gamma || !dx || !partials) return PA_ERR_NULL;
  if (!aligned16(x) || !aligned16(dy) || !aligned16(dx)) return PA_ERR_ALIGN;
  return pa::general::layernorm_backward(dtype, rows, C, x, dy, gamma, eps, dx, partials,
                                         static_cast<hipStream_t>(stream));
}

int64_t pa_cols_gemm_chunks(int64_t rows, int64_t cols_a) {
  if (rows <= 0 || cols_a <= 0) return PA_ERR_DIMS;
  if (!rows_ok(rows) || !cols_ok(cols_a)) return PA_ERR_UNSUPPORTED;
  return pa::gemm::cols_gemm_chunks(rows, cols_a, compute_units());
}

int pa_cols_gemm(int64_t rows, const void *a, int64_t lda, int64_t cols_a, const void *b, int64_t ldb, int64_t cols_b,
                 float *partials, float *col_sum_partials, void *stream) {
  if (rows <= 0 || cols_a <= 0 || cols_b <= 0 || lda < cols_a || ldb < cols_b) return PA_ERR_DIMS;
  if (!rows_ok(rows) || !cols_ok(lda) || !cols_ok(ldb)) return PA_ERR_UNSUPPORTED;
  if (!a || !b || !partials) return PA_ERR_NULL;
  if (!aligned16(a) || !aligned16(b) || !aligned16(partials)) return PA_ERR_ALIGN;
  return pa::gemm::cols_gemm(a, lda, cols_a, b, ldb, cols_b, rows, partials, col_sum_partials, compute_units(),
                             static_cast<hipStream_t>(stream));
}

int pa_ball_query(int64_t batch, int64_t n_points, int64_t n_queries, int64_t max_neighbors, float radius,
                  const float *points, const float *queries, int64_t *indices, float *neighbor_points,
                  float *neighbor_dists, int32_t *counts, void *stream) {
  if (batch <= 0 || n_points <= 0 || n_queries <= 0 || max_neighbors <= 0 || !(radius >= 0.f)) return PA_ERR_DIMS;
  if (!points || !queries || !indices) return PA_ERR_NULL;
  return pa::ballquery::ball_query(batch, n_points, n_queries, max_neighbors, radius, points, queries, indices,
                                   neighbor_points, neighbor_dists, counts, static_cast<hipStream_t>(stream));
}

int pa_ball_query_cells(int64_t batch, int64_t n_points, int64_t n_queries, int64_t max_neighbors, float radius,
                        int64_t cells_per_axis, const float *grid, const float *sorted_points,
                        const int32_t *sorted_index, const int32_t *cell_start, const float *queries,
                        const int32_t *query_order, int64_t *indices, float *neighbor_points, float *neighbor_dists,
                        int32_t *counts, void *stream) {
  if (batch <= 0 || n_points <= 0 || n_queries <= 0 || max_neighbors <= 0 || cells_per_axis <= 0 || !(radius >= 0.f))
    return PA_ERR_DIMS;
  if (!grid || !sorted_points || !sorted_index || !cell_start || !queries || !indices) return PA_ERR_NULL;
  return pa::ballquery::ball_query_cells(batch, n_points, n_queries, max_neighbors, radius, cells_per_axis, grid,
                                         sorted_points, sorted_index, cell_start, queries, query_order, indices,
                                         neighbor_points, neighbor_dists, counts, static_cast<hipStream_t>(stream));
}

int64_t pa_cols_gemm_f32_chunks(int64_t rows, int64_t cols_a, int64_t cols_b) {
  if (rows <= 0 || cols_a <= 0 || cols_b <= 0) return PA_ERR_DIMS;
  if (!rows_ok(rows) || !cols_ok(cols_a) || !cols_ok(cols_b)) return PA_ERR_UNSUPPORTED;
  return pa::gemm::cols_gemm_f32_chunks(rows, cols_a, cols_b, compute_units());
}

int pa_cols_gemm_f32(int64_t rows, const void *a, int64_t lda, int64_t cols_a, const void *b, int64_t ldb,
                     int64_t cols_b, float *partials, float *col_sum_partials, void *stream) {
  if (rows <= 0 || cols_a <= 0 || cols_b <= 0 || lda < cols_a || ldb < cols_b) return PA_ERR_DIMS;
  if (!rows_ok(rows) || !cols_ok(lda) || !cols_ok(ldb)) return PA_ERR_UNSUPPORTED;
  if (!a || !b || !partials) return PA_ERR_NULL;
  if (!aligned16(a) || !aligned16(b) || !aligned16(partials)) return PA_ERR_ALIGN;
  return pa::gemm::cols_gemm_f32(a, lda, cols_a, b, ldb, cols_b, rows, partials, col_sum_partials, compute_units(),
                                 static_cast<hipStream_t>(stream));
}

int pa_mfma_backward_query(const pa_shape *shape) {
  int rc = check_shape(PA_BF16, shape);
  if (rc) return rc;
  return pa::mfma::backward_supported(*shape) && check_backward_shape(PA_BF16, shape) == PA_OK ? 1 : 0;
}

int64_t pa_mfma_backward_tables_bytes(const pa_shape *shape) {
  int rc = check_shape(PA_BF16, shape);
  if (rc) return rc;
  if (!pa::mfma::backward_supported(*shape)) return PA_ERR_UNSUPPORTED;
  return pa::mfma::backward_tables_bytes(*shape);
}

int64_t pa_mfma_backward_groups(const pa_shape *shape) {
  int rc = check_shape(PA_BF16, shape);
  if (rc) return rc;
  if (!pa::mfma::backward_supported(*shape)) return PA_ERR_UNSUPPORTED;
  return pa::mfma::backward_groups(*shape, compute_units()) * shape->B;
}

int pa_rows_gemm_packed(const pa_shape *shape, int64_t c_in, const void *in, const void *weight, const float *bias,
                        void *out, void *out_pack, void *stream) {
  int rc = check_shape(PA_BF16, shape);
  if (rc) return rc;
  if (!pa::mfma::supported(PA_BF16, *shape)) return PA_ERR_UNSUPPORTED;
  if (c_in <= 0 || c_in > (1 << 16)) return PA_ERR_DIMS;
  if (!in || !weight || (!out && !out_pack)) return PA_ERR_NULL;
  if (!aligned16(in) || !aligned16(weight) || !aligned16(out) || !aligned16(out_pack)) return PA_ERR_ALIGN;
  return pa::general::rows_gemm_packed(*shape, c_in, in, weight, bias, out, out_pack, static_cast<hipStream_t>(stream));
}

int pa_mfma_slice_weighted_sum(const pa_shape *shape, const void *w_pack, const void *v_pack, float *partials, float *sums,
                               void *stream) {
  int rc = check_shape(PA_BF16, shape);
  if (rc) return rc;
  if (!pa::mfma::supported(PA_BF16, *shape)) return PA_ERR_UNSUPPORTED;
  if (!w_pack || !v_pack || !partials || !sums) return PA_ERR_NULL;
  if (!aligned16(w_pack) || !aligned16(v_pack) || !aligned16(partials) || !aligned16(sums)) return PA_ERR_ALIGN;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if ((rc = pa::mfma::slice_reduce(*shape, w_pack, v_pack, partials, st))) return rc;
  const float *total = nullptr;
  if ((rc = pa::general::combine_partials(*shape, partials, mfma_groups(*shape, false), &total, st))) return rc;
  const size_t bytes = (size_t)(shape->B * shape->H * shape->S * (shape->D + 1)) * 4;
  hipError_t e = hipMemcpyAsync(sums, total, bytes, hipMemcpyDeviceToDevice, st);
  return e == hipSuccess ? PA_OK : (int)e;
}

int pa_mfma_deslice(const pa_shape *shape, const void *w_pack, const void *tokp, void *out_x, void *stream) {
  int rc = check_shape(PA_BF16, shape);
  if (rc) return rc;
  if (!pa::mfma::supported(PA_BF16, *shape)) return PA_ERR_UNSUPPORTED;
  if (!w_pack || !tokp || !out_x) return PA_ERR_NULL;
  if (!aligned16(w_pack) || !aligned16(tokp) || !aligned16(out_x)) return PA_ERR_ALIGN;
  return pa::mfma::deslice_natural(*shape, w_pack, tokp, out_x, compute_units(), static_cast<hipStream_t>(stream));
}

int pa_mfma_slice_softmax_backward(const pa_shape *shape, const pa_params *p, const void *x_mid, const void *fx_mid,
                                   const void *d_out_x, const void *w_pack, const float *out_slice_token,
                                   const float *d_num, const float *d_norm, void *tables, void *d_proj, void *d_z,
                                   float *d_temperature_partials, void *stream) {
  int rc = check_shape(PA_BF16, shape);
  if (rc) return rc;
  if (!pa::mfma::backward_supported(*shape)) return PA_ERR_UNSUPPORTED;
  if (!p || !p->in_project_slice_weight || !p->in_project_slice_bias || !p->temperature) return PA_ERR_NULL;
  if (!x_mid || !fx_mid || !d_out_x || !w_pack || !out_slice_token || !d_num || !d_norm || !tables || !d_proj || !d_z ||
      !d_temperature_partials)
    return PA_ERR_NULL;
  if (!aligned16(x_mid) || !aligned16(fx_mid) || !aligned16(d_out_x) || !aligned16(w_pack) || !aligned16(tables) ||
      !aligned16(d_proj) || !aligned16(d_z))
    return PA_ERR_ALIGN;
  return pa::mfma::slice_softmax_backward(*shape, *p, x_mid, fx_mid, d_out_x, w_pack, out_slice_token, d_num, d_norm, tables,
                                          d_proj, d_z, d_temperature_partials, compute_units(),
                                          static_cast<hipStream_t>(stream));
}

int64_t pa_mfma_buffer_bytes(const pa_shape *shape, int which) {
  int rc = check_shape(PA_BF16, shape);
  if (rc) return rc;
  if (!pa::mfma::supported(PA_BF16, *shape)) return PA_ERR_UNSUPPORTED;
  switch (which) {
    case PA_BUF_BLOB: return pa::mfma::blob_bytes(*shape);
    case PA_BUF_FX_PACK: return pa::mfma::fx_pack_bytes(*shape);
    case PA_BUF_W_PACK: return pa::mfma::w_pack_bytes(*shape);
    case PA_BUF_PARTIALS: return mfma_partials_bytes(*shape);
    case PA_BUF_TOKP: return pa::mfma::tokp_bytes(*shape);
    default: return PA_ERR_DIMS;
  }
}

static int check_mfma(const pa_shape *shape) {
  int rc = check_shape(PA_BF16, shape);
  if (rc) return rc;
  return pa::mfma::supported(PA_BF16, *shape) ? PA_OK : PA_ERR_UNSUPPORTED;
}

int pa_mfma_pack_params(const pa_shape *shape, const pa_params *p, void *blob, void *stream) {
  int rc = check_mfma(shape);
  if (rc) return rc;
  if ((rc = check_params(p))) return rc;
  if (!blob) return PA_ERR_NULL;
  if (!aligned16(blob)) return PA_ERR_ALIGN;
  // all three scales (fp8-e4m3 large weights) or none (bf16)
  const int scales = (p->in_project_x_scale != nullptr) + (p->in_project_fx_scale != nullptr) + (p->out_linear_scale != nullptr);
  if (scales != 0 && scales != 3) return PA_ERR_NULL;
  return pa::mfma::pack_params(*shape, *p, blob, static_cast<hipStream_t>(stream));
}

int pa_mfma_project_softmax(const pa_shape *shape, const void *blob, const void *x, void *fx_pack, void *w_pack,
                            void *stream) {
  int rc = check_mfma(shape);
  if (rc) return rc;
  if (!blob || !x || !fx_pack || !w_pack) return PA_ERR_NULL;
  if (!aligned16(blob) || !aligned16(x) || !aligned16(fx_pack) || !aligned16(w_pack)) return PA_ERR_ALIGN;
  return pa::mfma::project_softmax(*shape, blob, x, fx_pack, w_pack, nullptr, compute_units(),
                                   static_cast<hipStream_t>(stream));
}

int64_t pa_mfma_partial_groups(const pa_shape *shape, int fused) {
  int rc = check_mfma(shape);
  if (rc) return rc;
  if (fused && !pa::mfma::fuse_reduce(*shape)) return PA_ERR_UNSUPPORTED;
  return mfma_groups(*shape, fused != 0);
}

int pa_mfma_project_softmax_reduce(const pa_shape *shape, const void *blob, const void *x, void *w_pack, float *partials,
                                   void *stream) {
  int rc = check_mfma(shape);
  if (rc) return rc;
  if (!pa::mfma::fuse_reduce(*shape)) return PA_ERR_UNSUPPORTED;
  if (!blob || !x || !w_pack || !partials) return PA_ERR_NULL;
  if (!aligned16(blob) || !aligned16(x) || !aligned16(w_pack) || !aligned16(partials)) return PA_ERR_ALIGN;
  return pa::mfma::project_softmax(*shape, blob, x, nullptr, w_pack, partials, compute_units(),
                                   static_cast<hipStream_t>(stream));
}

int pa_mfma_project_softmax_reduce_clocked(const pa_shape *shape, const void *blob, const void *x, void *w_pack,
                                           float *partials, uint64_t *clock_out, void *stream) {
  int rc = check_mfma(shape);
  if (rc) return rc;
  if (!pa::mfma::fuse_reduce(*shape) || shape->C != 256) return PA_ERR_UNSUPPORTED;
  if (!blob || !x || !w_pack || !partials || !clock_out) return PA_ERR_NULL;
  if (!aligned16(blob) || !aligned16(x) || !aligned16(w_pack) || !aligned16(partials) || !aligned16(clock_out))
    return PA_ERR_ALIGN;
  return pa::mfma::project_softmax_clocked(*shape, blob, x, w_pack, partials, clock_out, compute_units(),
                                           static_cast<hipStream_t>(stream));
}

int pa_mfma_slice_reduce(const pa_shape *shape, const void *w_pack, const void *fx_pack, float *partials, void *stream) {
  int rc = check_mfma(shape);
  if (rc) return rc;
  if (!w_pack || !fx_pack || !partials) return PA_ERR_NULL;
  if (!aligned16(w_pack) || !aligned16(fx_pack) || !aligned16(partials)) return PA_ERR_ALIGN;
  return pa::mfma::slice_reduce(*shape, w_pack, fx_pack, partials, static_cast<hipStream_t>(stream));
}

int pa_mfma_combine_attention(const pa_shape *shape, const pa_params *p, const float *partials, int64_t groups,
                              float *slice_token, float *slice_norm, float *out_slice_token, void *tokp, void *stream) {
  int rc = check_mfma(shape);
  if (rc) return rc;
  if (groups < 1 || (groups + 1) * shape->B * shape->H * shape->S * (shape->D + 1) * 4 > mfma_partials_bytes(*shape))
    return PA_ERR_DIMS;
  if (!p || !p->qkv_project_weight || !p->in_project_fx_bias || !partials || !out_slice_token || !tokp) return PA_ERR_NULL;
  if (!aligned16(partials) || !aligned16(tokp)) return PA_ERR_ALIGN;
  hipStream_t st = static_cast<hipStream_t>(stream);
  return pa::mfma::combine_attention(*shape, *p, p->in_project_fx_bias, partials, groups, slice_token, slice_norm,
                                     out_slice_token, tokp, st);
}

int pa_mfma_deslice_project(const pa_shape *shape, const void *blob, const void *w_pack, const void *tokp, void *y,
                            const pa_block_tail *tail, void *stream) {
  int rc = check_mfma(shape);
  if (rc) return rc;
  if (!blob || !w_pack || !tokp || !y) return PA_ERR_NULL;
  if (!aligned16(blob) || !aligned16(w_pack) || !aligned16(tokp) || !aligned16(y)) return PA_ERR_ALIGN;
  if ((rc = check_tail(tail))) return rc;
  return pa::mfma::deslice_project(*shape, blob, w_pack, tokp, y, tail_active(tail) ? tail : nullptr, compute_units(),
                                   static_cast<hipStream_t>(stream));
}

// float32 at C = 128 runs the split-bf16 row kernel, bf16 the MFMA kernels of pa_mlp.hip
static bool mlp_served(int dtype, int64_t rows, int64_t C, int64_t F) {
  return pa::mlp::supported(dtype, rows, C, F) || pa::f32rows::mlp_supported(dtype, rows, C, F);
}
static int64_t mlp_blob_bytes(int dtype, int64_t C, int64_t F) {
  return dtype == PA_F32 ? pa::f32rows::mlp_blob_bytes(F) : pa::mlp::blob_bytes(C, F);
}

int pa_mlp_query(int dtype, int64_t rows, int64_t C, int64_t F) { return mlp_served(dtype, rows, C, F) ? 1 : 0; }

int64_t pa_mlp_workspace_bytes(int dtype, int64_t rows, int64_t C, int64_t F) {
  if (rows <= 0 || C <= 0 || F <= 0) return PA_ERR_DIMS;
  if (!mlp_served(dtype, rows, C, F)) return PA_ERR_UNSUPPORTED;
  return round_up(mlp_blob_bytes(dtype, C, F), 256);
}

int pa_mlp_pack(int dtype, int64_t C, int64_t F, const pa_mlp_params *p, void *packed, int64_t packed_bytes,
                void *stream) {
  if (C <= 0 || F <= 0) return PA_ERR_DIMS;
  if (!mlp_served(dtype, 1, C, F)) return PA_ERR_UNSUPPORTED;
  if (!p || !p->w1 || !p->w2 || !packed) return PA_ERR_NULL;
  if (!aligned16(p->w1) || !aligned16(p->w2) || !aligned16(packed)) return PA_ERR_ALIGN;
  if (packed_bytes < mlp_blob_bytes(dtype, C, F)) return PA_ERR_WORKSPACE;
  if (dtype == PA_F32) return pa::f32rows::mlp_pack(F, p->w1, p->w2, packed, static_cast<hipStream_t>(stream));
  return pa::mlp::pack(C, F, p->w1, nullptr, p->w2, nullptr, packed, static_cast<hipStream_t>(stream));
}

int pa_mlp_pack_e4m3(int64_t C, int64_t F, const void *w1, const float *w1_scale, const void *w2, const float *w2_scale,
                     void *packed, int64_t packed_bytes, void *stream) {
  if (C <= 0 || F <= 0) return PA_ERR_DIMS;
  if (!mlp_served(PA_BF16, 1, C, F)) return PA_ERR_UNSUPPORTED;
  if (!w1 || !w1_scale || !w2 || !w2_scale || !packed) return PA_ERR_NULL;
  if ((reinterpret_cast<uintptr_t>(w1) & 7u) || (reinterpret_cast<uintptr_t>(w2) & 7u) || !aligned16(packed))
    return PA_ERR_ALIGN;
  if (packed_bytes < mlp_blob_bytes(PA_BF16, C, F)) return PA_ERR_WORKSPACE;
  return pa::mlp::pack(C, F, w1, w1_scale, w2, w2_scale, packed, static_cast<hipStream_t>(stream));
}

int pa_mlp_forward_packed(int dtype, int64_t rows, int64_t C, int64_t F, const void *packed, const float *b1,
                          const float *b2, const void *u, void *y, const pa_block_tail *tail, void *stream) {
  Range entry("pa_mlp_forward_packed");
  if (rows <= 0 || C <= 0 || F <= 0) return PA_ERR_DIMS;
  if (!mlp_served(dtype, rows, C, F)) return PA_ERR_UNSUPPORTED;
  if (!packed || !b1 || !b2 || !u || !y) return PA_ERR_NULL;
  if (!aligned16(packed) || !aligned16(u) || !aligned16(y)) return PA_ERR_ALIGN;
  int rc = check_tail(tail);
  if (rc) return rc;
  if (dtype == PA_F32)
    return pa::f32rows::mlp_forward(rows, F, packed, b1, b2, u, y, tail_active(tail) ? tail : nullptr,
                                    static_cast<hipStream_t>(stream));
  return pa::mlp::forward(rows, C, F, packed, b1, b2, u, y, tail_active(tail) ? tail : nullptr, pa::mlp::InputLn{},
                          compute_units(), static_cast<hipStream_t>(stream));
}

int pa_mlp_input_ln_query(int dtype, int64_t rows, int64_t C, int64_t F) {
  if (rows <= 0 || rows > PA_MAX_ROWS || C <= 0 || F <= 0) return 0;
  return pa::mlp::input_ln_supported(dtype, rows, C, F) ? 1 : 0;
}

int pa_mlp_forward_packed_ln(int dtype, int64_t rows, int64_t C, int64_t F, const void *packed, const float *b1,
                             const float *b2, const pa_input_ln *in_ln, const void *u, void *y, const pa_block_tail *tail,
                             void *stream) {
  Range entry("pa_mlp_forward_packed_ln");
  if (rows <= 0 || C <= 0 || F <= 0) return PA_ERR_DIMS;
  if (rows > PA_MAX_ROWS || !pa::mlp::input_ln_supported(dtype, rows, C, F)) return PA_ERR_UNSUPPORTED;
  if (!packed || !b1 || !b2 || !in_ln || !in_ln->gamma || !in_ln->beta || !u || !y) return PA_ERR_NULL;
  if (!aligned16(packed) || !aligned16(u) || !aligned16(y)) return PA_ERR_ALIGN;
  int rc = check_tail(tail);
  if (rc) return rc;
  pa::mlp::InputLn in;
  in.gamma = in_ln->gamma;
  in.beta = in_ln->beta;
  in.eps = in_ln->eps;
  return pa::mlp::forward(rows, C, F, packed, b1, b2, u, y, tail_active(tail) ? tail : nullptr, in, compute_units(),
                          static_cast<hipStream_t>(stream));
}

int pa_mlp_forward(int dtype, int64_t rows, int64_t C, int64_t F, const pa_mlp_params *p, const void *u, void *y,
                   const pa_block_tail *tail, void *workspace, int64_t workspace_bytes, void *stream) {
  Range entry("pa_mlp_forward");
  if (rows <= 0 || C <= 0 || F <= 0) return PA_ERR_DIMS;
  if (!mlp_served(dtype, rows, C, F)) return PA_ERR_UNSUPPORTED;
  if (!p || !p->w1 || !p->b1 || !p->w2 || !p->b2 || !u || !y || !workspace) return PA_ERR_NULL;
  if (!aligned16(p->w1) || !aligned16(p->w2) || !aligned16(u) || !aligned16(y) || !aligned16(workspace))
    return PA_ERR_ALIGN;
  int rc = check_tail(tail);
  if (rc) return rc;
  if (workspace_bytes < mlp_blob_bytes(dtype, C, F)) return PA_ERR_WORKSPACE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == PA_F32) {
    if ((rc = pa::f32rows::mlp_pack(F, p->w1, p->w2, workspace, st))) return rc;
    return pa::f32rows::mlp_forward(rows, F, workspace, p->b1, p->b2, u, y, tail_active(tail) ? tail : nullptr, st);
  }
  if ((rc = pa::mlp::pack(C, F, p->w1, nullptr, p->w2, nullptr, workspace, st))) return rc;
  return pa::mlp::forward(rows, C, F, workspace, p->b1, p->b2, u, y, tail_active(tail) ? tail : nullptr,
                          pa::mlp::InputLn{}, compute_units(), st);
}

int pa_preprocess_query(int dtype, int64_t rows, int64_t c_in, int64_t F, int64_t C) {
  if (rows <= 0 || rows > PA_MAX_ROWS || c_in <= 0 || F <= 0 || C <= 0) return 0;
  return pa::f32rows::premlp_supported(dtype, rows, c_in, F, C) || pa::mlp::premlp_supported(dtype, rows, c_in, F, C) ? 1 : 0;
}

int64_t pa_preprocess_workspace_bytes(int dtype, int64_t rows, int64_t c_in, int64_t F, int64_t C) {
  if (rows <= 0 || c_in <= 0 || F <= 0 || C <= 0) return PA_ERR_DIMS;
  if (rows > PA_MAX_ROWS) return PA_ERR_UNSUPPORTED;
  if (pa::mlp::premlp_supported(dtype, rows, c_in, F, C)) return round_up(pa::mlp::premlp_blob_bytes(F, C), 256);
  if (!pa::f32rows::premlp_supported(dtype, rows, c_in, F, C)) return PA_ERR_UNSUPPORTED;
  return round_up(pa::f32rows::premlp_blob_bytes(F), 256);
}

int pa_preprocess_forward(int dtype, int64_t rows, int64_t c_in, int64_t F, int64_t C, const pa_mlp_params *p,
                          const void *u, void *y, const pa_block_tail *tail, void *workspace, int64_t workspace_bytes,
                          void *stream) {
  Range entry("pa_preprocess_forward");
  if (rows <= 0 || c_in <= 0 || F <= 0 || C <= 0) return PA_ERR_DIMS;
  if (rows > PA_MAX_ROWS) return PA_ERR_UNSUPPORTED;
  if (pa::mlp::premlp_supported(dtype, rows, c_in, F, C)) {  // bf16: hidden layer on chip, MFMA row kernel
    if (!p || !p->w1 || !p->b1 || !p->w2 || !p->b2 || !u || !y || !workspace) return PA_ERR_NULL;
    if (!aligned16(p->w2) || !aligned16(y) || !aligned16(workspace)) return PA_ERR_ALIGN;
    int rc = check_tail(tail);
    if (rc) return rc;
    if (workspace_bytes < pa::mlp::premlp_blob_bytes(F, C)) return PA_ERR_WORKSPACE;
    hipStream_t st = static_cast<hipStream_t>(stream);
    // the LayerNorm rides in the kernel's epilogue when a wave holds whole rows (C = 256) and nothing is added first
    const bool ln_inside = tail && tail->ln_out && !tail->residual && C == 256;
    rc = pa::mlp::premlp(rows, c_in, F, C, p->w1, p->b1, p->w2, p->b2, u, y, ln_inside ? tail->ln_gamma : nullptr,
                         ln_inside ? tail->ln_beta : nullptr, ln_inside ? tail->ln_eps : 0.f,
                         ln_inside ? tail->ln_out : nullptr, workspace, compute_units(), st);
    if (rc || ln_inside || !tail_active(tail)) return rc;
    pa_shape s{};
    s.B = 1;
    s.N = rows;
    s.C = C;
    s.H = 1;
    s.D = 1;
    s.S = 1;
    return pa::general::residual_ln(dtype, s, y, *tail, st);
  }
  if (!pa::f32rows::premlp_supported(dtype, rows, c_in, F, C)) return PA_ERR_UNSUPPORTED;
  if (!p || !p->w1 || !p->b1 || !p->w2 || !p->b2 || !u || !y || !workspace) return PA_ERR_NULL;
  if (!aligned16(p->w2) || !aligned16(y) || !aligned16(workspace)) return PA_ERR_ALIGN;
  int rc = check_tail(tail);
  if (rc) return rc;
  if (workspace_bytes < pa::f32rows::premlp_blob_bytes(F)) return PA_ERR_WORKSPACE;
  return pa::f32rows::premlp_forward(rows, c_in, F, p->w1, p->b1, p->w2, p->b2, u, y, tail_active(tail) ? tail : nullptr,
                                     workspace, static_cast<hipStream_t>(stream));
}

int pa_mfma_layer_forward(const pa_shape *shape, const pa_params *p, const void *blob, const void *x, void *y,
                          const pa_block_tail *tail, float *slice_token_out, void *workspace, int64_t workspace_bytes,
                          void *stream) {
  Range entry("pa_mfma_layer_forward");
  int rc = check_mfma(shape);
  if (rc) return rc;
  // the kernels sum fx_mid without its bias; the combine step adds bias * (sum of the weights) from p
  if (!p || !p->qkv_project_weight || !p->in_project_fx_bias || !blob || !x || !y || !workspace) return PA_ERR_NULL;
  if (!aligned16(blob) || !aligned16(x) || !aligned16(y) || !aligned16(workspace)) return PA_ERR_ALIGN;
  if ((rc = check_tail(tail))) return rc;
  if (mfma_layer_on_tiles(*shape)) {  // this sequence reads the parameters themselves, not the blob
    if (!p->in_project_x_weight || !p->in_project_x_bias || !p->in_project_fx_weight || !p->in_project_slice_weight ||
        !p->in_project_slice_bias || !p->temperature || !p->out_linear_weight || !p->out_linear_bias)
      return PA_ERR_NULL;
    if (!aligned16(p->in_project_x_weight) || !aligned16(p->in_project_fx_weight) || !aligned16(p->out_linear_weight))
      return PA_ERR_ALIGN;
  }
  const MfmaPlan mp = plan_mfma(*shape);
  if (workspace_bytes < mp.total) return PA_ERR_WORKSPACE;
  return mfma_layer(*shape, *p, blob, x, y, tail, slice_token_out, static_cast<char *>(workspace), mp,
                    static_cast<hipStream_t>(stream));
}

int pa_layer_forward(int dtype, const pa_shape *shape, const pa_params *p, const void *x, void *y,
                     const pa_block_tail *tail, float *slice_token_out, void *workspace, int64_t workspace_bytes,
                     void *stream) {
  Range entry("pa_layer_forward");
  int rc = check_shape(dtype, shape);
  if (rc) return rc;
  if ((rc = check_params(p))) return rc;
  if (!x || !y || !workspace) return PA_ERR_NULL;
  if (!aligned16(x) || !aligned16(y) || !aligned16(workspace)) return PA_ERR_ALIGN;
  if ((rc = check_tail(tail))) return rc;
  const pa_shape &s = *shape;
  hipStream_t st = static_cast<hipStream_t>(stream);

  char *ws = static_cast<char *>(workspace);
  pa_params local = *p;  // bf16 / float32: no scales, whatever the caller left in those fields
  if (dtype != PA_BF16_W8) {
    local.in_project_x_scale = local.in_project_fx_scale = local.out_linear_scale = nullptr;
    p = &local;
  } else {
    // fp8-e4m3 large weights.  Where the shape runs on kernels that take their weights as repacked operand fragments
    // (the fused MFMA kernels; the packed-tile sequence of the staged family) the repacking kernels read the e4m3
    // bytes and scales themselves, so the call does the same launches as with bf16 weights.  The remaining shapes
    // read weights in natural layout: for those the three matrices are first expanded to bf16 in the workspace tail.
    if (!p->in_project_x_scale || !p->in_project_fx_scale || !p->out_linear_scale) return PA_ERR_NULL;
    const int64_t body = body_bytes(PA_BF16, s);
    const int64_t one = round_up(s.H * s.D * s.C * 2, 256);
    if (workspace_bytes < body + 3 * one) return PA_ERR_WORKSPACE;
    dtype = PA_BF16;
    const bool packers_read_e4m3 =
        pa::mfma::supported(dtype, s) ||
        (pa::mfma::staged_supported(dtype, s) && s.conv_k == 0 && pa::mlp::linear_supported(dtype, s.B * s.N, s.C));
    if (!packers_read_e4m3) {
      char *w0 = ws + body;
      if ((rc = pa::general::dequant_e4m3(p->in_project_x_weight, p->in_project_x_scale, w0, s.H * s.D, s.C, st)))
        return rc;
      if ((rc = pa::general::dequant_e4m3(p->in_project_fx_weight, p->in_project_fx_scale, w0 + one, s.H * s.D, s.C, st)))
        return rc;
      if ((rc = pa::general::dequant_e4m3(p->out_linear_weight, p->out_linear_scale, w0 + 2 * one, s.C, s.H * s.D, st)))
        return rc;
      local.in_project_x_weight = w0;
      local.in_project_fx_weight = w0 + one;
      local.out_linear_weight = w0 + 2 * one;
      local.in_project_x_scale = local.in_project_fx_scale = local.out_linear_scale = nullptr;
      p = &local;
    }
  }
  if (pa::mfma::supported(dtype, s)) {
    const MfmaPlan mp = plan_mfma(s);
    if (workspace_bytes < mp.total) return PA_ERR_WORKSPACE;
    void *blob = ws + mp.off_blob;
    if ((rc = pa::mfma::pack_params(s, *p, blob, st))) return rc;
    return mfma_layer(s, *p, blob, x, y, tail, slice_token_out, ws, mp, st);
  }
  if (pa::mfma::staged_supported(dtype, s)) {
    const StagedPlan sp = plan_staged(s);
    if (workspace_bytes < sp.total) return PA_ERR_WORKSPACE;
    void *x_mid = ws + sp.off_x_mid, *fxp = ws + sp.off_fx, *tokp = ws + sp.off_tokp;
    float *partials = reinterpret_cast<float *>(ws + sp.off_partials);
    float *tok = slice_token_out ? slice_token_out : reinterpret_cast<float *>(ws + sp.off_tok);
    float *norm = reinterpret_cast<float *>(ws + sp.off_norm);
    float *tok_out = reinterpret_cast<float *>(ws + sp.off_tok_out);
    if (s.conv_k == 0 && pa::mlp::linear_supported(dtype, s.B * s.N, s.C)) {
      // every stage on packed tiles of 32 points: projections, token sums, hand-back, out_linear with the tail
      char *blob = ws + sp.off_wout;
      if ((rc = pa::mlp::project_packed(s.B, s.N, s.C, p->in_project_x_weight, p->in_project_x_scale,
                                        p->in_project_x_bias, p->in_project_fx_weight, p->in_project_fx_scale,
                                        p->in_project_fx_bias, x, x_mid, fxp, blob, compute_units(), st)))
        return rc;
      if ((rc = pa::mfma::slice_softmax_reduce(s, *p, x_mid, true, fxp, partials, compute_units(), st))) return rc;
      if ((rc = pa::mfma::combine_attention(s, *p, nullptr, partials, sp.G, tok, norm, tok_out, tokp, st))) return rc;
      if ((rc = pa::mfma::deslice_recompute(s, *p, x_mid, true, tokp, x_mid, compute_units(), st))) return rc;
      return pa::mlp::linear_packed(s.B, s.N, s.C, p->out_linear_weight, p->out_linear_scale, p->out_linear_bias, x_mid, y,
                                    tail_active(tail) ? tail : nullptr, blob + 2 * pa::mlp::linear_blob_bytes(s.C),
                                    compute_units(), st);
    }
    if (staged_conv_on_tiles(s)) {
      // the same sequence behind the implicit-GEMM convolution kernel
      char *blob = ws + sp.off_wout;
      if ((rc = pa::mlp::conv_project_packed(s.B, s.N, s.C, s.grid_h, s.grid_w, s.grid_d, s.conv_k,
                                             (int)s.conv_tap_major, p->in_project_x_weight, p->in_project_x_bias,
                                             p->in_project_fx_weight, p->in_project_fx_bias, x, x_mid, fxp, blob,
                                             compute_units(), st)))
        return rc;
      if ((rc = pa::mfma::slice_softmax_reduce(s, *p, x_mid, true, fxp, partials, compute_units(), st))) return rc;
      if ((rc = pa::mfma::combine_attention(s, *p, nullptr, partials, sp.G, tok, norm, tok_out, tokp, st))) return rc;
      if ((rc = pa::mfma::deslice_recompute(s, *p, x_mid, true, tokp, x_mid, compute_units(), st))) return rc;
      return pa::mlp::linear_packed(s.B, s.N, s.C, p->out_linear_weight, nullptr, p->out_linear_bias, x_mid, y,
                                    tail_active(tail) ? tail : nullptr,
                                    blob + round_up(pa::mlp::conv_project_blob_bytes(s.C, conv_taps(s)), 256),
                                    compute_units(), st);
    }
    pa::GemmArgs a{};  // x -> x_mid (natural) and fx_mid (packed): two weight sets over the same rows
    a.in = x;
    a.w[0] = p->in_project_x_weight;
    a.w[1] = p->in_project_fx_weight;
    a.bias[0] = p->in_project_x_bias;
    a.bias[1] = p->in_project_fx_bias;
    a.out[0] = x_mid;
    a.out_pack[1] = fxp;
    a.M = s.B * s.N;
    a.N = (int)s.N;
    a.C = (int)s.C;
    a.gh = (int)s.grid_h;
    a.gw = (int)s.grid_w;
    a.gd = (int)s.grid_d;
    a.ks = (int)s.conv_k;
    a.w_tap_major = (int)s.conv_tap_major;
    a.K = s.conv_k > 0 ? (int)(s.conv_k * s.conv_k * (s.grid_d > 0 ? s.conv_k : 1) * s.C) : (int)s.C;
    a.O = (int)(s.H * 32);
    a.pack_tpb = (int)pa::mfma::tiles_per_batch(s);
    a.pack_heads = (int)s.H;
    if (!pa::gemm::serves(a, 2, 2)) return PA_ERR_UNSUPPORTED;
    if ((rc = pa::gemm::launch(a, 2, PA_BF16, st))) return rc;
    if ((rc = pa::mfma::slice_softmax_reduce(s, *p, x_mid, false, fxp, partials, compute_units(), st))) return rc;
    if ((rc = pa::mfma::combine_attention(s, *p, nullptr, partials, sp.G, tok, norm, tok_out, tokp, st))) return rc;
    void *out_x = x_mid;
    if ((rc = pa::mfma::deslice_recompute(s, *p, x_mid, false, tokp, out_x, compute_units(), st))) return rc;
    if (pa::mlp::linear_supported(dtype, s.B * s.N, s.C))  // out_linear, the residual and the LayerNorm in one pass
      return pa::mlp::linear(s.B * s.N, s.C, p->out_linear_weight, nullptr, p->out_linear_bias, out_x, y,
                             tail_active(tail) ? tail : nullptr, ws + sp.off_wout, compute_units(), st);
    if ((rc = pa::general::out_linear(dtype, s, *p, out_x, y, st))) return rc;
    if (tail_active(tail)) rc = pa::general::residual_ln(dtype, s, y, *tail, st);
    return rc;
  }
  const GeneralPlan plan = plan_general(dtype, s);
  if (workspace_bytes < plan.total) return PA_ERR_WORKSPACE;
  void *x_mid = ws + plan.off_x_mid, *fx_mid = ws + plan.off_fx_mid, *w = ws + plan.off_w;
  float *partials = reinterpret_cast<float *>(ws + plan.off_partials);
  float *tok = slice_token_out ? slice_token_out : reinterpret_cast<float *>(ws + plan.off_tok);
  float *norm = reinterpret_cast<float *>(ws + plan.off_norm);
  float *tok_out = reinterpret_cast<float *>(ws + plan.off_tok_out);

  if (plan.conv_front) {  // both convolutions, the slice softmax and the partial token sums in one launch
    if ((rc = pa::conv::front(s, *p, x, ws + plan.off_blob, w, partials,
                              plan.rows_back ? ws + plan.off_blob_out : nullptr, nullptr, st)))
      return rc;
  } else {
    if ((rc = pa::general::project_inputs(dtype, s, *p, x, x_mid, fx_mid, st))) return rc;
    if ((rc = pa::general::slice_softmax(dtype, s, *p, x_mid, w, st))) return rc;
    if ((rc = pa::general::slice_partial(dtype, s, w, fx_mid, partials, st))) return rc;
  }
  if ((rc = pa::general::combine_attention(s, *p, partials, plan.G, tok, norm, tok_out, st))) return rc;
  if (plan.rows_back)  // hand-back, out_linear, residual and LayerNorm in one launch
    return pa::f32rows::backend(s, *p, w, tok_out, y, tail_active(tail) ? tail : nullptr, ws + plan.off_blob_out,
                                plan.conv_front, st);
  void *out_x = x_mid;
  if ((rc = pa::general::deslice(dtype, s, w, tok_out, out_x, st))) return rc;
  if ((rc = pa::general::out_linear(dtype, s, *p, out_x, y, st))) return rc;
  if (tail_active(tail)) rc = pa::general::residual_ln(dtype, s, y, *tail, st);
  return rc;
}

int pa_block_query(int dtype, const pa_shape *shape, int64_t F) {
  if (check_shape(dtype, shape)) return 0;
  return pa::f32rows::block_supported(dtype, *shape, F) ? 1 : 0;
}

int64_t pa_block_workspace_bytes(int dtype, const pa_shape *shape, int64_t F) {
  int rc = check_shape(dtype, shape);
  if (rc) return rc;
  if (!pa::f32rows::block_supported(dtype, *shape, F)) return PA_ERR_UNSUPPORTED;
  return plan_general(dtype, *shape).total + round_up(pa::f32rows::block_blob_bytes(F), 256);
}

int pa_block_forward(int dtype, const pa_shape *shape, const pa_params *p, const pa_block_mlp *mlp, const void *x,
                     const void *fx_in, void *fx_out, const pa_block_tail *next, const pa_block_head *head,
                     void *workspace, int64_t workspace_bytes, void *stream) {
  Range entry("pa_block_forward");
  int rc = check_shape(dtype, shape);
  if (rc) return rc;
  if ((rc = check_params(p))) return rc;
  if (!mlp || !mlp->ln_gamma || !mlp->ln_beta || !mlp->w1 || !mlp->b1 || !mlp->w2 || !mlp->b2) return PA_ERR_NULL;
  if (!x || !fx_in || !fx_out || !workspace) return PA_ERR_NULL;
  if (!aligned16(x) || !aligned16(fx_in) || !aligned16(fx_out) || !aligned16(workspace) || !aligned16(mlp->w1) ||
      !aligned16(mlp->w2))
    return PA_ERR_ALIGN;
  if ((rc = check_tail(next))) return rc;
  if (next && next->residual) return PA_ERR_UNSUPPORTED;  // the block's own residual is fx1
  if (head) {  // behind the next LayerNorm, whose parameters must then be given (its output need not be stored)
    if (!head->weight || !head->out || !next || !next->ln_gamma || !next->ln_beta) return PA_ERR_NULL;
    if (head->O < 1 || head->O > 4) return PA_ERR_UNSUPPORTED;
    if (!aligned16(head->weight)) return PA_ERR_ALIGN;
  }
  const pa_shape &s = *shape;
  if (!pa::f32rows::block_supported(dtype, s, mlp->F)) return PA_ERR_UNSUPPORTED;
  const GeneralPlan plan = plan_general(dtype, s);
  if (workspace_bytes < plan.total + pa::f32rows::block_blob_bytes(mlp->F)) return PA_ERR_WORKSPACE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  char *ws = static_cast<char *>(workspace);
  void *x_mid = ws + plan.off_x_mid, *fx_mid = ws + plan.off_fx_mid, *w = ws + plan.off_w;
  float *partials = reinterpret_cast<float *>(ws + plan.off_partials);
  float *tok = reinterpret_cast<float *>(ws + plan.off_tok), *norm = reinterpret_cast<float *>(ws + plan.off_norm);
  float *tok_out = reinterpret_cast<float *>(ws + plan.off_tok_out);
  if (plan.conv_front) {
    if ((rc = pa::conv::front(s, *p, x, ws + plan.off_blob, w, partials, ws + plan.total, mlp, st))) return rc;
  } else {
    if ((rc = pa::general::project_inputs(dtype, s, *p, x, x_mid, fx_mid, st))) return rc;
    if ((rc = pa::general::slice_softmax(dtype, s, *p, x_mid, w, st))) return rc;
    if ((rc = pa::general::slice_partial(dtype, s, w, fx_mid, partials, st))) return rc;
  }
  if ((rc = pa::general::combine_attention(s, *p, partials, plan.G, tok, norm, tok_out, st))) return rc;
  return pa::f32rows::block_tail(s, *p, *mlp, w, tok_out, fx_in, fx_out, next, head, ws + plan.total, plan.conv_front,
                                 st);
}

// Workspace plan of the FLARE layer on the MFMA kernels.
struct FlarePlan {
  int64_t off_scores, off_v, off_wc, off_wr, off_partials, off_z, off_tokp, off_colmax, off_cmpart, off_out_x, off_blob, total;
  int64_t G;
};

static FlarePlan plan_flare(const pa_shape &s) {
  FlarePlan p{};
  p.G = mfma_groups(s, false);
  const int64_t tiles = s.B * pa::mfma::tiles_per_batch(s);
  int64_t off = 0;
  p.off_scores = off;  // later the natural-layout attention output (B, N, H*32)
  off += round_up(s.B * s.N * s.H * (s.S > 32 ? s.S : 32) * 2, 256);
  p.off_v = off;
  off += round_up(tiles * s.H * 2 * 1024, 256);
  p.off_wc = off;
  off += round_up(tiles * s.H * (s.S / 16) * 1024, 256);
  p.off_wr = off;
  off += round_up(tiles * s.H * (s.S / 16) * 1024, 256);
  p.off_partials = off;
  off += round_up((p.G + 1) * s.B * s.H * s.S * (s.D + 1) * 4, 256);
  p.off_z = off;
  off += round_up(s.B * s.H * s.S * s.D * 4, 256);
  p.off_tokp = off;
  off += round_up(pa::mfma::tokp_bytes(s), 256);
  p.off_colmax = off;
  off += round_up(s.B * s.H * s.S * 4, 256);
  p.off_cmpart = off;
  off += round_up(pa::flare::column_max_chunks(s) * s.B * s.H * s.S * 4, 256);
  p.off_out_x = p.off_scores;  // the scores are dead once both weight packs exist
  p.off_blob = off;            // the parameter blob of kernel (d)
  off += round_up(pa::mfma::blob_bytes(s), 256);
  p.total = off;
  return p;
}

static bool flare_mfma_supported(const pa_shape &s) {
  return pa::mfma::supported(PA_BF16, s) && s.B * s.N >= 4096;
}

int pa_flare_forward_mfma_supported(const pa_shape *shape) {
  if (check_shape(PA_BF16, shape)) return 0;
  return flare_mfma_supported(*shape) ? 1 : 0;
}

int64_t pa_flare_forward_mfma_workspace_bytes(const pa_shape *shape) {
  int rc = check_shape(PA_BF16, shape);
  if (rc) return rc;
  if (!flare_mfma_supported(*shape)) return PA_ERR_UNSUPPORTED;
  return plan_flare(*shape).total;
}

int pa_flare_forward_mfma(const pa_shape *shape, const void *scores_weight, const float *scores_bias,
                          const void *values_weight, const float *values_bias, const void *out_linear_weight,
                          const float *out_linear_bias, const void *x, void *y, const pa_block_tail *tail,
                          void *workspace, int64_t workspace_bytes, void *stream) {
  int rc = check_shape(PA_BF16, shape);
  if (rc) return rc;
  if (!scores_weight || !values_weight || !x || !y || !workspace) return PA_ERR_NULL;
  if (!aligned16(scores_weight) || !aligned16(values_weight) || !aligned16(out_linear_weight) || !aligned16(x) ||
      !aligned16(y) || !aligned16(workspace))
    return PA_ERR_ALIGN;
  if ((rc = check_tail(tail))) return rc;
  if (!out_linear_weight && tail_active(tail)) return PA_ERR_UNSUPPORTED;  // the tail follows out_linear
  const pa_shape &s = *shape;
  if (!flare_mfma_supported(s)) return PA_ERR_UNSUPPORTED;
  const FlarePlan fp = plan_flare(s);
  if (workspace_bytes < fp.total) return PA_ERR_WORKSPACE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  char *ws = static_cast<char *>(workspace);
  void *scores = ws + fp.off_scores, *vp = ws + fp.off_v, *wc = ws + fp.off_wc, *wr = ws + fp.off_wr;
  void *tokp = ws + fp.off_tokp, *out_x = out_linear_weight ? ws + fp.off_out_x : y;  // no out_linear: y is out_x
  float *partials = reinterpret_cast<float *>(ws + fp.off_partials), *z = reinterpret_cast<float *>(ws + fp.off_z);
  float *colmax = reinterpret_cast<float *>(ws + fp.off_colmax), *cmpart = reinterpret_cast<float *>(ws + fp.off_cmpart);
  pa::GemmArgs a{};  // scores A = x . W_a^T + b_a, natural layout (B, N, H*S)
  a.in = x;
  a.w[0] = scores_weight;
  a.bias[0] = scores_bias;
  a.out[0] = scores;
  a.M = s.B * s.N;
  a.N = (int)s.N;
  a.K = a.C = (int)s.C;
  a.O = (int)(s.H * s.S);
  if (!pa::gemm::serves(a, 1, 2)) return PA_ERR_UNSUPPORTED;
  if ((rc = pa::gemm::launch(a, 1, PA_BF16, st))) return rc;
  pa::GemmArgs v{};  // values, packed operand layout
  v.in = x;
  v.w[0] = values_weight;
  v.bias[0] = values_bias;
  v.out_pack[0] = vp;
  v.M = s.B * s.N;
  v.N = (int)s.N;
  v.K = v.C = (int)s.C;
  v.O = (int)(s.H * 32);
  v.pack_tpb = (int)pa::mfma::tiles_per_batch(s);
  v.pack_heads = (int)s.H;
  if (!pa::gemm::serves(v, 1, 2)) return PA_ERR_UNSUPPORTED;
  if ((rc = pa::gemm::launch(v, 1, PA_BF16, st))) return rc;
  if ((rc = pa::flare::column_max(PA_BF16, s, scores, cmpart, colmax, st))) return rc;
  if ((rc = pa::flare::pack_weights(s, scores, colmax, wc, wr, compute_units(), st))) return rc;
  if ((rc = pa::mfma::slice_reduce(s, wc, vp, partials, st))) return rc;
  const float *sums = nullptr;
  if ((rc = pa::general::combine_partials(s, partials, fp.G, &sums, st))) return rc;
  if ((rc = pa::flare::normalise(s, sums, z, st))) return rc;
  if ((rc = pa::gale::pack_tokens(s, z, tokp, st))) return rc;
  if (out_linear_weight && out_linear_bias && pa::mfma::supported(PA_BF16, s)) {
    // hand-back, out_linear and the block's tail in kernel (d)
    void *blob = ws + fp.off_blob;
    if ((rc = pa::mfma::pack_out_linear(s, out_linear_weight, nullptr, out_linear_bias, blob, st))) return rc;
    return pa::mfma::deslice_project(s, blob, wr, tokp, y, tail_active(tail) ? tail : nullptr, compute_units(), st);
  }
  if ((rc = pa::mfma::deslice_natural(s, wr, tokp, out_x, compute_units(), st))) return rc;
  if (!out_linear_weight) return PA_OK;
  pa_params po{};
  po.out_linear_weight = out_linear_weight;
  po.out_linear_bias = out_linear_bias;
  if ((rc = pa::general::out_linear(PA_BF16, s, po, out_x, y, st))) return rc;
  if (tail_active(tail)) rc = pa::general::residual_ln(PA_BF16, s, y, *tail, st);
  return rc;
}

int pa_layer_forward_plus_supported(int dtype, const pa_shape *shape) {
  if (check_shape(dtype, shape)) return 0;
  return pa::mfma::staged_supported(dtype, *shape) ? 1 : 0;
}

int64_t pa_layer_forward_plus_workspace_bytes(int dtype, const pa_shape *shape) {
  int rc = check_shape(dtype, shape);
  if (rc) return rc;
  if (!pa::mfma::staged_supported(dtype, *shape)) return PA_ERR_UNSUPPORTED;
  return plan_plus(*shape).total;
}

int pa_layer_forward_plus(int dtype, const pa_shape *shape, const pa_params *p, const pa_plus_params *plus,
                          const void *x, const void *uniform, void *y, const pa_block_tail *tail,
                          float *slice_token_out, void *workspace, int64_t workspace_bytes, void *stream) {
  Range entry("pa_layer_forward_plus");
  int rc = check_shape(dtype, shape);
  if (rc) return rc;
  if (!p || !plus || !x || !uniform || !y || !workspace) return PA_ERR_NULL;
  if (!p->in_project_x_weight || !p->in_project_slice_weight || !p->in_project_slice_bias || !p->temperature ||
      !p->qkv_project_weight || !p->out_linear_weight || !plus->proj_temperature_0_weight ||
      !plus->proj_temperature_0_bias || !plus->proj_temperature_2_weight || !plus->proj_temperature_2_bias)
    return PA_ERR_NULL;
  if (!aligned16(x) || !aligned16(uniform) || !aligned16(y) || !aligned16(workspace)) return PA_ERR_ALIGN;
  if ((rc = check_tail(tail))) return rc;
  const pa_shape &s = *shape;
  if (!pa::mfma::staged_supported(dtype, s)) return PA_ERR_UNSUPPORTED;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const PlusPlan sp = plan_plus(s);
  if (workspace_bytes < sp.total) return PA_ERR_WORKSPACE;
  char *ws = static_cast<char *>(workspace);
  void *x_mid = ws + sp.off_x_mid, *fxp = ws + sp.off_fx, *wp = ws + sp.off_w, *tokp = ws + sp.off_tokp;
  float *partials = reinterpret_cast<float *>(ws + sp.off_partials);
  float *tok = slice_token_out ? slice_token_out : reinterpret_cast<float *>(ws + sp.off_tok);
  float *norm = reinterpret_cast<float *>(ws + sp.off_norm);
  float *tok_out = reinterpret_cast<float *>(ws + sp.off_tok_out);
  pa::GemmArgs a{};  // x -> x_mid, natural layout for the slice weights and packed for the aggregation (fx_mid is x_mid)
  a.in = x;
  a.w[0] = p->in_project_x_weight;
  a.bias[0] = p->in_project_x_bias;
  a.out[0] = x_mid;
  a.out_pack[0] = fxp;
  a.M = s.B * s.N;
  a.N = (int)s.N;
  a.C = (int)s.C;
  a.gh = (int)s.grid_h;
  a.gw = (int)s.grid_w;
  a.gd = (int)s.grid_d;
  a.ks = (int)s.conv_k;
  a.w_tap_major = (int)s.conv_tap_major;
  a.K = s.conv_k > 0 ? (int)(s.conv_k * s.conv_k * (s.grid_d > 0 ? s.conv_k : 1) * s.C) : (int)s.C;
  a.O = (int)(s.H * 32);
  a.pack_tpb = (int)pa::mfma::tiles_per_batch(s);
  a.pack_heads = (int)s.H;
  if (!pa::gemm::serves(a, 1, 2)) return PA_ERR_UNSUPPORTED;
  if ((rc = pa::gemm::launch(a, 1, PA_BF16, st))) return rc;
  if ((rc = pa::mfma::slice_softmax_pack_plus(s, *p, *plus, x_mid, uniform, wp, compute_units(), st))) return rc;
  if ((rc = pa::mfma::slice_reduce(s, wp, fxp, partials, st))) return rc;
  if ((rc = pa::mfma::combine_attention(s, *p, nullptr, partials, sp.G, tok, norm, tok_out, tokp, st))) return rc;
  if (pa::mfma::supported(dtype, s) && p->out_linear_bias) {
    // hand-back, out_linear and the block's tail in kernel (d), which reads the out_linear part of the parameter blob
    void *blob = ws + sp.off_blob;
    if ((rc = pa::mfma::pack_out_linear(s, p->out_linear_weight, nullptr, p->out_linear_bias, blob, st))) return rc;
    return pa::mfma::deslice_project(s, blob, wp, tokp, y, tail_active(tail) ? tail : nullptr, compute_units(), st);
  }
  void *out_x = x_mid;
  if ((rc = pa::mfma::deslice_natural(s, wp, tokp, out_x, compute_units(), st))) return rc;
  if ((rc = pa::general::out_linear(dtype, s, *p, out_x, y, st))) return rc;
  if (tail_active(tail)) rc = pa::general::residual_ln(dtype, s, y, *tail, st);
  return rc;
}

}  // extern "C"
