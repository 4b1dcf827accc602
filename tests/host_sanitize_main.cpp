// Host-side checks of libphysattn's dispatch layer under AddressSanitizer + UndefinedBehaviorSanitizer.
// Built by tests/test_host_sanitized.py from the library's own sources with the sanitizers on the host pass only;
// no GPU is needed: every call here is answered by the shape / plan / validation code before anything would be
// enqueued (queries, workspace sizes over a wide grid of shapes including extreme ones, and the argument-error paths
// of the compute entry points).  Exit code 0 = every answer was well-formed and no sanitizer report was raised.
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "../include/physattn.h"

static int failures = 0;
#define CHECK(cond)                                              \
  do {                                                           \
    if (!(cond)) {                                               \
      ++failures;                                                \
      fprintf(stderr, "line %d: %s\n", __LINE__, #cond);         \
    }                                                            \
  } while (0)

static pa_shape make(int64_t B, int64_t N, int64_t C, int64_t H, int64_t D, int64_t S, int64_t gh = 0, int64_t gw = 0,
                     int64_t k = 0, int64_t gd = 0, int64_t tap = 0) {
  pa_shape s;
  memset(&s, 0, sizeof s);
  s.B = B; s.N = N; s.C = C; s.H = H; s.D = D; s.S = S;
  s.grid_h = gh; s.grid_w = gw; s.conv_k = k; s.grid_d = gd; s.conv_tap_major = tap;
  return s;
}

int main() {
  CHECK(pa_version() >= 100);
  for (int code = -32; code <= 1100; ++code) {
    const char *t = pa_status_string(code);
    CHECK(t != nullptr && strlen(t) > 0);
  }
  CHECK(pa_static_scratch_bytes() == PA_STATIC_SCRATCH_BYTES);
  CHECK(pa_markers_enabled() == 0 || pa_markers_enabled() == 1);

  // ---- queries and workspace sizes over a grid of shapes, extremes included ----
  const int64_t Bs[] = {-1, 0, 1, 2, 7, 1 << 20, (int64_t)1 << 40};
  const int64_t Ns[] = {-5, 0, 1, 31, 32, 33, 700, 4096, 28900, 1 << 20, PA_MAX_N, (int64_t)1 << 31, ((int64_t)1 << 31) + 1,
                        (int64_t)1 << 62};
  const int64_t Cs[] = {0, 1, 64, 128, 256, 512, 1 << 16, (1 << 16) + 1};
  const int64_t Hs[] = {0, 1, 4, 8, 16, 1024, 1025};
  const int64_t Ds[] = {0, 1, 16, 32, 64, 128, 129};
  const int64_t Ss[] = {0, 1, 16, 32, 64, 128, 256, 257};
  long long answered = 0;
  for (int dtype = -1; dtype <= 3; ++dtype)
    for (int64_t B : Bs)
      for (int64_t N : Ns)
        for (int64_t C : Cs)
          for (int64_t H : Hs)
            for (int64_t D : Ds)
              for (int64_t S : Ss) {
                const pa_shape s = make(B, N, C, H, D, S);
                const int path = pa_query_path(dtype, &s);
                const int64_t ws = pa_workspace_bytes(dtype, &s);
                CHECK(path <= 2);
                CHECK((path < 0) == (ws < 0));  // a shape is either served with a size or refused by both
                if (path >= 0) CHECK(ws >= 0);
                if (N > PA_MAX_N) CHECK(path < 0);
                const int64_t pc = pa_reduce_partial_count(&s);
                CHECK(pc != 0);
                (void)pa_backward_query(dtype, &s);
                (void)pa_backward_point_tiles(&s);
                (void)pa_backward_point_tiles_plus(&s);
                (void)pa_flare_column_max_chunks(&s);
                (void)pa_flare_forward_mfma_supported(&s);
                (void)pa_flare_forward_mfma_workspace_bytes(&s);
                for (int which = -1; which <= 5; ++which) (void)pa_mfma_buffer_bytes(&s, which);
                (void)pa_mfma_partial_groups(&s, 0);
                (void)pa_mfma_partial_groups(&s, 1);
                (void)pa_mfma_backward_query(&s);
                (void)pa_mfma_backward_tables_bytes(&s);
                (void)pa_mfma_backward_groups(&s);
                (void)pa_layer_forward_plus_supported(dtype, &s);
                (void)pa_layer_forward_plus_workspace_bytes(dtype, &s);
                for (int64_t F : {(int64_t)0, (int64_t)128, (int64_t)512, (int64_t)1024, (int64_t)1 << 40}) {
                  (void)pa_block_query(dtype, &s, F);
                  (void)pa_block_workspace_bytes(dtype, &s, F);
                }
                ++answered;
              }
  // structured grids: 2-D and 3-D, odd and even kernels, products that do and do not match N, both weight layouts
  for (int dtype = 0; dtype <= 2; ++dtype)
    for (int64_t k : {(int64_t)-1, (int64_t)0, (int64_t)1, (int64_t)2, (int64_t)3, (int64_t)5, (int64_t)7, (int64_t)1 << 20})
      for (int64_t gh : {(int64_t)-3, (int64_t)0, (int64_t)1, (int64_t)17, (int64_t)85, (int64_t)1 << 31})
        for (int64_t gw : {(int64_t)0, (int64_t)1, (int64_t)23, (int64_t)85})
          for (int64_t gd : {(int64_t)-1, (int64_t)0, (int64_t)1, (int64_t)9})
            for (int64_t tap : {(int64_t)-1, (int64_t)0, (int64_t)1, (int64_t)2})
              for (int64_t C : {(int64_t)64, (int64_t)128, (int64_t)256, (int64_t)512}) {
                const int64_t H = 8, D = C / 8 >= 16 ? (C == 128 ? 16 : 32) : 8;
                const int64_t n = gh * gw * (gd > 0 ? gd : 1);
                for (int64_t N : {n, n + 1}) {
                  const pa_shape s = make(4, N, C, H, D, 32, gh, gw, k, gd, tap);
                  const int path = pa_query_path(dtype, &s);
                  const int64_t ws = pa_workspace_bytes(dtype, &s);
                  CHECK((path < 0) == (ws < 0));
                  (void)pa_block_query(dtype, &s, 512);
                  (void)pa_block_workspace_bytes(dtype, &s, 512);
                  (void)pa_backward_query(dtype, &s);
                  ++answered;
                }
              }
  // row-count helpers
  for (int64_t rows : {(int64_t)-1, (int64_t)0, (int64_t)1, (int64_t)127, (int64_t)1 << 20, (int64_t)1 << 40, (int64_t)1 << 62})
    for (int64_t C : {(int64_t)-1, (int64_t)0, (int64_t)8, (int64_t)128, (int64_t)256, (int64_t)512, (int64_t)1 << 40}) {
      (void)pa_layernorm_backward_groups(rows);
      (void)pa_cols_gemm_chunks(rows, C);
      (void)pa_cols_gemm_f32_chunks(rows, C, C);
      for (int dtype = -1; dtype <= 3; ++dtype)
        for (int64_t F : {(int64_t)-64, (int64_t)0, (int64_t)64, (int64_t)100, (int64_t)1024, (int64_t)8192, (int64_t)1 << 40}) {
          const int q = pa_mlp_query(dtype, rows, C, F);
          const int64_t b = pa_mlp_workspace_bytes(dtype, rows, C, F);
          CHECK(q == 0 || q == 1);
          if (q == 1) CHECK(b > 0);
          for (int64_t c_in : {(int64_t)0, (int64_t)2, (int64_t)8, (int64_t)9}) {
            const int pq = pa_preprocess_query(dtype, rows, c_in, F, C);
            const int64_t pb = pa_preprocess_workspace_bytes(dtype, rows, c_in, F, C);
            CHECK(pq == 0 || pq == 1);
            if (pq == 1) CHECK(pb > 0);
          }
        }
    }

  // ---- argument errors of the compute entry points: answered before anything is enqueued ----
  alignas(16) static char buf[256];
  const pa_shape ok = make(1, 4096, 256, 8, 32, 64);
  pa_params p;
  memset(&p, 0, sizeof p);
  CHECK(pa_layer_forward(PA_BF16, nullptr, &p, buf, buf, nullptr, nullptr, buf, 1 << 20, nullptr) < 0);
  CHECK(pa_layer_forward(PA_BF16, &ok, nullptr, buf, buf, nullptr, nullptr, buf, 1 << 20, nullptr) < 0);
  CHECK(pa_layer_forward(PA_BF16, &ok, &p, buf, buf, nullptr, nullptr, buf, 1 << 20, nullptr) < 0);  // null parameters
  p.in_project_x_weight = p.in_project_fx_weight = p.out_linear_weight = buf;
  p.in_project_x_bias = p.in_project_fx_bias = p.in_project_slice_weight = p.in_project_slice_bias = p.temperature =
      p.qkv_project_weight = p.out_linear_bias = reinterpret_cast<const float *>(buf);
  CHECK(pa_layer_forward(PA_BF16, &ok, &p, nullptr, buf, nullptr, nullptr, buf, 1 << 20, nullptr) < 0);
  CHECK(pa_layer_forward(PA_BF16, &ok, &p, buf + 2, buf, nullptr, nullptr, buf, 1 << 20, nullptr) < 0);  // misaligned
  CHECK(pa_layer_forward(PA_BF16, &ok, &p, buf, buf, nullptr, nullptr, buf, 16, nullptr) < 0);           // workspace too small
  CHECK(pa_layer_forward(7, &ok, &p, buf, buf, nullptr, nullptr, buf, 1 << 20, nullptr) < 0);
  pa_block_tail tail;
  memset(&tail, 0, sizeof tail);
  tail.ln_out = buf;  // LayerNorm output asked for without its weight and bias
  CHECK(pa_layer_forward(PA_BF16, &ok, &p, buf, buf, &tail, nullptr, buf, (int64_t)1 << 40, nullptr) < 0);
  CHECK(pa_mfma_layer_forward(&ok, &p, nullptr, buf, buf, nullptr, nullptr, buf, 1 << 20, nullptr) < 0);
  CHECK(pa_mfma_layer_forward(&ok, &p, buf, buf, buf, nullptr, nullptr, buf, 16, nullptr) < 0);
  pa_mlp_params mp;
  memset(&mp, 0, sizeof mp);
  CHECK(pa_mlp_forward(PA_BF16, 4096, 256, 1024, &mp, buf, buf, nullptr, buf, 1 << 20, nullptr) < 0);
  CHECK(pa_mlp_forward(PA_BF16, 0, 256, 1024, &mp, buf, buf, nullptr, buf, 1 << 20, nullptr) < 0);
  CHECK(pa_mlp_forward(PA_BF16, 4096, 200, 1024, &mp, buf, buf, nullptr, buf, 1 << 20, nullptr) < 0);
  CHECK(pa_preprocess_forward(PA_F32, 4096, 2, 256, 128, &mp, buf, buf, nullptr, buf, 1 << 20, nullptr) < 0);
  CHECK(pa_preprocess_forward(PA_F32, 4096, 9, 256, 128, &mp, buf, buf, nullptr, buf, 1 << 20, nullptr) < 0);
  const pa_shape cfg1 = make(4, 85 * 85, 128, 8, 16, 32, 85, 85, 3, 0, 1);
  pa_block_mlp bm;
  memset(&bm, 0, sizeof bm);
  bm.F = 512;
  CHECK(pa_block_forward(PA_F32, &cfg1, &p, nullptr, buf, buf, buf, nullptr, nullptr, buf, 1 << 20, nullptr) < 0);
  CHECK(pa_block_forward(PA_F32, &cfg1, &p, &bm, buf, buf, buf, nullptr, nullptr, buf, 1 << 20, nullptr) < 0);
  CHECK(pa_block_forward(PA_BF16, &cfg1, &p, &bm, buf, buf, buf, nullptr, nullptr, buf, 1 << 20, nullptr) < 0);
  CHECK(pa_slice_reduce_static(PA_BF16, nullptr, buf, buf, reinterpret_cast<float *>(buf), reinterpret_cast<float *>(buf),
                               nullptr) < 0);
  const pa_shape big = make(1, (int64_t)1 << 20, 256, 8, 32, 128);
  CHECK(pa_slice_reduce_static(PA_BF16, &big, buf, buf, reinterpret_cast<float *>(buf), reinterpret_cast<float *>(buf),
                               nullptr) < 0);  // partial sums beyond the static array

  // the row GEMM entry point forms its grid products itself: extreme extents must be refused before any product
  for (int64_t gh : {(int64_t)1, (int64_t)85, (int64_t)1 << 31, (int64_t)1 << 40, (int64_t)1 << 62})
    for (int64_t gw : {(int64_t)1, (int64_t)85, (int64_t)1 << 31, (int64_t)1 << 62})
      for (int64_t gd : {(int64_t)0, (int64_t)7, (int64_t)1 << 31, (int64_t)1 << 62})
        for (int64_t k : {(int64_t)1, (int64_t)3, (int64_t)1 << 20, (int64_t)1 << 40}) {
          const pa_shape g = make(1, 85 * 85, 128, 8, 16, 32, gh, gw, k, gd, 0);
          const int rc = pa_rows_gemm_act(PA_F32, &g, 128, 128, nullptr, nullptr, nullptr, 0, nullptr, nullptr);
          CHECK(rc < 0);  // a bad grid, or (85 x 85, k = 1 / 3, no depth) the null tensors
        }
  // the fused layer needs in_project_fx_bias even with the parameters already repacked
  {
    pa_params q = p;
    q.in_project_fx_bias = nullptr;
    CHECK(pa_mfma_layer_forward(&ok, &q, buf, buf, buf, nullptr, nullptr, buf, (int64_t)1 << 40, nullptr) == PA_ERR_NULL);
    q = p;
    q.in_project_x_scale = reinterpret_cast<const float *>(buf);  // one scale of three
    CHECK(pa_mfma_pack_params(&ok, &q, buf, nullptr) == PA_ERR_NULL);
    CHECK(pa_mlp_pack_e4m3(256, 1024, buf, nullptr, buf, nullptr, buf, (int64_t)1 << 40, nullptr) == PA_ERR_NULL);
    CHECK(pa_mlp_pack_e4m3(256, (int64_t)1 << 40, buf, reinterpret_cast<const float *>(buf), buf,
                           reinterpret_cast<const float *>(buf), buf, (int64_t)1 << 40, nullptr) < 0);
  }

  printf("host sanitize: %lld shapes answered, %d failures\n", answered, failures);
  return failures == 0 ? 0 : 1;
}
