// pa_slice_reduce_static: stage (b), the slice-token aggregation, for callers that cannot allocate device memory
// (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  Same kernels as
// pa_slice_reduce; the per-chunk partial sums between its two passes live in a file-scope device array instead of a
// caller-provided buffer.  Every GPU the library runs on holds its own copy of that array until the process ends.
//
// Calls on one GPU share that GPU's array: two calls that overlap in time on the same GPU (different streams or
// threads) race on it.  Nothing in it has to start at zero -- the first pass writes every partial slot it later reads.
#include <mutex>

#include "pa_common.h"
#include "pa_host.h"

namespace {

static __device__ __align__(256) unsigned char scratch[PA_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
std::mutex g_lock;
void *g_scratch_ptr[kMaxDevices];  // device address of `scratch` on each GPU, looked up once per device

// Device address of this GPU's copy of `scratch` (the array's name itself is only a host-side handle).
int scratch_of_current_device(void **out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kMaxDevices) return PA_ERR_UNSUPPORTED;
  std::lock_guard<std::mutex> guard(g_lock);
  if (!g_scratch_ptr[dev]) {
    void *ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (!ptr) return PA_ERR_NULL;
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return PA_OK;
}

int64_t partial_bytes(const pa_shape &s) {
  return (pa::general::partial_count(s) + 1) * s.B * s.H * s.S * (s.D + 1) * 4;
}

}  // namespace

extern "C" {

int64_t pa_static_scratch_bytes(void) { return PA_STATIC_SCRATCH_BYTES; }

int pa_slice_reduce_static(int dtype, const pa_shape *shape, const void *w, const void *fx_mid, float *slice_token,
                           float *slice_norm, void *stream) {
  if (!shape) return PA_ERR_NULL;
  if (dtype != PA_F32 && dtype != PA_BF16) return PA_ERR_UNSUPPORTED;
  const pa_shape &s = *shape;
  if (s.B <= 0 || s.N <= 0 || s.H <= 0 || s.D <= 0 || s.S <= 0) return PA_ERR_DIMS;
  if (s.D > PA_MAX_D || s.S > PA_MAX_S || s.N > PA_MAX_N || s.B * s.H > 65535) return PA_ERR_UNSUPPORTED;
  if (pa::general::combine_attn_lds_bytes(s) > pa::kMaxLdsBytes) return PA_ERR_UNSUPPORTED;
  if (!w || !fx_mid || !slice_token || !slice_norm) return PA_ERR_NULL;
  if (!pa::aligned16(w) || !pa::aligned16(fx_mid)) return PA_ERR_ALIGN;
  if (partial_bytes(s) > PA_STATIC_SCRATCH_BYTES) return PA_ERR_SCRATCH;
  void *ptr = nullptr;
  int rc = scratch_of_current_device(&ptr);
  if (rc) return rc;
  float *partials = static_cast<float *>(ptr);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if ((rc = pa::general::slice_partial(dtype, s, w, fx_mid, partials, st))) return rc;
  pa_params none{};  // the combine kernel also serves the slice attention; only its token / norm outputs are wanted
  return pa::general::combine_attention(s, none, partials, pa::general::partial_count(s), slice_token, slice_norm, nullptr,
                                        st);
}

}  // extern "C"
