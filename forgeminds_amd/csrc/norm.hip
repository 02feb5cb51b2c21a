// RMSNorm and fused residual-add + RMSNorm, forward and backward, for gfx950.
//
// Reference semantics: forgemind/kernels/_fallback.py:26-35 (forward, rounding points),
// forgemind/kernels/norm.py:179-231 (backward row math), norm.py:571-593 (fixed-order
// column sum of the fp32 weight-gradient partials). Kernels: fm_norm.hip.h with LN = false.
#include "fm_norm.hip.h"

#include <atomic>

namespace {

// Scratch of fm_rmsnorm_bwd_static: the fp32 partial weight-gradient rows that the other
// backward entry points take from the caller's workspace. One copy per GPU, held until the
// process ends. 8 MiB covers every shape of the register and streamed paths up to d = 8192
// (at most 256 partial rows of d floats).
constexpr size_t kStaticScratchBytes = FM_RMSNORM_BWD_STATIC_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// `scratch` is only a host-side handle: the device address is asked for once per device and
// kept here; every launch gets this pointer, never the array's name.
constexpr int kMaxScratchDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxScratchDevices];

int static_scratch(const char* what, void** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxScratchDevices) {
    fm_host::set_error("%s: no usable current device (%s)", what, hipGetErrorString(e));
    return FM_ERR_INVALID;
  }
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr) {
      fm_host::set_error("%s: hipGetSymbolAddress(scratch) failed on device %d: %s", what, dev,
                         hipGetErrorString(e));
      return FM_ERR_LAUNCH;
    }
    g_scratch_ptr[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return FM_OK;
}

}  // namespace

extern "C" {

int fm_rmsnorm_fwd(const void* x, const void* w, void* y, float* rstd, int64_t n, int64_t d,
                   int x_dtype, int w_dtype, float eps, fm_stream_t stream) {
  return fwd_entry<false, false>("fm_rmsnorm_fwd", x, nullptr, w, nullptr, nullptr, y, nullptr, rstd, n, d,
                                 x_dtype, w_dtype, eps, stream);
}

int fm_add_rmsnorm_fwd(const void* x, const void* delta, const void* w, void* xn, void* y,
                       float* rstd, int64_t n, int64_t d, int x_dtype, int w_dtype, float eps,
                       fm_stream_t stream) {
  return fwd_entry<true, false>("fm_add_rmsnorm_fwd", x, delta, w, nullptr, xn, y, nullptr, rstd, n, d,
                                x_dtype, w_dtype, eps, stream);
}

size_t fm_rmsnorm_bwd_workspace(int64_t n, int64_t d, int x_dtype) {
  return bwd_workspace_bytes(n, d, x_dtype, false);
}

int fm_rmsnorm_bwd(const void* x, const void* w, const float* rstd, const void* dy, void* dx,
                   void* dw, void* workspace, size_t workspace_bytes, int64_t n, int64_t d,
                   int x_dtype, int w_dtype, fm_stream_t stream) {
  return bwd_entry<false>("fm_rmsnorm_bwd", x, w, nullptr, rstd, dy, nullptr, dx, nullptr, dw, nullptr,
                          workspace, workspace_bytes, n, d, x_dtype, w_dtype, stream);
}

int fm_rmsnorm_bwd_static(const void* x, const void* w, const float* rstd, const void* dy, void* dx,
                          void* dw, int64_t n, int64_t d, int x_dtype, int w_dtype,
                          fm_stream_t stream) {
  const char* what = "fm_rmsnorm_bwd_static";
  int rc = check_common(what, n, d, x_dtype, w_dtype);
  if (rc != FM_OK) return rc;
  void* ws = nullptr;
  size_t need = 0;
  if (dw != nullptr && n > 0) {
    need = bwd_workspace_bytes(n, d, x_dtype, false);
    if (need > kStaticScratchBytes) {
      fm_host::set_error("%s: n=%lld d=%lld needs %zu bytes of scratch, the built-in buffer holds %zu; "
                         "use fm_rmsnorm_bwd with a workspace of the caller's",
                         what, (long long)n, (long long)d, need, kStaticScratchBytes);
      return FM_ERR_UNSUPPORTED;
    }
    rc = static_scratch(what, &ws);
    if (rc != FM_OK) return rc;
  }
  return bwd_entry<false>(what, x, w, nullptr, rstd, dy, nullptr, dx, nullptr, dw, nullptr, ws,
                          ws != nullptr ? kStaticScratchBytes : 0, n, d, x_dtype, w_dtype, stream);
}

int fm_add_rmsnorm_bwd(const void* xn, const void* w, const float* rstd, const void* gy,
                       const void* gxn, void* dx, void* ddelta, void* dw, void* workspace,
                       size_t workspace_bytes, int64_t n, int64_t d, int x_dtype, int w_dtype,
                       fm_stream_t stream) {
  return bwd_entry<false>("fm_add_rmsnorm_bwd", xn, w, nullptr, rstd, gy, gxn, dx, ddelta, dw, nullptr,
                          workspace, workspace_bytes, n, d, x_dtype, w_dtype, stream);
}

}  // extern "C"
