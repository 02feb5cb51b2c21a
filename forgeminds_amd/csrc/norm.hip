// RMSNorm and fused residual-add + RMSNorm, forward and backward, for gfx950.
//
// Reference semantics: forgemind/kernels/_fallback.py:26-35 (forward, rounding points),
// forgemind/kernels/norm.py:179-231 (backward row math), norm.py:571-593 (fixed-order
// column sum of the fp32 weight-gradient partials). Kernels: fm_norm.cuh with LN = false.
#include "fm_norm.cuh"

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

int fm_add_rmsnorm_bwd(const void* xn, const void* w, const float* rstd, const void* gy,
                       const void* gxn, void* dx, void* ddelta, void* dw, void* workspace,
                       size_t workspace_bytes, int64_t n, int64_t d, int x_dtype, int w_dtype,
                       fm_stream_t stream) {
  return bwd_entry<false>("fm_add_rmsnorm_bwd", xn, w, nullptr, rstd, gy, gxn, dx, ddelta, dw, nullptr,
                          workspace, workspace_bytes, n, d, x_dtype, w_dtype, stream);
}

}  // extern "C"
