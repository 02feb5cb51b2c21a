// LayerNorm and fused residual-add + LayerNorm, forward and backward, for gfx950.
//
// Semantics: torch.nn.functional.layer_norm in fp32 on the stored values with one rounding at
// the store -- the same rounding rule the reference applies to RMSNorm
// (forgemind/kernels/_fallback.py:15-35); the reference has no LayerNorm kernel of its own.
//   mean = sum(x)/d, rstd = rsqrt(sum((x-mean)^2)/d + eps), y = ((x-mean)*rstd)*w + b
//   dx = ((g - mean(g)) - xhat*mean(g*xhat))*rstd with g = dy*w; dw = sum_rows dy*xhat;
//   db = sum_rows dy.
// Kernels: fm_norm.hip.h with LN = true.
#include "fm_norm.hip.h"

extern "C" {

int fm_layernorm_fwd(const void* x, const void* w, const void* bias, void* y, float* mean, float* rstd,
                     int64_t n, int64_t d, int x_dtype, int w_dtype, float eps, fm_stream_t stream) {
  return fwd_entry<false, true>("fm_layernorm_fwd", x, nullptr, w, bias, nullptr, y, mean, rstd, n, d,
                                x_dtype, w_dtype, eps, stream);
}

int fm_add_layernorm_fwd(const void* x, const void* delta, const void* w, const void* bias, void* xn,
                         void* y, float* mean, float* rstd, int64_t n, int64_t d, int x_dtype,
                         int w_dtype, float eps, fm_stream_t stream) {
  return fwd_entry<true, true>("fm_add_layernorm_fwd", x, delta, w, bias, xn, y, mean, rstd, n, d, x_dtype,
                               w_dtype, eps, stream);
}

size_t fm_layernorm_bwd_workspace(int64_t n, int64_t d, int x_dtype) {
  return bwd_workspace_bytes(n, d, x_dtype, true);
}

int fm_layernorm_bwd(const void* x, const void* w, const float* mean, const float* rstd, const void* dy,
                     const void* gxn, void* dx, void* dw, void* db, void* workspace,
                     size_t workspace_bytes, int64_t n, int64_t d, int x_dtype, int w_dtype,
                     fm_stream_t stream) {
  return bwd_entry<true>("fm_layernorm_bwd", x, w, mean, rstd, dy, gxn, dx, nullptr, dw, db, workspace,
                         workspace_bytes, n, d, x_dtype, w_dtype, stream);
}

}  // extern "C"
