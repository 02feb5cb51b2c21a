// Library-wide host plumbing: version, thread-local error text, tuning parameters and the
// cached compute-unit count. No kernels live here.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <atomic>

#include "fm_common.cuh"

namespace {
thread_local char g_error[512] = "";
std::atomic<int> g_params[fm_host::P_COUNT];
const char* const kParamNames[fm_host::P_COUNT] = {
    "norm_bwd_blocks_per_cu",
    "vocab_threads",
    "norm_tpr",
    "topk_variant",
    "vocab_unroll",
    "norm_fwd_blocks_per_cu",
    "ce_rows_max_v",
    "norm_wide_min_vec",
    "rows_vec_max",
};
constexpr int kMaxDevices = 64;
std::atomic<int> g_cus[kMaxDevices];
}  // namespace

namespace fm_host {

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

int get_param(int which) {
  if (which < 0 || which >= P_COUNT) return 0;
  return g_params[which].load(std::memory_order_relaxed);
}

int num_cus() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
  int c = g_cus[dev].load(std::memory_order_relaxed);
  if (c > 0) return c;
  int v = 0;
  if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0)
    v = 256;
  g_cus[dev].store(v, std::memory_order_relaxed);
  return v;
}

}  // namespace fm_host

extern "C" {

int fm_version(void) { return 1; }

const char* fm_last_error(void) { return g_error; }

int fm_set_param(const char* name, int value) {
  if (name == nullptr) {
    fm_host::set_error("fm_set_param: name is NULL");
    return FM_ERR_INVALID;
  }
  for (int i = 0; i < fm_host::P_COUNT; ++i) {
    if (strcmp(name, kParamNames[i]) == 0) {
      g_params[i].store(value > 0 ? value : 0, std::memory_order_relaxed);
      return FM_OK;
    }
  }
  fm_host::set_error("fm_set_param: unknown parameter '%s'", name);
  return FM_ERR_INVALID;
}

}  // extern "C"
