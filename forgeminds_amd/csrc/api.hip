// Library-wide host plumbing: version, thread-local error text, tuning parameters and the
// cached compute-unit count. No kernels live here.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>
#include <stdlib.h>
#include <cxxabi.h>

#include <atomic>

#include "fm_common.hip.h"

namespace {
thread_local char g_error[512] = "";
thread_local const void* g_kernel = nullptr;     // host-side handle of the last main kernel
thread_local char g_kernel_text[384] = "";
std::atomic<int> g_params[fm_host::P_COUNT];
const char* const kParamNames[fm_host::P_COUNT] = {
    "norm_bwd_blocks_per_cu",
    "norm_fwd_blocks_per_cu",
    "vocab_threads",
    "vocab_unroll",
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

void note_kernel(const void* host_function) { g_kernel = host_function; }

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

const char* fm_last_kernel(void) {
  // "void (anonymous namespace)::ce_bwd_kernel<fm::bf16_t, 1024, 4>(fm::bf16_t const*, ...)"
  //   -> "ce_bwd_kernel<bf16_t, 1024, 4>"
  g_kernel_text[0] = 0;
  if (g_kernel == nullptr) return g_kernel_text;
  const char* mangled = hipKernelNameRefByPtr(g_kernel, nullptr);
  if (mangled == nullptr) return g_kernel_text;
  int status = 0;
  char* full = abi::__cxa_demangle(mangled, nullptr, nullptr, &status);
  const char* a = (status == 0 && full != nullptr) ? full : mangled;
  if (strncmp(a, "void ", 5) == 0) a += 5;
  size_t o = 0;
  int depth = 0;
  static const char* const kDrop[] = {"(anonymous namespace)::", "fm::"};
  while (*a != 0 && o + 1 < sizeof(g_kernel_text)) {
    bool dropped = false;
    for (const char* d : kDrop) {
      const size_t n = strlen(d);
      if (strncmp(a, d, n) == 0) { a += n; dropped = true; break; }
    }
    if (dropped) continue;
    if (*a == '<') ++depth;
    if (*a == '>') --depth;
    if (*a == '(' && depth == 0) break;       // the parameter list
    g_kernel_text[o++] = *a++;
  }
  g_kernel_text[o] = 0;
  free(full);
  return g_kernel_text;
}

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
