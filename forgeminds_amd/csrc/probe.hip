// STREAM-style bandwidth probe: the yardstick the row kernels are measured against.
//
// Two plain kernels with the same 16-byte non-temporal accesses the row kernels use: a
// read-only sweep and a copy. bench.py runs them to report the HBM ceiling this GPU actually
// reaches next to the published peak, and profiling runs use the copy (whose traffic is known
// exactly) to calibrate the FETCH_SIZE / WRITE_SIZE counters.
#include "fm_common.cuh"

using namespace fm;

namespace {

__global__ __launch_bounds__(1024) void probe_read_kernel(const u32x4* __restrict__ src,
                                                           uint32_t* __restrict__ sink,
                                                           int64_t nvec, int vec_per_block) {
  const u32x4* p = src + (int64_t)blockIdx.x * vec_per_block;
  int64_t left = nvec - (int64_t)blockIdx.x * vec_per_block;
  const int n = left < vec_per_block ? (int)left : vec_per_block;
  u32x4 acc = {0u, 0u, 0u, 0u};
  for (int c0 = 0; c0 < n; c0 += 1024 * 4) {
    u32x4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int c = c0 + u * 1024 + (int)threadIdx.x;
      v[u] = c < n ? load16_stream(p + c) : acc;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) acc ^= v[u];
  }
  // never true for the probe's fill pattern; keeps the loads alive
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x9e3779b9u) sink[0] = acc[0];
}

__global__ __launch_bounds__(1024) void probe_copy_kernel(const u32x4* __restrict__ src,
                                                           u32x4* __restrict__ dst, int64_t nvec,
                                                           int vec_per_block) {
  const int64_t base = (int64_t)blockIdx.x * vec_per_block;
  const int64_t left = nvec - base;
  const int n = left < vec_per_block ? (int)left : vec_per_block;
  for (int c0 = 0; c0 < n; c0 += 1024 * 4) {
    u32x4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int c = c0 + u * 1024 + (int)threadIdx.x;
      if (c < n) v[u] = load16_stream(src + base + c);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int c = c0 + u * 1024 + (int)threadIdx.x;
      if (c < n) store16_stream(dst + base + c, v[u]);
    }
  }
}

}  // namespace

extern "C" int fm_stream_probe(const void* src, void* dst, uint32_t* sink, size_t bytes, int mode,
                               fm_stream_t stream) {
  FM_CHECK_ARG(src != nullptr && bytes >= 16 && bytes % 16 == 0, "fm_stream_probe: bad buffer");
  FM_CHECK_ARG(mode == 0 || mode == 1, "fm_stream_probe: mode is 0 (read) or 1 (copy)");
  FM_CHECK_ARG(fm_host::aligned16(src) && fm_host::aligned16(dst), "fm_stream_probe: unaligned");
  FM_CHECK_ARG((mode == 0 && sink != nullptr) || (mode == 1 && dst != nullptr),
               "fm_stream_probe: missing output");
  const int64_t nvec = (int64_t)(bytes / 16);
  const int vec_per_block = 4096;   // 64 KiB per workgroup, the size of one 32000-logit bf16 row
  const int64_t blocks = (nvec + vec_per_block - 1) / vec_per_block;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (mode == 0)
    hipLaunchKernelGGL(probe_read_kernel, dim3((unsigned)blocks), dim3(1024), 0, st,
                       static_cast<const u32x4*>(src), sink, nvec, vec_per_block);
  else
    hipLaunchKernelGGL(probe_copy_kernel, dim3((unsigned)blocks), dim3(1024), 0, st,
                       static_cast<const u32x4*>(src), static_cast<u32x4*>(dst), nvec, vec_per_block);
  FM_CHECK_LAUNCH("fm_stream_probe");
  return FM_OK;
}
