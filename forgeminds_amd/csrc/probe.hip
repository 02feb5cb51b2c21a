// STREAM-style bandwidth probe: the yardstick the row kernels are measured against.
//
// Two plain kernels with the same 16-byte non-temporal accesses the row kernels use: a
// read-only sweep and a copy. bench.py runs them to report the HBM ceiling this GPU actually
// reaches next to the published peak, and profiling runs use the copy (whose traffic is known
// exactly) to calibrate the FETCH_SIZE / WRITE_SIZE counters.
//
// A third kernel, probe_mix_kernel, sweeps up to three input streams and up to two output
// streams of equal size with no arithmetic beyond an xor: the floor of a row kernel with the
// same read / write mix, the same bytes and the same store kinds. bench.py times it on each
// workload's own buffers and reports the workload's time as a fraction of that floor.
#include "fm_common.hip.h"

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

// R input streams, W output streams, every stream `nvec` 16-byte vectors. A workgroup moves tiles
// of THREADS * U vectors (U vectors of every input per thread in flight before the first store),
// tile, tile + gridDim.x, ... Loads are non-temporal; `store_kind`: 0 plain, 1 non-temporal,
// 2 first output plain and second non-temporal. nvec is a whole number of tiles (checked on the
// host), so no access is predicated.
template <int THREADS, int U, int R, int W>
__global__ __launch_bounds__(THREADS) void probe_mix_kernel(
    const u32x4* __restrict__ a, const u32x4* __restrict__ b, const u32x4* __restrict__ c,
    u32x4* __restrict__ o1, u32x4* __restrict__ o2, uint32_t* __restrict__ sink, int64_t tiles,
    int store_kind) {
  u32x4 keep = {0u, 0u, 0u, 0u};
  for (int64_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
    const int64_t base = tile * (THREADS * U) + threadIdx.x;
    u32x4 v[U], w[R > 1 ? U : 1], z[R > 2 ? U : 1];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      v[u] = load16_stream(a + base + u * THREADS);
      if constexpr (R > 1) w[u] = load16_stream(b + base + u * THREADS);
      if constexpr (R > 2) z[u] = load16_stream(c + base + u * THREADS);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      u32x4 r = v[u];
      if constexpr (R > 1) r ^= w[u];
      if constexpr (R > 2) r += z[u];
      if constexpr (W == 0) keep ^= r;
      if constexpr (W >= 1) {
        if (store_kind == 1) store16_stream(o1 + base + u * THREADS, r);
        else store16(o1 + base + u * THREADS, r);
      }
      if constexpr (W >= 2) {
        if (store_kind == 0) store16(o2 + base + u * THREADS, r ^ v[u]);
        else store16_stream(o2 + base + u * THREADS, r ^ v[u]);
      }
    }
  }
  if constexpr (W == 0) {
    // never true for the probe's inputs in practice; keeps the loads alive
    if ((keep[0] ^ keep[1] ^ keep[2] ^ keep[3]) == 0x9e3779b9u && sink != nullptr) sink[0] = keep[0];
  }
}

template <int THREADS, int U>
int launch_mix(int reads, int writes, const u32x4* a, const u32x4* b, const u32x4* c, u32x4* o1,
               u32x4* o2, uint32_t* sink, int64_t tiles, int store_kind, int64_t grid,
               hipStream_t st) {
#define GO(R_, W_)                                                                              \
  if (reads == R_ && writes == W_) {                                                            \
    hipLaunchKernelGGL((probe_mix_kernel<THREADS, U, R_, W_>), dim3((unsigned)grid), dim3(THREADS), 0, \
                       st, a, b, c, o1, o2, sink, tiles, store_kind);                           \
    return FM_OK;                                                                               \
  }
  GO(1, 0) GO(2, 0) GO(3, 0) GO(1, 1) GO(2, 1) GO(3, 1) GO(1, 2) GO(2, 2) GO(3, 2)
#undef GO
  fm_host::set_error("fm_stream_probe_mix: no kernel for %d reads + %d writes", reads, writes);
  return FM_ERR_UNSUPPORTED;
}

}  // namespace

extern "C" int fm_stream_probe_mix(const void* a, const void* b, const void* c, void* o1, void* o2,
                                   uint32_t* sink, size_t bytes, int reads, int writes,
                                   int store_kind, int threads, int vecs_per_thread, int64_t grid,
                                   fm_stream_t stream) {
  const char* what = "fm_stream_probe_mix";
  FM_CHECK_ARG(reads >= 1 && reads <= 3 && writes >= 0 && writes <= 2, "%s: 1-3 reads, 0-2 writes", what);
  FM_CHECK_ARG(store_kind >= 0 && store_kind <= 2, "%s: store_kind is 0, 1 or 2", what);
  FM_CHECK_ARG(a != nullptr && (reads < 2 || b != nullptr) && (reads < 3 || c != nullptr) &&
                   (writes < 1 || o1 != nullptr) && (writes < 2 || o2 != nullptr) &&
                   (writes > 0 || sink != nullptr),
               "%s: NULL stream", what);
  FM_CHECK_ARG(fm_host::aligned16(a) && fm_host::aligned16(b) && fm_host::aligned16(c) &&
                   fm_host::aligned16(o1) && fm_host::aligned16(o2),
               "%s: unaligned", what);
  const int64_t tile_bytes = (int64_t)threads * vecs_per_thread * 16;
  FM_CHECK_ARG(tile_bytes > 0 && bytes >= (size_t)tile_bytes && bytes % (size_t)tile_bytes == 0,
               "%s: bytes must be a whole number of tiles of threads * vecs_per_thread * 16", what);
  const int64_t tiles = (int64_t)(bytes / (size_t)tile_bytes);
  if (grid <= 0 || grid > tiles) grid = tiles;
  FM_CHECK_ARG(grid <= 0x7fffffffLL, "%s: grid too large", what);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const u32x4* ap = static_cast<const u32x4*>(a);
  const u32x4* bp = static_cast<const u32x4*>(b);
  const u32x4* cp = static_cast<const u32x4*>(c);
  u32x4* p1 = static_cast<u32x4*>(o1);
  u32x4* p2 = static_cast<u32x4*>(o2);
  int rc = FM_OK;
  bool known = false;
#define SHAPE(T_, U_)                                                                        \
  if (threads == T_ && vecs_per_thread == U_) {                                              \
    known = true;                                                                            \
    rc = launch_mix<T_, U_>(reads, writes, ap, bp, cp, p1, p2, sink, tiles, store_kind, grid, st); \
  }
  SHAPE(256, 1) SHAPE(256, 2) SHAPE(256, 4) SHAPE(512, 2) SHAPE(512, 4) SHAPE(1024, 1) SHAPE(1024, 4)
#undef SHAPE
  if (!known) {
    fm_host::set_error("%s: threads x vecs_per_thread is one of 256x1, 256x2, 256x4, 512x2, 512x4, "
                       "1024x1, 1024x4", what);
    return FM_ERR_UNSUPPORTED;
  }
  if (rc != FM_OK) return rc;
  FM_CHECK_LAUNCH(what);
  return FM_OK;
}

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
