// Token movement around the expert dispatch permutation, for gfx950.
//
// Reference semantics: forgemind/moe.py:234-235 (xs = x[order // k]: tokens gathered into
// expert-grouped order) and moe.py:247-248 (ys * w[order], then index_add_ back to tokens).
// With the `slot` array of fm_route (slot[p] = grouped position of flat assignment p) the
// scatter-add becomes a gather per token: out[t] = sum_j w[t,j] * ys[slot[t*k+j]], summed in
// fp32 in j order and rounded once -- no atomics, deterministic, and each output row is
// written exactly once. The same two kernels serve the backward passes: the gradient of the
// gather is a combine with unit weights, the gradient of the combine is a weighted gather.
//
// Pure HBM-bound row moves: one workgroup per destination row, 16-byte vectors.
#include "fm_common.hip.h"

using namespace fm;

namespace {

constexpr int kMaxK = 16;   // the kernels keep a token's slots in registers: built for 8 and for 16

// dst[s, :] = scale * src[order[s] / k, :],  scale = w[order[s]] if w else 1
// A destination row is owned by `g` threads (a power of two up to 256: as many as the row has
// 16-byte vectors), 256 / g rows per workgroup.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void gather_kernel(const T* __restrict__ src,
                                                      const int32_t* __restrict__ order,
                                                      const float* __restrict__ w,
                                                      T* __restrict__ dst, int64_t total, int d, int k,
                                                      int g) {
  constexpr int EPV = Elem<T>::kVec;
  const int rib = threadIdx.x / g, l = threadIdx.x % g;
  const int64_t s = (int64_t)blockIdx.x * (256 / g) + rib;
  if (s >= total) return;
  const int p = order[s];
  const int64_t t = p / k;
  const float scale = w != nullptr ? w[p] : 1.f;
  const T* sp = src + t * (int64_t)d;
  T* dp = dst + s * (int64_t)d;
  if constexpr (VEC) {
    const int nvec = d / EPV;
    // four loads in flight per thread: a row is a few vectors per thread, and one load at a
    // time leaves the memory system idle between a load and its store
    for (int c0 = l; c0 < nvec; c0 += 4 * g) {
      u32x4 raw[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int c = c0 + u * g;
        if (c < nvec) raw[u] = load16(sp + c * EPV);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int c = c0 + u * g;
        if (c < nvec) {
          if (w != nullptr) {
            float f[EPV];
            Elem<T>::unpack(raw[u], f);
#pragma unroll
            for (int e = 0; e < EPV; ++e) f[e] *= scale;
            raw[u] = Elem<T>::pack(f);
          }
          store16_stream(dp + c * EPV, raw[u]);
        }
      }
    }
  } else {
    for (int j = l; j < d; j += g) Elem<T>::store1(dp + j, Elem<T>::load1(sp + j) * scale);
  }
}

// The same move from the token's side: dst[slot[t*k + j], :] = scale * src[t, :] for j < k,
// scale = w[t*k + j] if w else 1. A token row is read once and written k times (the gather
// above reads it k times). The copies alternate between plain and non-temporal stores: two
// write streams of one kind share one path through the memory system and reach 5.5 TB/s in a
// bare 1-read-2-writes sweep, one of each kind reaches 6.9 TB/s.
template <typename T, bool VEC, int KMAX = 8>
__global__ __launch_bounds__(256) void scatter_kernel(const T* __restrict__ src,
                                                       const int32_t* __restrict__ slot,
                                                       const float* __restrict__ w,
                                                       T* __restrict__ dst, int64_t n, int d, int k, int g) {
  constexpr int EPV = Elem<T>::kVec;
  const int rib = threadIdx.x / g, l = threadIdx.x % g;
  const int64_t t = (int64_t)blockIdx.x * (256 / g) + rib;
  if (t >= n) return;
  int64_t to[KMAX];
  float sc[KMAX];
#pragma unroll
  for (int j = 0; j < KMAX; ++j) {
    to[j] = j < k ? (int64_t)slot[t * k + j] * d : 0;
    sc[j] = j < k && w != nullptr ? w[t * k + j] : 1.f;
  }
  const T* sp = src + t * (int64_t)d;
  if constexpr (VEC) {
    const int nvec = d / EPV;
    for (int c0 = l; c0 < nvec; c0 += 4 * g) {
      u32x4 raw[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int c = c0 + u * g;
        if (c < nvec) raw[u] = load16_stream(sp + c * EPV);
      }
#pragma unroll
      for (int j = 0; j < KMAX; ++j) {
        if (j < k) {
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const int c = c0 + u * g;
            if (c < nvec) {
              u32x4 v = raw[u];
              if (w != nullptr) {
                float f[EPV];
                Elem<T>::unpack(v, f);
#pragma unroll
                for (int e = 0; e < EPV; ++e) f[e] *= sc[j];
                v = Elem<T>::pack(f);
              }
              if (j & 1) store16_stream(dst + to[j] + c * EPV, v);
              else store16(dst + to[j] + c * EPV, v);
            }
          }
        }
      }
    }
  } else {
    for (int i = l; i < d; i += g) {
      const float v = Elem<T>::load1(sp + i);
      for (int j = 0; j < k; ++j) Elem<T>::store1(dst + to[j] + i, v * sc[j]);
    }
  }
}

// out[t, :] = sum_j w[t*k+j] * ys[slot[t*k+j], :]   (w == NULL: unit weights)
template <typename T, bool VEC, int KMAX = 8>
__global__ __launch_bounds__(256) void combine_kernel(const T* __restrict__ ys,
                                                       const float* __restrict__ w,
                                                       const int32_t* __restrict__ slot,
                                                       T* __restrict__ out, int d, int k) {
  constexpr int EPV = Elem<T>::kVec;
  const int64_t t = blockIdx.x;
  int sl[KMAX];
  float wt[KMAX];
#pragma unroll
  for (int j = 0; j < KMAX; ++j) {
    sl[j] = j < k ? slot[t * k + j] : 0;
    wt[j] = j < k ? (w != nullptr ? w[t * k + j] : 1.f) : 0.f;
  }
  T* op = out + t * (int64_t)d;
  if constexpr (VEC) {
    const int nvec = d / EPV;
    for (int c = threadIdx.x; c < nvec; c += 256) {
      float acc[EPV];
#pragma unroll
      for (int e = 0; e < EPV; ++e) acc[e] = 0.f;
#pragma unroll
      for (int j = 0; j < KMAX; ++j) {
        if (j < k) {
          float f[EPV];
          Elem<T>::unpack(load16_stream(ys + sl[j] * (int64_t)d + c * EPV), f);
#pragma unroll
          for (int e = 0; e < EPV; ++e) acc[e] += wt[j] * f[e];
        }
      }
      store16(op + c * EPV, Elem<T>::pack(acc));
    }
  } else {
    for (int i = threadIdx.x; i < d; i += 256) {
      float acc = 0.f;
      for (int j = 0; j < k; ++j) acc += wt[j] * Elem<T>::load1(ys + sl[j] * (int64_t)d + i);
      Elem<T>::store1(op + i, acc);
    }
  }
}

// Backward of the combine wrt the weights: dw[t*k+j] = <ys[slot[t*k+j], :], dout[t, :]>
template <typename T, bool VEC, int KMAX = 8>
__global__ __launch_bounds__(256) void combine_dw_kernel(const T* __restrict__ ys,
                                                          const T* __restrict__ dout,
                                                          const int32_t* __restrict__ slot,
                                                          float* __restrict__ dw, int d, int k) {
  constexpr int EPV = Elem<T>::kVec;
  __shared__ float smem[4];
  const int64_t t = blockIdx.x;
  float dot[KMAX];
  int sl[KMAX];
#pragma unroll
  for (int j = 0; j < KMAX; ++j) { dot[j] = 0.f; sl[j] = j < k ? slot[t * k + j] : 0; }
  const T* gp = dout + t * (int64_t)d;
  if constexpr (VEC) {
    const int nvec = d / EPV;
    for (int c = threadIdx.x; c < nvec; c += 256) {
      float g[EPV];
      Elem<T>::unpack(load16(gp + c * EPV), g);
#pragma unroll
      for (int j = 0; j < KMAX; ++j) {
        if (j < k) {
          float f[EPV];
          Elem<T>::unpack(load16_stream(ys + sl[j] * (int64_t)d + c * EPV), f);
#pragma unroll
          for (int e = 0; e < EPV; ++e) dot[j] += f[e] * g[e];
        }
      }
    }
  } else {
    for (int i = threadIdx.x; i < d; i += 256) {
      const float g = Elem<T>::load1(gp + i);
      for (int j = 0; j < k; ++j) dot[j] += Elem<T>::load1(ys + sl[j] * (int64_t)d + i) * g;
    }
  }
#pragma unroll
  for (int j = 0; j < KMAX; ++j) {
    if (j < k) {   // k is uniform, so every thread reaches the barriers inside row_reduce
      const float tot = row_reduce<256, OpSum>(dot[j], smem, 0, threadIdx.x);
      if (threadIdx.x == 0) dw[t * k + j] = tot;
    }
  }
}

int check(const char* what, int64_t n, int64_t d, int k, int dtype) {
  FM_CHECK_ARG(n >= 0 && d > 0, "%s: bad shape n=%lld d=%lld", what, (long long)n, (long long)d);
  FM_CHECK_ARG(k >= 1 && k <= kMaxK, "%s: k must be in [1, %d] (got %d)", what, kMaxK, k);
  FM_CHECK_ARG(dtype == FM_F32 || dtype == FM_F16 || dtype == FM_BF16, "%s: bad dtype %d", what, dtype);
  if (n * (int64_t)k >= 0x7fffffffLL || d > 0x7fffffffLL) {
    fm_host::set_error("%s: n*k and d must be below 2^31", what);
    return FM_ERR_UNSUPPORTED;
  }
  return FM_OK;
}

template <typename T>
bool vec_ok(int64_t d, const void* a, const void* b, const void* c = nullptr) {
  return d % Elem<T>::kVec == 0 && fm_host::aligned16(a) && fm_host::aligned16(b) && fm_host::aligned16(c);
}

#define FM_BY_DTYPE(dtype, CALL)                 \
  do {                                           \
    if ((dtype) == FM_F32) { CALL(float); }      \
    else if ((dtype) == FM_BF16) { CALL(bf16_t); } \
    else { CALL(f16_t); }                        \
  } while (0)

}  // namespace

extern "C" {

int fm_moe_gather(const void* x, const int32_t* order, const float* scale, void* xs, int64_t n,
                  int64_t d, int k, int dtype, fm_stream_t stream) {
  int rc = check("fm_moe_gather", n, d, k, dtype);
  if (rc != FM_OK) return rc;
  if (n == 0) return FM_OK;
  FM_CHECK_ARG(x && order && xs, "fm_moe_gather: NULL pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int64_t total = n * k;
#define CALL(T)                                                                                  \
  {                                                                                              \
    const bool vec = vec_ok<T>(d, x, xs);                                                        \
    const int64_t units = vec ? d / Elem<T>::kVec : d;   /* loads a row takes */                  \
    int g = 8;                                                                                   \
    while (g < 256 && g < units) g *= 2;                                                         \
    const dim3 grid((unsigned)((total + 256 / g - 1) / (256 / g)));                              \
    if (vec)                                                                                     \
      FM_LAUNCH((gather_kernel<T, true>), grid, dim3(256), 0, st, static_cast<const T*>(x), \
                         order, scale, static_cast<T*>(xs), total, (int)d, k, g);                \
    else                                                                                         \
      FM_LAUNCH((gather_kernel<T, false>), grid, dim3(256), 0, st, static_cast<const T*>(x), \
                         order, scale, static_cast<T*>(xs), total, (int)d, k, g);                \
  }
  FM_BY_DTYPE(dtype, CALL);
#undef CALL
  FM_CHECK_LAUNCH("fm_moe_gather");
  return FM_OK;
}

int fm_moe_scatter(const void* x, const int32_t* slot, const float* scale, void* xs, int64_t n,
                   int64_t d, int k, int dtype, fm_stream_t stream) {
  int rc = check("fm_moe_scatter", n, d, k, dtype);
  if (rc != FM_OK) return rc;
  if (n == 0) return FM_OK;
  FM_CHECK_ARG(x && slot && xs, "fm_moe_scatter: NULL pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
#define CALL(T)                                                                                  \
  {                                                                                              \
    const bool vec = vec_ok<T>(d, x, xs);                                                        \
    const int64_t units = vec ? d / Elem<T>::kVec : d;                                           \
    int g = 8;                                                                                   \
    while (g < 256 && g < units) g *= 2;                                                         \
    const dim3 grid((unsigned)((n + 256 / g - 1) / (256 / g)));                                  \
    if (vec && k <= 8)                                                                           \
      FM_LAUNCH((scatter_kernel<T, true>), grid, dim3(256), 0, st, static_cast<const T*>(x),     \
                slot, scale, static_cast<T*>(xs), n, (int)d, k, g);                              \
    else if (vec)                                                                                \
      FM_LAUNCH((scatter_kernel<T, true, 16>), grid, dim3(256), 0, st, static_cast<const T*>(x), \
                slot, scale, static_cast<T*>(xs), n, (int)d, k, g);                              \
    else if (k <= 8)                                                                             \
      FM_LAUNCH((scatter_kernel<T, false>), grid, dim3(256), 0, st, static_cast<const T*>(x),    \
                slot, scale, static_cast<T*>(xs), n, (int)d, k, g);                              \
    else                                                                                         \
      FM_LAUNCH((scatter_kernel<T, false, 16>), grid, dim3(256), 0, st, static_cast<const T*>(x), \
                slot, scale, static_cast<T*>(xs), n, (int)d, k, g);                              \
  }
  FM_BY_DTYPE(dtype, CALL);
#undef CALL
  FM_CHECK_LAUNCH("fm_moe_scatter");
  return FM_OK;
}

int fm_moe_combine(const void* ys, const float* weights, const int32_t* slot, void* out, int64_t n,
                   int64_t d, int k, int dtype, fm_stream_t stream) {
  int rc = check("fm_moe_combine", n, d, k, dtype);
  if (rc != FM_OK) return rc;
  if (n == 0) return FM_OK;
  FM_CHECK_ARG(ys && slot && out, "fm_moe_combine: NULL pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)n);
#define GO(T, VEC_, KMAX_)                                                                         \
  FM_LAUNCH((combine_kernel<T, VEC_, KMAX_>), grid, dim3(256), 0, st, static_cast<const T*>(ys),   \
            weights, slot, static_cast<T*>(out), (int)d, k)
#define CALL(T)                                                                                    \
  if (vec_ok<T>(d, ys, out)) {                                                                     \
    if (k <= 8) GO(T, true, 8);                                                                       \
    else GO(T, true, 16);                                                                             \
  } else {                                                                                         \
    if (k <= 8) GO(T, false, 8);                                                                      \
    else GO(T, false, 16);                                                                            \
  }
  FM_BY_DTYPE(dtype, CALL);
#undef CALL
#undef GO
  FM_CHECK_LAUNCH("fm_moe_combine");
  return FM_OK;
}

int fm_moe_combine_dw(const void* ys, const void* dout, const int32_t* slot, float* dweights,
                      int64_t n, int64_t d, int k, int dtype, fm_stream_t stream) {
  int rc = check("fm_moe_combine_dw", n, d, k, dtype);
  if (rc != FM_OK) return rc;
  if (n == 0) return FM_OK;
  FM_CHECK_ARG(ys && dout && slot && dweights, "fm_moe_combine_dw: NULL pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)n);
#define GO(T, VEC_, KMAX_)                                                                       \
  FM_LAUNCH((combine_dw_kernel<T, VEC_, KMAX_>), grid, dim3(256), 0, st, static_cast<const T*>(ys), \
            static_cast<const T*>(dout), slot, dweights, (int)d, k)
#define CALL(T)                                                                                  \
  if (vec_ok<T>(d, ys, dout)) {                                                                  \
    if (k <= 8) GO(T, true, 8);                                                                     \
    else GO(T, true, 16);                                                                           \
  } else {                                                                                       \
    if (k <= 8) GO(T, false, 8);                                                                    \
    else GO(T, false, 16);                                                                          \
  }
  FM_BY_DTYPE(dtype, CALL);
#undef CALL
#undef GO
  FM_CHECK_LAUNCH("fm_moe_combine_dw");
  return FM_OK;
}

}  // extern "C"
