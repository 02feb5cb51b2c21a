// SwiGLU epilogues for gfx950: silu(gate) * up on two tensors, and on the two halves of a
// fused gate|up projection, forward and backward.
//
// Reference semantics: forgemind/kernels/_fallback.py:48-49 (fp32 math, one rounding) and
// forgemind/kernels/swiglu.py:48-120 (the derivative: with s = sigmoid(g),
// d/dg [g*s*u] = u * s * (1 + g*(1 - s)), d/du = g*s).
// Flat element-wise streams: 16-byte vectors, one-shot grid, scalar tail / unaligned path.
#include "fm_common.hip.h"

using namespace fm;

namespace {

__device__ __forceinline__ float sigmoidf_fast(float x) {
  return 1.f / (1.f + fast_exp2(-x * kLog2e));
}

template <typename T, bool VEC>
__global__ __launch_bounds__(256) void swiglu_fwd_kernel(const T* __restrict__ g, const T* __restrict__ u,
                                                          T* __restrict__ y, int64_t n) {
  constexpr int EPV = Elem<T>::kVec;
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if constexpr (VEC) {
    if (i * EPV + EPV <= n) {
      float a[EPV], b[EPV], o[EPV];
      Elem<T>::unpack(load16_stream(g + i * EPV), a);
      Elem<T>::unpack(load16_stream(u + i * EPV), b);
#pragma unroll
      for (int e = 0; e < EPV; ++e) o[e] = a[e] * sigmoidf_fast(a[e]) * b[e];
      store16_stream(y + i * EPV, Elem<T>::pack(o));
    } else {
      for (int64_t j = i * EPV; j < n; ++j) {
        const float a = Elem<T>::load1(g + j);
        Elem<T>::store1(y + j, a * sigmoidf_fast(a) * Elem<T>::load1(u + j));
      }
    }
  } else {
    if (i < n) {
      const float a = Elem<T>::load1(g + i);
      Elem<T>::store1(y + i, a * sigmoidf_fast(a) * Elem<T>::load1(u + i));
    }
  }
}

template <typename T, bool VEC>
__global__ __launch_bounds__(256) void swiglu_bwd_kernel(const T* __restrict__ g, const T* __restrict__ u,
                                                          const T* __restrict__ dy, T* __restrict__ dg,
                                                          T* __restrict__ du, int64_t n) {
  constexpr int EPV = Elem<T>::kVec;
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  auto one = [](float a, float b, float d, float& oa, float& ob) {
    const float s = sigmoidf_fast(a);
    oa = d * b * s * (1.f + a * (1.f - s));
    ob = d * a * s;
  };
  if constexpr (VEC) {
    if (i * EPV + EPV <= n) {
      float a[EPV], b[EPV], d[EPV], oa[EPV], ob[EPV];
      Elem<T>::unpack(load16_stream(g + i * EPV), a);
      Elem<T>::unpack(load16_stream(u + i * EPV), b);
      Elem<T>::unpack(load16_stream(dy + i * EPV), d);
#pragma unroll
      for (int e = 0; e < EPV; ++e) one(a[e], b[e], d[e], oa[e], ob[e]);
      store16_stream(dg + i * EPV, Elem<T>::pack(oa));
      store16_stream(du + i * EPV, Elem<T>::pack(ob));
    } else {
      for (int64_t j = i * EPV; j < n; ++j) {
        float oa, ob;
        one(Elem<T>::load1(g + j), Elem<T>::load1(u + j), Elem<T>::load1(dy + j), oa, ob);
        Elem<T>::store1(dg + j, oa);
        Elem<T>::store1(du + j, ob);
      }
    }
  } else {
    if (i < n) {
      float oa, ob;
      one(Elem<T>::load1(g + i), Elem<T>::load1(u + i), Elem<T>::load1(dy + i), oa, ob);
      Elem<T>::store1(dg + i, oa);
      Elem<T>::store1(du + i, ob);
    }
  }
}

// x: [rows, 2h]; y: [rows, h]. grid.y = row, grid.x covers the h outputs of the row.
template <typename T, bool VEC, bool BWD>
__global__ __launch_bounds__(256) void swiglu_split_kernel(const T* __restrict__ x, const T* __restrict__ dy,
                                                            T* __restrict__ out, int h) {
  constexpr int EPV = Elem<T>::kVec;
  const int64_t row = blockIdx.y;
  const T* gp = x + row * 2 * (int64_t)h;
  const T* up = gp + h;
  const int i = blockIdx.x * 256 + threadIdx.x;
  if constexpr (VEC) {
    if (i * EPV < h) {
      float a[EPV], b[EPV];
      Elem<T>::unpack(load16_stream(gp + i * EPV), a);
      Elem<T>::unpack(load16_stream(up + i * EPV), b);
      if constexpr (!BWD) {
        float o[EPV];
#pragma unroll
        for (int e = 0; e < EPV; ++e) o[e] = a[e] * sigmoidf_fast(a[e]) * b[e];
        store16_stream(out + row * (int64_t)h + i * EPV, Elem<T>::pack(o));
      } else {
        float d[EPV], oa[EPV], ob[EPV];
        Elem<T>::unpack(load16_stream(dy + row * (int64_t)h + i * EPV), d);
#pragma unroll
        for (int e = 0; e < EPV; ++e) {
          const float s = sigmoidf_fast(a[e]);
          oa[e] = d[e] * b[e] * s * (1.f + a[e] * (1.f - s));
          ob[e] = d[e] * a[e] * s;
        }
        T* dx = out + row * 2 * (int64_t)h;
        store16_stream(dx + i * EPV, Elem<T>::pack(oa));
        store16_stream(dx + h + i * EPV, Elem<T>::pack(ob));
      }
    }
  } else {
    if (i < h) {
      const float a = Elem<T>::load1(gp + i), b = Elem<T>::load1(up + i);
      const float s = sigmoidf_fast(a);
      if constexpr (!BWD) {
        Elem<T>::store1(out + row * (int64_t)h + i, a * s * b);
      } else {
        const float d = Elem<T>::load1(dy + row * (int64_t)h + i);
        T* dx = out + row * 2 * (int64_t)h;
        Elem<T>::store1(dx + i, d * b * s * (1.f + a * (1.f - s)));
        Elem<T>::store1(dx + h + i, d * a * s);
      }
    }
  }
}

int check_dtype(const char* what, int dtype) {
  FM_CHECK_ARG(dtype == FM_F32 || dtype == FM_F16 || dtype == FM_BF16, "%s: bad dtype %d", what, dtype);
  return FM_OK;
}

#define FM_BY_DTYPE(dtype, CALL)                   \
  do {                                             \
    if ((dtype) == FM_F32) { CALL(float); }        \
    else if ((dtype) == FM_BF16) { CALL(bf16_t); } \
    else { CALL(f16_t); }                          \
  } while (0)

}  // namespace

extern "C" {

int fm_swiglu_fwd(const void* gate, const void* up, void* y, int64_t n, int dtype, fm_stream_t stream) {
  int rc = check_dtype("fm_swiglu_fwd", dtype);
  if (rc != FM_OK) return rc;
  FM_CHECK_ARG(n >= 0, "fm_swiglu_fwd: negative size");
  if (n == 0) return FM_OK;
  FM_CHECK_ARG(gate && up && y, "fm_swiglu_fwd: NULL pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool vec = fm_host::aligned16(gate) && fm_host::aligned16(up) && fm_host::aligned16(y);
#define CALL(T)                                                                                     \
  if (vec) {                                                                                        \
    const int64_t nv = (n + Elem<T>::kVec - 1) / Elem<T>::kVec;                                     \
    FM_LAUNCH((swiglu_fwd_kernel<T, true>), dim3((unsigned)((nv + 255) / 256)), dim3(256), 0, st, \
                       static_cast<const T*>(gate), static_cast<const T*>(up), static_cast<T*>(y), n); \
  } else {                                                                                          \
    FM_LAUNCH((swiglu_fwd_kernel<T, false>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, \
                       static_cast<const T*>(gate), static_cast<const T*>(up), static_cast<T*>(y), n); \
  }
  FM_BY_DTYPE(dtype, CALL);
#undef CALL
  FM_CHECK_LAUNCH("fm_swiglu_fwd");
  return FM_OK;
}

int fm_swiglu_bwd(const void* gate, const void* up, const void* dy, void* dgate, void* dup, int64_t n,
                  int dtype, fm_stream_t stream) {
  int rc = check_dtype("fm_swiglu_bwd", dtype);
  if (rc != FM_OK) return rc;
  FM_CHECK_ARG(n >= 0, "fm_swiglu_bwd: negative size");
  if (n == 0) return FM_OK;
  FM_CHECK_ARG(gate && up && dy && dgate && dup, "fm_swiglu_bwd: NULL pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool vec = fm_host::aligned16(gate) && fm_host::aligned16(up) && fm_host::aligned16(dy) &&
                   fm_host::aligned16(dgate) && fm_host::aligned16(dup);
#define CALL(T)                                                                                     \
  if (vec) {                                                                                        \
    const int64_t nv = (n + Elem<T>::kVec - 1) / Elem<T>::kVec;                                     \
    FM_LAUNCH((swiglu_bwd_kernel<T, true>), dim3((unsigned)((nv + 255) / 256)), dim3(256), 0, st, \
                       static_cast<const T*>(gate), static_cast<const T*>(up), static_cast<const T*>(dy), \
                       static_cast<T*>(dgate), static_cast<T*>(dup), n);                            \
  } else {                                                                                          \
    FM_LAUNCH((swiglu_bwd_kernel<T, false>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, \
                       static_cast<const T*>(gate), static_cast<const T*>(up), static_cast<const T*>(dy), \
                       static_cast<T*>(dgate), static_cast<T*>(dup), n);                            \
  }
  FM_BY_DTYPE(dtype, CALL);
#undef CALL
  FM_CHECK_LAUNCH("fm_swiglu_bwd");
  return FM_OK;
}

static int split_entry(const char* what, const void* x, const void* dy, void* out, int64_t rows, int64_t h,
                       int dtype, bool bwd, fm_stream_t stream) {
  int rc = check_dtype(what, dtype);
  if (rc != FM_OK) return rc;
  FM_CHECK_ARG(rows >= 0 && h > 0, "%s: bad shape rows=%lld h=%lld", what, (long long)rows, (long long)h);
  if (rows > 0x7fffffffLL / 2 || h > 0x3fffffffLL || rows > 65535LL * 65535LL) {
    fm_host::set_error("%s: shape too large", what);
    return FM_ERR_UNSUPPORTED;
  }
  if (rows == 0) return FM_OK;
  FM_CHECK_ARG(x && out && (!bwd || dy), "%s: NULL pointer", what);
  hipStream_t st = static_cast<hipStream_t>(stream);
  // blockIdx.y carries the row; very tall inputs are launched in slabs of 65535 rows
  for (int64_t r0 = 0; r0 < rows; r0 += 65535) {
    const int64_t nr = rows - r0 < 65535 ? rows - r0 : 65535;
#define CALL(T)                                                                                    \
  {                                                                                                \
    const T* xp = static_cast<const T*>(x) + r0 * 2 * h;                                           \
    const T* dp = bwd ? static_cast<const T*>(dy) + r0 * h : nullptr;                              \
    T* op = static_cast<T*>(out) + r0 * (bwd ? 2 * h : h);                                         \
    const bool vec = h % Elem<T>::kVec == 0 && fm_host::aligned16(x) && fm_host::aligned16(out) && \
                     fm_host::aligned16(dy);                                                       \
    const int64_t per = vec ? h / Elem<T>::kVec : h;                                               \
    const dim3 grid((unsigned)((per + 255) / 256), (unsigned)nr);                                  \
    if (vec && !bwd) FM_LAUNCH((swiglu_split_kernel<T, true, false>), grid, dim3(256), 0, st, xp, dp, op, (int)h); \
    else if (vec) FM_LAUNCH((swiglu_split_kernel<T, true, true>), grid, dim3(256), 0, st, xp, dp, op, (int)h);     \
    else if (!bwd) FM_LAUNCH((swiglu_split_kernel<T, false, false>), grid, dim3(256), 0, st, xp, dp, op, (int)h);  \
    else FM_LAUNCH((swiglu_split_kernel<T, false, true>), grid, dim3(256), 0, st, xp, dp, op, (int)h);             \
  }
    FM_BY_DTYPE(dtype, CALL);
#undef CALL
  }
  FM_CHECK_LAUNCH(what);
  return FM_OK;
}

int fm_swiglu_split_fwd(const void* x, void* y, int64_t rows, int64_t h, int dtype, fm_stream_t stream) {
  return split_entry("fm_swiglu_split_fwd", x, nullptr, y, rows, h, dtype, false, stream);
}

int fm_swiglu_split_bwd(const void* x, const void* dy, void* dx, int64_t rows, int64_t h, int dtype,
                        fm_stream_t stream) {
  return split_entry("fm_swiglu_split_bwd", x, dy, dx, rows, h, dtype, true, stream);
}

}  // extern "C"
