// Row normalisation kernels shared by RMSNorm (norm.hip) and LayerNorm (layernorm.hip), gfx950.
// The flag LN selects mean subtraction, the bias, and the second set of parameter-gradient
// columns; everything else (row ownership, register residency, persistent backward, fixed-order
// column sums) is common.
//
// Layout: rows are dense, row-major. A row is owned by TPR threads (a lane group, a wave or
// several waves of one workgroup); each thread keeps ITERS 16-byte vectors of the row in
// registers between the reduction and the store, so every tensor is read exactly once.
// The backward is persistent: a fixed grid walks the row tiles, each thread accumulates its
// columns of dW (and db) in fp32 registers, the workgroup folds its rows through LDS and writes
// one partial row; a second kernel sums the partial rows in a fixed order.
#pragma once

#include "fm_common.hip.h"

using namespace fm;

namespace {

constexpr int kMinBlock = 256;
// The backward always runs 16-wave workgroups: many rows per workgroup are folded through
// LDS, so the number of fp32 partial rows (one per workgroup) stays at the CU count while
// each SIMD still has four waves to hide load latency.
constexpr int kBwdBlock = 1024;

template <int TPR> struct BlockOf { static constexpr int value = TPR > kMinBlock ? TPR : kMinBlock; };

// Load the EPV weights that line up with one 16-byte vector of the activations.
template <typename T, typename WT>
__device__ __forceinline__ void load_w(const WT* w, int col, float (&o)[Elem<T>::kVec]) {
  constexpr int EPV = Elem<T>::kVec;
  if constexpr (sizeof(WT) == sizeof(T)) {
    Elem<WT>::unpack(load16(w + col), o);
  } else {  // fp32 weights next to 16-bit activations: two 16-byte loads
    static_assert(sizeof(WT) == 4 && EPV == 8, "weights are either x's dtype or fp32");
    float a[4], b[4];
    Elem<float>::unpack(load16(w + col), a);
    Elem<float>::unpack(load16(w + col + 4), b);
#pragma unroll
    for (int i = 0; i < 4; ++i) { o[i] = a[i]; o[4 + i] = b[i]; }
  }
}

// ---------------------------------------------------------------- forward (vector path)
// Persistent over row tiles: the grid holds a few workgroups per compute unit, each keeps its
// columns of w (and the bias) in registers and walks tiles blockIdx.x, blockIdx.x + gridDim.x, ...
// so the parameters are fetched once per workgroup instead of once per row.
// XKEEP: x is read with cached loads so that it stays in the memory-side cache for the backward
// (or a recompute's backward) that reads it again; the launcher sets it for a plain norm whose x
// fits that cache. Not for the fused add: its backward reads xn, and x kept there only evicts it.
template <typename T, typename WT, int TPR, int ITERS, bool ADD, bool LN, bool XKEEP = false>
__global__ __launch_bounds__(BlockOf<TPR>::value) void norm_fwd_kernel(
    const T* __restrict__ x, const T* __restrict__ delta, const WT* __restrict__ w,
    const WT* __restrict__ bias, T* __restrict__ xn, T* __restrict__ y, float* __restrict__ mean,
    float* __restrict__ rstd, int64_t n, int d, float eps, int64_t tiles) {
  constexpr int EPV = Elem<T>::kVec;
  constexpr int BLOCK = BlockOf<TPR>::value;
  constexpr int RPB = BLOCK / TPR;
  constexpr int NB = LN ? ITERS : 1;
  __shared__ float smem[RPB * (TPR > 64 ? TPR / 64 : 1)];

  const int tid = threadIdx.x;
  const int rib = tid / TPR;
  const int t = tid % TPR;
  const int nvec = d / EPV;

  float wv[ITERS][EPV];
  float bv[NB][EPV];
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
    const int c = i * TPR + t;
    if (c < nvec) {
      load_w<T, WT>(w, c * EPV, wv[i]);
    } else {
#pragma unroll
      for (int e = 0; e < EPV; ++e) wv[i][e] = 0.f;
    }
  }
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    const int c = i * TPR + t;
    if (LN && bias != nullptr && c < nvec) {
      load_w<T, WT>(bias, c * EPV, bv[i]);
    } else {
#pragma unroll
      for (int e = 0; e < EPV; ++e) bv[i][e] = 0.f;
    }
  }

  int64_t first = blockIdx.x;
  {
    // One tile per workgroup (small inputs): the tiles are dealt so that a row is handled here by
    // the same eighth of the device (workgroup index mod 8, one L2 each) that reads it in the
    // backward, whose tiles are G of these and go round the same way. What this launch leaves in
    // that L2 -- x read with cached loads, or the xn it wrote -- is what the backward reads first.
    constexpr int G = kBwdBlock / BLOCK;
    if (G >= 1 && gridDim.x == tiles && tiles % (8 * G) == 0) {
      const int64_t j = blockIdx.x >> 3;
      first = ((j / G) * 8 + (blockIdx.x & 7)) * G + (j % G);
    }
  }
  for (int64_t tile = first; tile < tiles; tile += gridDim.x) {
    const int64_t row = tile * RPB + rib;
    const bool valid = row < n;
    const int64_t base = row * (int64_t)d;

    float v[ITERS][EPV];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      const int c = i * TPR + t;
      if (valid && c < nvec) {
        u32x4 rx;
        if constexpr (XKEEP) rx = load16(x + base + (int64_t)c * EPV);
        else rx = load16_stream(x + base + (int64_t)c * EPV);
        Elem<T>::unpack(rx, v[i]);
        if constexpr (ADD) {
          float dv[EPV];
          Elem<T>::unpack(load16_stream(delta + base + (int64_t)c * EPV), dv);
#pragma unroll
          for (int e = 0; e < EPV; ++e) v[i][e] += dv[e];
          // statistics come from the value a tensor add would have stored
          u32x4 packed = Elem<T>::pack(v[i]);
          store16(xn + base + (int64_t)c * EPV, packed);
          Elem<T>::unpack(packed, v[i]);
        }
#pragma unroll
        for (int e = 0; e < EPV; ++e) ss += LN ? v[i][e] : v[i][e] * v[i][e];
      } else {
#pragma unroll
        for (int e = 0; e < EPV; ++e) v[i][e] = 0.f;
      }
    }
    ss = row_reduce<TPR, OpSum>(ss, smem, rib, t);
    float mu = 0.f;
    if constexpr (LN) {
      // mean first, then the centred second moment: the row is in registers, so the second
      // sweep is free and there is no E[x^2] - mean^2 cancellation
      mu = ss / (float)d;
      ss = 0.f;
#pragma unroll
      for (int i = 0; i < ITERS; ++i) {
        const int c = i * TPR + t;
        if (valid && c < nvec) {
#pragma unroll
          for (int e = 0; e < EPV; ++e) ss += (v[i][e] - mu) * (v[i][e] - mu);
        }
      }
      ss = row_reduce<TPR, OpSum>(ss, smem, rib, t);
    }
    const float r = rsqrtf(ss / (float)d + eps);
    if (valid && t == 0) {
      rstd[row] = r;
      if constexpr (LN) mean[row] = mu;
    }
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      const int c = i * TPR + t;
      if (valid && c < nvec) {
        float o[EPV];
#pragma unroll
        for (int e = 0; e < EPV; ++e) o[e] = ((v[i][e] - mu) * r) * wv[i][e];
        if constexpr (LN) {
#pragma unroll
          for (int e = 0; e < EPV; ++e) o[e] += bv[i][e];
        }
        store16_stream(y + base + (int64_t)c * EPV, Elem<T>::pack(o));
      }
    }
  }
}

// ---------------------------------------------------------------- backward (vector path)
// grid-persistent; `partial` is [gridDim.x, d] fp32 (LN: [gridDim.x, 2 d], weight then bias
// columns), or NULL when the parameter gradients are not wanted.
// XCACHED: x is read with cached loads instead of streaming ones. x is the one operand a forward
// (or a recompute of it) may have written just before, with cached stores, and a cached load finds
// it in the L2 / the memory-side cache where a streaming load does not: add-RMSNorm pair at
// [16384,8192] bf16 334 -> 325 us, [8192,1024] 21.1 -> 20.0; on an x that is NOT there it costs 1 %
// (183 -> 185 us). Only for an x that fits that cache: on a larger one the loads of its first
// rows push out the last rows before they are read ([32768,8192]: pair 696 -> 768 us).
template <typename T, typename WT, int TPR, int ITERS, bool LN, bool XCACHED = false>
__global__ __launch_bounds__(kBwdBlock) void norm_bwd_kernel(
    const T* __restrict__ x, const WT* __restrict__ w, const float* __restrict__ mean,
    const float* __restrict__ rstd, const T* __restrict__ dy, const T* __restrict__ gxn,
    T* __restrict__ dx, T* __restrict__ dd, float* __restrict__ partial, int64_t n, int d,
    int64_t tiles) {
  constexpr int EPV = Elem<T>::kVec;
  constexpr int BLOCK = kBwdBlock;
  constexpr int RPB = BLOCK / TPR;
  constexpr int COVER = TPR * ITERS * EPV;   // columns covered by one row's threads
  constexpr int NB = LN ? ITERS : 1;         // bias-gradient accumulators exist only for LN
  // Rows of 512 threads: the 8 * ITERS weight registers do not fit next to the packed rows and
  // the fp32 column sums (the compiler spilled 12-20 bytes per lane to scratch), so the weight
  // columns live in LDS as fp32 instead, one 16-byte quad per lane and read, laid out so that
  // neighbouring lanes read neighbouring quads (no bank conflicts).
  constexpr bool WLDS = TPR >= 512;
  constexpr int QPV = EPV / 4;
  __shared__ float red[RPB * (TPR > 64 ? TPR / 64 : 1)];
  __shared__ float fold[RPB > 1 ? RPB * COVER : 1];
  __shared__ f32x4 wsm[WLDS ? ITERS * QPV * TPR : 1];

  const int tid = threadIdx.x;
  const int rib = tid / TPR;
  const int t = tid % TPR;
  const int nvec = d / EPV;
  const float inv_d = 1.f / (float)d;
  const int pcols = LN ? 2 * d : d;

  float wv[WLDS ? 1 : ITERS][EPV];
  float acc[ITERS][EPV];
  float accb[NB][EPV];
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
    const int c = i * TPR + t;
    float wl[EPV];
    if (c < nvec) {
      load_w<T, WT>(w, c * EPV, wl);
    } else {
#pragma unroll
      for (int e = 0; e < EPV; ++e) wl[e] = 0.f;
    }
    if constexpr (WLDS) {
      if (rib == 0) {
#pragma unroll
        for (int q = 0; q < QPV; ++q) {
          const f32x4 v4 = {wl[4 * q], wl[4 * q + 1], wl[4 * q + 2], wl[4 * q + 3]};
          wsm[(i * QPV + q) * TPR + t] = v4;
        }
      }
    } else {
#pragma unroll
      for (int e = 0; e < EPV; ++e) wv[i][e] = wl[e];
    }
#pragma unroll
    for (int e = 0; e < EPV; ++e) acc[i][e] = 0.f;
  }
  if constexpr (WLDS) __syncthreads();
  auto weights = [&](int i, float (&o)[EPV]) {
    if constexpr (WLDS) {
#pragma unroll
      for (int q = 0; q < QPV; ++q) {
        const f32x4 v4 = wsm[(i * QPV + q) * TPR + t];
        o[4 * q] = v4.x; o[4 * q + 1] = v4.y; o[4 * q + 2] = v4.z; o[4 * q + 3] = v4.w;
      }
    } else {
#pragma unroll
      for (int e = 0; e < EPV; ++e) o[e] = wv[i][e];
    }
  };
#pragma unroll
  for (int i = 0; i < NB; ++i) {
#pragma unroll
    for (int e = 0; e < EPV; ++e) accb[i][e] = 0.f;
  }

  for (int64_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
    const int64_t row = tile * RPB + rib;
    const bool valid = row < n;
    const int64_t base = row * (int64_t)d;
    // x and dy stay packed in registers between the two sweeps (half the footprint of fp32)
    // rr: the residual-stream gradient, fetched with the rest where the register budget allows
    // (the LayerNorm form carries a second set of accumulators and fetches it late instead)
    constexpr bool EARLY_RES = !LN;
    u32x4 rx[ITERS], rg[ITERS], rr[EARLY_RES ? ITERS : 1];
    const float r = valid ? rstd[row] : 0.f;
    float mu = 0.f;
    if constexpr (LN) mu = valid ? mean[row] : 0.f;
    float dot = 0.f, gsum = 0.f;
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      const int c = i * TPR + t;
      if (valid && c < nvec) {
        if constexpr (XCACHED) rx[i] = load16(x + base + (int64_t)c * EPV);
        else rx[i] = load16_stream(x + base + (int64_t)c * EPV);
        rg[i] = load16_stream(dy + base + (int64_t)c * EPV);
        if constexpr (EARLY_RES) {
          if (gxn != nullptr) rr[i] = load16_stream(gxn + base + (int64_t)c * EPV);
        }
      }
    }
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      const int c = i * TPR + t;
      if (valid && c < nvec) {
        float xv[EPV], gv[EPV], wc[EPV];
        Elem<T>::unpack(rx[i], xv);
        Elem<T>::unpack(rg[i], gv);
        weights(i, wc);
#pragma unroll
        for (int e = 0; e < EPV; ++e) {
          const float xh = (xv[e] - mu) * r;
          acc[i][e] += gv[e] * xh;
          dot += (gv[e] * wc[e]) * xh;
          if constexpr (LN) {
            accb[i][e] += gv[e];
            gsum += gv[e] * wc[e];
          }
        }
      }
    }
    dot = row_reduce<TPR, OpSum>(dot, red, rib, t);
    const float cmean = dot * inv_d;
    float gmean = 0.f;
    if constexpr (LN) gmean = row_reduce<TPR, OpSum>(gsum, red, rib, t) * inv_d;
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      const int c = i * TPR + t;
      if (valid && c < nvec) {
        float xv[EPV], gv[EPV], o[EPV], wc[EPV];
        Elem<T>::unpack(rx[i], xv);
        Elem<T>::unpack(rg[i], gv);
        weights(i, wc);
#pragma unroll
        for (int e = 0; e < EPV; ++e)
          o[e] = ((gv[e] * wc[e] - gmean) - ((xv[e] - mu) * r) * cmean) * r;
        if (gxn != nullptr) {
          float rv[EPV];
          if constexpr (EARLY_RES) Elem<T>::unpack(rr[i], rv);
          else Elem<T>::unpack(load16_stream(gxn + base + (int64_t)c * EPV), rv);
#pragma unroll
          for (int e = 0; e < EPV; ++e) o[e] += rv[e];
        }
        const u32x4 packed = Elem<T>::pack(o);
        store16_stream(dx + base + (int64_t)c * EPV, packed);
        if (dd != nullptr) store16_stream(dd + base + (int64_t)c * EPV, packed);
      }
    }
  }

  if (partial == nullptr) return;
  float* prow = partial + (int64_t)blockIdx.x * pcols;
  // weight-gradient columns first, then (LN) the bias-gradient columns through the same LDS
#pragma unroll
  for (int which = 0; which < (LN ? 2 : 1); ++which) {
    float* out = prow + which * d;
    if constexpr (RPB == 1) {
#pragma unroll
      for (int i = 0; i < ITERS; ++i) {
        const int c = i * TPR + t;
        if (c < nvec) {
#pragma unroll
          for (int q = 0; q < EPV / 4; ++q) {
            float o4[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) o4[j] = which == 0 ? acc[i][4 * q + j] : accb[LN ? i : 0][4 * q + j];
            store16(out + c * EPV + 4 * q, Elem<float>::pack(o4));
          }
        }
      }
    } else {
      // fold the RPB rows of this workgroup in row order, then write one partial row
      if (which == 1) __syncthreads();
#pragma unroll
      for (int i = 0; i < ITERS; ++i) {
        const int c = i * TPR + t;
#pragma unroll
        for (int e = 0; e < EPV; ++e)
          fold[rib * COVER + c * EPV + e] = which == 0 ? acc[i][e] : accb[LN ? i : 0][e];
      }
      __syncthreads();
      for (int j = tid; j < d; j += BLOCK) {
        float s = fold[j];
#pragma unroll
        for (int rr = 1; rr < RPB; ++rr) s += fold[rr * COVER + j];
        out[j] = s;
      }
    }
  }
}

// Column sum of `p` partial rows, [p, d] fp32 -> dw[d] in WT. One workgroup owns 64 columns
// as 16 quads; thread (g, q) adds rows g, g+64, ... of quad q with 16-byte loads, then the 64
// row-group results are added in group order. The order depends only on (p, d), never on
// timing. Rows of `partial` are `stride` floats apart. Requires d % 4 == 0 (the register path
// guarantees it); otherwise colsum_scalar.
template <typename WT>
__global__ __launch_bounds__(1024) void colsum_kernel(const float* __restrict__ partial,
                                                       WT* __restrict__ dw, int p, int d,
                                                       int stride, WT* __restrict__ dw_second) {
  // a launch with two rows of workgroups sums two column sets at once: the second row takes the
  // columns d .. 2d - 1 of every partial row into `dw_second` (LayerNorm: weight and bias gradient)
  if (blockIdx.y == 1) { partial += d; dw = dw_second; }
  __shared__ float s[64][64 + 4];
  const int q = threadIdx.x & 15;
  const int g = threadIdx.x >> 4;
  const int col = blockIdx.x * 64 + q * 4;
  float a[4] = {0.f, 0.f, 0.f, 0.f};
  if (col < d) {
    int r = g;
    for (; r + 192 < p; r += 256) {
      float v[4][4];
#pragma unroll
      for (int u = 0; u < 4; ++u) Elem<float>::unpack(load16(partial + (int64_t)(r + 64 * u) * stride + col), v[u]);
#pragma unroll
      for (int u = 0; u < 4; ++u) {
#pragma unroll
        for (int c = 0; c < 4; ++c) a[c] += v[u][c];
      }
    }
    for (; r < p; r += 64) {
      float v[4];
      Elem<float>::unpack(load16(partial + (int64_t)r * stride + col), v);
#pragma unroll
      for (int c = 0; c < 4; ++c) a[c] += v[c];
    }
  }
#pragma unroll
  for (int c = 0; c < 4; ++c) s[g][q * 4 + c] = a[c];
  __syncthreads();
  if (threadIdx.x < 64) {
    const int cc = blockIdx.x * 64 + threadIdx.x;
    if (cc < d) {
      float tot = s[0][threadIdx.x];
#pragma unroll 8
      for (int i = 1; i < 64; ++i) tot += s[i][threadIdx.x];
      Elem<WT>::store1(dw + cc, tot);
    }
  }
}

template <typename WT>
__global__ __launch_bounds__(1024) void colsum_scalar_kernel(const float* __restrict__ partial,
                                                              WT* __restrict__ dw, int p, int d,
                                                              int stride, WT* __restrict__ dw_second) {
  if (blockIdx.y == 1) { partial += d; dw = dw_second; }
  __shared__ float s[16][64];
  const int lane = threadIdx.x & 63;
  const int g = threadIdx.x >> 6;
  const int col = blockIdx.x * 64 + lane;
  float a = 0.f;
  if (col < d) {
    for (int r = g; r < p; r += 16) a += partial[(int64_t)r * stride + col];
  }
  s[g][lane] = a;
  __syncthreads();
  if (g == 0 && col < d) {
    float tot = s[0][lane];
#pragma unroll
    for (int i = 1; i < 16; ++i) tot += s[i][lane];
    Elem<WT>::store1(dw + col, tot);
  }
}

// ---------------------------------------------------------------- any-width path
// One 256-thread workgroup per row, two passes over the row (the second one hits cache).
// Used when d is not a multiple of the 16-byte vector width, a pointer is not 16-byte
// aligned, or the row is wider than the register path covers.
template <typename T, typename WT, bool ADD, bool LN>
__global__ __launch_bounds__(256) void norm_fwd_generic(
    const T* __restrict__ x, const T* __restrict__ delta, const WT* __restrict__ w,
    const WT* __restrict__ bias, T* __restrict__ xn, T* __restrict__ y, float* __restrict__ mean,
    float* __restrict__ rstd, int64_t d, float eps) {
  __shared__ float smem[4];
  const int64_t base = (int64_t)blockIdx.x * d;
  auto value = [&](int64_t j) {
    float v = Elem<T>::load1(x + base + j);
    if constexpr (ADD) v = Elem<T>::round(v + Elem<T>::load1(delta + base + j));
    return v;
  };
  float ss = 0.f;
  for (int64_t j = threadIdx.x; j < d; j += 256) {
    const float v = value(j);
    if constexpr (ADD) Elem<T>::store1(xn + base + j, v);
    ss += LN ? v : v * v;
  }
  ss = row_reduce<256, OpSum>(ss, smem, 0, threadIdx.x);
  float mu = 0.f;
  if constexpr (LN) {
    mu = ss / (float)d;
    ss = 0.f;
    for (int64_t j = threadIdx.x; j < d; j += 256) {
      const float c = value(j) - mu;
      ss += c * c;
    }
    ss = row_reduce<256, OpSum>(ss, smem, 0, threadIdx.x);
  }
  const float r = rsqrtf(ss / (float)d + eps);
  if (threadIdx.x == 0) {
    rstd[blockIdx.x] = r;
    if constexpr (LN) mean[blockIdx.x] = mu;
  }
  for (int64_t j = threadIdx.x; j < d; j += 256) {
    float o = ((value(j) - mu) * r) * Elem<WT>::load1(w + j);
    if constexpr (LN) {
      if (bias != nullptr) o += Elem<WT>::load1(bias + j);
    }
    Elem<T>::store1(y + base + j, o);
  }
}

template <typename T, typename WT, bool LN>
__global__ __launch_bounds__(256) void norm_bwd_generic(
    const T* __restrict__ x, const WT* __restrict__ w, const float* __restrict__ mean,
    const float* __restrict__ rstd, const T* __restrict__ dy, const T* __restrict__ gxn,
    T* __restrict__ dx, T* __restrict__ dd, int64_t d) {
  __shared__ float smem[4];
  const int64_t base = (int64_t)blockIdx.x * d;
  const float r = rstd[blockIdx.x];
  float mu = 0.f;
  if constexpr (LN) mu = mean[blockIdx.x];
  float dot = 0.f, gsum = 0.f;
  for (int64_t j = threadIdx.x; j < d; j += 256) {
    const float xh = (Elem<T>::load1(x + base + j) - mu) * r;
    const float g = Elem<T>::load1(dy + base + j) * Elem<WT>::load1(w + j);
    dot += g * xh;
    gsum += g;
  }
  dot = row_reduce<256, OpSum>(dot, smem, 0, threadIdx.x);
  const float cmean = dot / (float)d;
  float gmean = 0.f;
  if constexpr (LN) gmean = row_reduce<256, OpSum>(gsum, smem, 0, threadIdx.x) / (float)d;
  for (int64_t j = threadIdx.x; j < d; j += 256) {
    const float xh = (Elem<T>::load1(x + base + j) - mu) * r;
    const float g = Elem<T>::load1(dy + base + j) * Elem<WT>::load1(w + j);
    float o = ((g - gmean) - xh * cmean) * r;
    if (gxn != nullptr) o += Elem<T>::load1(gxn + base + j);
    Elem<T>::store1(dx + base + j, o);
    if (dd != nullptr) Elem<T>::store1(dd + base + j, o);
  }
}

// dW (and, for LN, db) partials for the any-width path: grid (ceil(d/64), chunks); chunk c owns
// rows [c*rows_per_chunk, ...); 4 row lanes x 64 columns per workgroup. Partial rows are
// `pcols` floats wide: d weight columns, then d bias columns for LN.
template <typename T, bool LN>
__global__ __launch_bounds__(256) void dw_generic(const T* __restrict__ x,
                                                   const float* __restrict__ mean,
                                                   const float* __restrict__ rstd,
                                                   const T* __restrict__ dy,
                                                   float* __restrict__ partial, int64_t n,
                                                   int64_t d, int64_t rows_per_chunk) {
  __shared__ float s[4][64];
  __shared__ float sb[LN ? 4 : 1][64];
  const int lane = threadIdx.x & 63;
  const int g = threadIdx.x >> 6;
  const int64_t col = (int64_t)blockIdx.x * 64 + lane;
  const int64_t r0 = (int64_t)blockIdx.y * rows_per_chunk;
  const int64_t r1 = (r0 + rows_per_chunk < n) ? r0 + rows_per_chunk : n;
  const int64_t pcols = LN ? 2 * d : d;
  float a = 0.f, ab = 0.f;
  if (col < d) {
    for (int64_t r = r0 + g; r < r1; r += 4) {
      const float gv = Elem<T>::load1(dy + r * d + col);
      float xv = Elem<T>::load1(x + r * d + col);
      if constexpr (LN) { xv -= mean[r]; ab += gv; }
      a += gv * (xv * rstd[r]);
    }
  }
  s[g][lane] = a;
  if constexpr (LN) sb[g][lane] = ab;
  __syncthreads();
  if (g == 0 && col < d) {
    partial[(int64_t)blockIdx.y * pcols + col] = (s[0][lane] + s[1][lane]) + (s[2][lane] + s[3][lane]);
    if constexpr (LN)
      partial[(int64_t)blockIdx.y * pcols + d + col] = (sb[0][lane] + sb[1][lane]) + (sb[2][lane] + sb[3][lane]);
  }
}

// The same sum for narrow weights (few column blocks of 64 would leave most of the device idle and
// each workgroup with a long serial tail): 16 columns per workgroup, four lanes per partial row,
// 256 partial rows at a time, then a two-level fold in LDS whose order depends only on (p, d).
template <typename WT>
__global__ __launch_bounds__(1024) void colsum16_kernel(const float* __restrict__ partial,
                                                         WT* __restrict__ dw, int p, int d,
                                                         int stride, WT* __restrict__ dw_second) {
  if (blockIdx.y == 1) { partial += d; dw = dw_second; }
  __shared__ float s[256][16 + 1];
  __shared__ float s2[16][16 + 1];
  const int q = threadIdx.x & 3;
  const int g = threadIdx.x >> 2;
  const int col = blockIdx.x * 16 + q * 4;
  float a[4] = {0.f, 0.f, 0.f, 0.f};
  if (col < d) {
    for (int r = g; r < p; r += 256) {
      float v[4];
      Elem<float>::unpack(load16(partial + (int64_t)r * stride + col), v);
#pragma unroll
      for (int c = 0; c < 4; ++c) a[c] += v[c];
    }
  }
#pragma unroll
  for (int c = 0; c < 4; ++c) s[g][q * 4 + c] = a[c];
  __syncthreads();
  if (threadIdx.x < 256) {   // thread (gg, c): row groups gg * 16 .. gg * 16 + 15 of column c, in order
    const int gg = threadIdx.x >> 4, c = threadIdx.x & 15;
    float t = s[gg * 16][c];
#pragma unroll
    for (int i = 1; i < 16; ++i) t += s[gg * 16 + i][c];
    s2[gg][c] = t;
  }
  __syncthreads();
  if (threadIdx.x < 16) {
    const int cc = blockIdx.x * 16 + threadIdx.x;
    if (cc < d) {
      float tot = s2[0][threadIdx.x];
#pragma unroll
      for (int i = 1; i < 16; ++i) tot += s2[i][threadIdx.x];
      Elem<WT>::store1(dw + cc, tot);
    }
  }
}

// ---------------------------------------------------------------- wide rows (16-byte vectors, streamed)
// Rows too wide for the register path (more than 4096 vectors) whose width is a whole number
// of vectors and whose buffers are aligned: one 1024-thread workgroup per row, the row read
// with 16-byte loads, reduced, and read again from cache for the output (LayerNorm: once more
// in between, for the centred second moment). Thread t owns the same vectors in every pass, so
// the sum x + delta it stored in the first pass is its own to re-read.
constexpr int kWideThreads = 1024;

template <typename T, typename WT, bool ADD, bool LN>
__global__ __launch_bounds__(kWideThreads) void norm_fwd_wide(
    const T* __restrict__ x, const T* __restrict__ delta, const WT* __restrict__ w,
    const WT* __restrict__ bias, T* __restrict__ xn, T* __restrict__ y, float* __restrict__ mean,
    float* __restrict__ rstd, int d, float eps) {
  constexpr int EPV = Elem<T>::kVec;
  __shared__ float smem[kWideThreads / 64];
  const int tid = threadIdx.x;
  const int nvec = d / EPV;
  const int64_t base = (int64_t)blockIdx.x * d;
  const T* src = ADD ? xn + base : x + base;   // what the later passes read
  float ss = 0.f;
  for (int c0 = tid; c0 < nvec; c0 += 2 * kWideThreads) {
    const int c1 = c0 + kWideThreads;
    u32x4 ra[2], rb[2];
    ra[0] = load16_stream(x + base + (int64_t)c0 * EPV);
    if (c1 < nvec) ra[1] = load16_stream(x + base + (int64_t)c1 * EPV);
    if constexpr (ADD) {
      rb[0] = load16_stream(delta + base + (int64_t)c0 * EPV);
      if (c1 < nvec) rb[1] = load16_stream(delta + base + (int64_t)c1 * EPV);
    }
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int c = u == 0 ? c0 : c1;
      if (c < nvec) {
        float v[EPV];
        Elem<T>::unpack(ra[u], v);
        if constexpr (ADD) {
          float dv[EPV];
          Elem<T>::unpack(rb[u], dv);
#pragma unroll
          for (int e = 0; e < EPV; ++e) v[e] += dv[e];
          const u32x4 packed = Elem<T>::pack(v);
          store16(xn + base + (int64_t)c * EPV, packed);
          Elem<T>::unpack(packed, v);          // normalise the rounded sum, as the reference does
        }
#pragma unroll
        for (int e = 0; e < EPV; ++e) ss += LN ? v[e] : v[e] * v[e];
      }
    }
  }
  ss = row_reduce<kWideThreads, OpSum>(ss, smem, 0, tid);
  float mu = 0.f;
  if constexpr (LN) {
    mu = ss / (float)d;
    ss = 0.f;
    for (int c = tid; c < nvec; c += kWideThreads) {
      float v[EPV];
      Elem<T>::unpack(load16(src + (int64_t)c * EPV), v);
#pragma unroll
      for (int e = 0; e < EPV; ++e) ss += (v[e] - mu) * (v[e] - mu);
    }
    ss = row_reduce<kWideThreads, OpSum>(ss, smem, 0, tid);
  }
  const float r = rsqrtf(ss / (float)d + eps);
  if (tid == 0) {
    rstd[blockIdx.x] = r;
    if constexpr (LN) mean[blockIdx.x] = mu;
  }
  for (int c = tid; c < nvec; c += kWideThreads) {
    float v[EPV], wv[EPV], o[EPV];
    Elem<T>::unpack(load16(src + (int64_t)c * EPV), v);
    load_w<T, WT>(w, c * EPV, wv);
#pragma unroll
    for (int e = 0; e < EPV; ++e) o[e] = ((v[e] - mu) * r) * wv[e];
    if constexpr (LN) {
      if (bias != nullptr) {
        float bv[EPV];
        load_w<T, WT>(bias, c * EPV, bv);
#pragma unroll
        for (int e = 0; e < EPV; ++e) o[e] += bv[e];
      }
    }
    store16_stream(y + base + (int64_t)c * EPV, Elem<T>::pack(o));
  }
}

template <typename T, typename WT, bool LN>
__global__ __launch_bounds__(kWideThreads) void norm_bwd_wide(
    const T* __restrict__ x, const WT* __restrict__ w, const float* __restrict__ mean,
    const float* __restrict__ rstd, const T* __restrict__ dy, const T* __restrict__ gxn,
    T* __restrict__ dx, T* __restrict__ dd, int d) {
  constexpr int EPV = Elem<T>::kVec;
  __shared__ float smem[kWideThreads / 64];
  const int tid = threadIdx.x;
  const int nvec = d / EPV;
  const int64_t base = (int64_t)blockIdx.x * d;
  const float r = rstd[blockIdx.x];
  float mu = 0.f;
  if constexpr (LN) mu = mean[blockIdx.x];
  float dot = 0.f, gsum = 0.f;
  for (int c0 = tid; c0 < nvec; c0 += 2 * kWideThreads) {
    const int c1 = c0 + kWideThreads;
    u32x4 rx[2], rg[2];
    rx[0] = load16(x + base + (int64_t)c0 * EPV);
    rg[0] = load16(dy + base + (int64_t)c0 * EPV);
    if (c1 < nvec) {
      rx[1] = load16(x + base + (int64_t)c1 * EPV);
      rg[1] = load16(dy + base + (int64_t)c1 * EPV);
    }
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int c = u == 0 ? c0 : c1;
      if (c < nvec) {
        float xv[EPV], gv[EPV], wv[EPV];
        Elem<T>::unpack(rx[u], xv);
        Elem<T>::unpack(rg[u], gv);
        load_w<T, WT>(w, c * EPV, wv);
#pragma unroll
        for (int e = 0; e < EPV; ++e) {
          const float g = gv[e] * wv[e];
          dot += g * ((xv[e] - mu) * r);
          gsum += g;
        }
      }
    }
  }
  dot = row_reduce<kWideThreads, OpSum>(dot, smem, 0, tid);
  const float cmean = dot / (float)d;
  float gmean = 0.f;
  if constexpr (LN) gmean = row_reduce<kWideThreads, OpSum>(gsum, smem, 0, tid) / (float)d;
  for (int c = tid; c < nvec; c += kWideThreads) {
    float xv[EPV], gv[EPV], wv[EPV], o[EPV];
    Elem<T>::unpack(load16(x + base + (int64_t)c * EPV), xv);
    Elem<T>::unpack(load16(dy + base + (int64_t)c * EPV), gv);
    load_w<T, WT>(w, c * EPV, wv);
#pragma unroll
    for (int e = 0; e < EPV; ++e) o[e] = ((gv[e] * wv[e] - gmean) - ((xv[e] - mu) * r) * cmean) * r;
    if (gxn != nullptr) {
      float rv[EPV];
      Elem<T>::unpack(load16_stream(gxn + base + (int64_t)c * EPV), rv);
#pragma unroll
      for (int e = 0; e < EPV; ++e) o[e] += rv[e];
    }
    const u32x4 packed = Elem<T>::pack(o);
    store16_stream(dx + base + (int64_t)c * EPV, packed);
    if (dd != nullptr) store16_stream(dd + base + (int64_t)c * EPV, packed);
  }
}

// Rows just past the register path (up to ITERS vectors per thread of a 1024-thread workgroup,
// ITERS * EPV <= 32: 32768 columns): the per-thread fp32 column sums of the weight gradient still
// fit the registers, so one persistent kernel does the whole backward. A workgroup walks a
// contiguous chunk of rows and holds the packed x and dy of a row on the chip between the
// reduction and the output sweep (2 reads + 1 write from HBM, as on the register path; re-reading
// them through the caches instead was 1.5 times slower). The weight comes from cache each time,
// not from registers or LDS.
//
// Loads are unconditional, from clamped columns (a load behind a lane-dependent branch is waited
// for at once). With PARK the dy vectors live in LDS instead of registers, filled straight from
// memory (16 bytes a lane, no register in between): the forms with the most accumulators
// (LayerNorm from four vectors a thread, fp32 rows) otherwise push registers out to scratch.
// With PIPE the NEXT row is loaded from inside the output sweep (a vector that has given its
// output hands its registers, or its LDS slot, to the same columns of the next row): the one
// workgroup a compute unit holds otherwise loads, reduces and stores in turn. That pays for the
// widest fp32 rows only; elsewhere the wait for the previous row's stores at the top of a row
// (one counter for a wave's loads and stores) costs what the overlap gains.
template <typename T, typename WT, bool LN, int ITERS, bool PARK = false, bool PIPE = false>
__global__ __launch_bounds__(kWideThreads) void norm_bwd_wide_acc(
    const T* __restrict__ x, const WT* __restrict__ w, const float* __restrict__ mean,
    const float* __restrict__ rstd, const T* __restrict__ dy, const T* __restrict__ gxn,
    T* __restrict__ dx, T* __restrict__ dd, float* __restrict__ partial, int64_t n, int d,
    int64_t rows_per_chunk) {
  constexpr int EPV = Elem<T>::kVec;
  constexpr int NB = LN ? ITERS : 1;
  __shared__ float smem[kWideThreads / 64];
  extern __shared__ u32x4 parked[];   // PARK: [ITERS][threads], dy of the row (64 KB at four vectors)
  const int tid = threadIdx.x;
  const int wave_first = __builtin_amdgcn_readfirstlane(tid & ~63);
  const int nvec = d / EPV;
  const float inv_d = 1.f / (float)d;
  float acc[ITERS][EPV], accb[NB][EPV];
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
#pragma unroll
    for (int e = 0; e < EPV; ++e) acc[i][e] = 0.f;
  }
#pragma unroll
  for (int i = 0; i < NB; ++i) {
#pragma unroll
    for (int e = 0; e < EPV; ++e) accb[i][e] = 0.f;
  }
  const int64_t r0 = (int64_t)blockIdx.x * rows_per_chunk;
  const int64_t r1 = (r0 + rows_per_chunk < n) ? r0 + rows_per_chunk : n;
  // column of this thread in slot i, clamped into the row for the loads
  int col[ITERS];
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
    const int c = i * kWideThreads + tid;
    col[i] = (c < nvec ? c : nvec - 1) * EPV;
  }
  u32x4 rx[ITERS], rg[PARK ? 1 : ITERS];
  auto fetch = [&](int i, int64_t base) {
    rx[i] = load16_stream(x + base + col[i]);
    if constexpr (PARK) load16_stream_to_lds(dy + base + col[i], parked + i * kWideThreads + wave_first);
    else rg[i] = load16_stream(dy + base + col[i]);
  };
  if (PIPE && r0 < r1) {
#pragma unroll
    for (int i = 0; i < ITERS; ++i) fetch(i, r0 * (int64_t)d);
  }
  for (int64_t row = r0; row < r1; ++row) {
    const int64_t base = row * (int64_t)d;
    if constexpr (!PIPE) {
#pragma unroll
      for (int i = 0; i < ITERS; ++i) fetch(i, base);
    }
    const float r = rstd[row];
    float mu = 0.f;
    if constexpr (LN) mu = mean[row];
    if constexpr (PARK) wait_vmem_all();   // the LDS slots were filled by loads that name no register
    float dot = 0.f, gsum = 0.f;
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      const int c = i * kWideThreads + tid;
      touch(rx[i]);
      u32x4 g;
      if constexpr (PARK) g = parked[i * kWideThreads + tid];
      else { touch(rg[i]); g = rg[i]; }
      if (c < nvec) {
        float xv[EPV], gv[EPV], wv[EPV];
        Elem<T>::unpack(rx[i], xv);
        Elem<T>::unpack(g, gv);
        load_w<T, WT>(w, c * EPV, wv);
#pragma unroll
        for (int e = 0; e < EPV; ++e) {
          const float xh = (xv[e] - mu) * r;
          acc[i][e] += gv[e] * xh;
          dot += (gv[e] * wv[e]) * xh;
          if constexpr (LN) {
            accb[i][e] += gv[e];
            gsum += gv[e] * wv[e];
          }
        }
      }
    }
    dot = row_reduce<kWideThreads, OpSum>(dot, smem, 0, tid);
    const float cmean = dot * inv_d;
    float gmean = 0.f;
    if constexpr (LN) gmean = row_reduce<kWideThreads, OpSum>(gsum, smem, 0, tid) * inv_d;
    const bool more = row + 1 < r1;   // the same for the whole workgroup
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      const int c = i * kWideThreads + tid;
      touch(rx[i]);
      u32x4 g;
      if constexpr (PARK) {
        g = parked[i * kWideThreads + tid];
        touch(g);   // in registers before the slot is given away
      } else {
        touch(rg[i]);
        g = rg[i];
      }
      const u32x4 xr = rx[i];
      if (PIPE && more) fetch(i, base + d);
      if (c < nvec) {
        float xv[EPV], gv[EPV], wv[EPV], o[EPV];
        Elem<T>::unpack(xr, xv);
        Elem<T>::unpack(g, gv);
        load_w<T, WT>(w, c * EPV, wv);
#pragma unroll
        for (int e = 0; e < EPV; ++e) o[e] = ((gv[e] * wv[e] - gmean) - ((xv[e] - mu) * r) * cmean) * r;
        if (gxn != nullptr) {
          float rv[EPV];
          Elem<T>::unpack(load16_stream(gxn + base + (int64_t)c * EPV), rv);
#pragma unroll
          for (int e = 0; e < EPV; ++e) o[e] += rv[e];
        }
        const u32x4 packed = Elem<T>::pack(o);
        store16_stream(dx + base + (int64_t)c * EPV, packed);
        if (dd != nullptr) store16_stream(dd + base + (int64_t)c * EPV, packed);
      }
    }
  }
  if (partial == nullptr) return;
  const int64_t pcols = LN ? 2 * (int64_t)d : d;
  float* prow = partial + (int64_t)blockIdx.x * pcols;
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
    const int c = i * kWideThreads + tid;
    if (c < nvec) {
#pragma unroll
      for (int q = 0; q < EPV / 4; ++q) {
        float o4[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) o4[j] = acc[i][4 * q + j];
        store16(prow + c * EPV + 4 * q, Elem<float>::pack(o4));
        if constexpr (LN) {
#pragma unroll
          for (int j = 0; j < 4; ++j) o4[j] = accb[i][4 * q + j];
          store16(prow + d + c * EPV + 4 * q, Elem<float>::pack(o4));
        }
      }
    }
  }
}

// dW (and, for LN, db) partials of the wide path: grid (ceil(nvec / 64), chunks); a workgroup
// owns 64 vector columns and the rows of its chunk, four row lanes of 64 threads each; the
// four are folded in a fixed order. Partial rows as in dw_generic.
template <typename T, bool LN>
__global__ __launch_bounds__(256) void dw_wide(const T* __restrict__ x, const float* __restrict__ mean,
                                                const float* __restrict__ rstd,
                                                const T* __restrict__ dy, float* __restrict__ partial,
                                                int64_t n, int d, int64_t rows_per_chunk) {
  constexpr int EPV = Elem<T>::kVec;
  __shared__ float s[4][64][EPV + 1];
  const int lane = threadIdx.x & 63, g = threadIdx.x >> 6;
  const int nvec = d / EPV;
  const int c = blockIdx.x * 64 + lane;
  const int64_t r0 = (int64_t)blockIdx.y * rows_per_chunk;
  const int64_t r1 = (r0 + rows_per_chunk < n) ? r0 + rows_per_chunk : n;
  const int64_t pcols = LN ? 2 * (int64_t)d : d;
  float acc[EPV], accb[EPV];
#pragma unroll
  for (int e = 0; e < EPV; ++e) { acc[e] = 0.f; accb[e] = 0.f; }
  if (c < nvec) {
    for (int64_t r = r0 + g; r < r1; r += 4) {
      float xv[EPV], gv[EPV];
      Elem<T>::unpack(load16(x + r * d + (int64_t)c * EPV), xv);
      Elem<T>::unpack(load16(dy + r * d + (int64_t)c * EPV), gv);
      const float rs = rstd[r];
      float mu = 0.f;
      if constexpr (LN) mu = mean[r];
#pragma unroll
      for (int e = 0; e < EPV; ++e) {
        acc[e] += gv[e] * ((xv[e] - mu) * rs);
        if constexpr (LN) accb[e] += gv[e];
      }
    }
  }
#pragma unroll
  for (int which = 0; which < (LN ? 2 : 1); ++which) {
    if (which == 1) __syncthreads();
#pragma unroll
    for (int e = 0; e < EPV; ++e) s[g][lane][e] = which == 0 ? acc[e] : accb[e];
    __syncthreads();
    if (g == 0 && c < nvec) {
      float* out = partial + (int64_t)blockIdx.y * pcols + (int64_t)which * d + (int64_t)c * EPV;
#pragma unroll
      for (int e = 0; e < EPV; ++e) out[e] = (s[0][lane][e] + s[1][lane][e]) + (s[2][lane][e] + s[3][lane][e]);
    }
  }
}

__global__ void zero_u16_kernel(uint16_t* p, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

// ---------------------------------------------------------------- host: plan + dispatch
struct Plan {
  bool vec;        // register-resident vector path
  bool wide;       // streamed vector path (rows past the register path)
  bool bwd_vec, bwd_wide;  // the same two for the backward, whose register path ends earlier
  int tpr, iters;  // threads per row, 16-byte vectors per thread
  int rpb;         // rows per workgroup
  int64_t tiles;   // row tiles of the forward (vector path)
  int64_t bwd_tiles;  // row tiles of the backward
  int bwd_blocks;  // persistent grid of the backward == partial rows
  int64_t rows_per_chunk;  // any-width path
};

int elem_size(int dt) { return dt == FM_F32 ? 4 : 2; }

Plan make_plan(int64_t n, int64_t d, int x_dtype, bool aligned) {
  Plan p{};
  const int epv = 16 / elem_size(x_dtype);
  const int64_t nvec = d / epv;
  // rows of more than `reg_max` vectors are streamed
  const int64_t reg_max = 4096;
  p.vec = aligned && (d % epv == 0) && nvec <= reg_max;
  p.wide = aligned && (d % epv == 0) && nvec > reg_max;
  // the backward of half types keeps x, dy and two fp32 column sets per thread: past 2048
  // vectors that no longer fits 128 registers, and streaming the row is faster than spilling
  const int64_t bwd_max = (elem_size(x_dtype) == 2 && reg_max > 2048) ? 2048 : reg_max;
  p.bwd_vec = p.vec && nvec <= bwd_max;
  p.bwd_wide = aligned && (d % epv == 0) && nvec > bwd_max;
  if (p.vec) {
    if (nvec <= 64) {
      int t = 4;
      while (t < nvec) t *= 2;
      p.tpr = t; p.iters = 1;
    } else {
      static const int kPairs[][3] = {{128, 64, 2},   {192, 64, 3},    {256, 128, 2},  {384, 128, 3},
                                      {512, 256, 2},  {768, 256, 3},   {1024, 512, 2}, {1536, 512, 3},
                                      {2048, 1024, 2}, {3072, 1024, 3}, {4096, 1024, 4}};
      for (auto& pr : kPairs) {
        if (nvec <= pr[0]) { p.tpr = pr[1]; p.iters = pr[2]; break; }
      }
    }
    const int block = p.tpr > kMinBlock ? p.tpr : kMinBlock;
    p.rpb = block / p.tpr;
    p.tiles = (n + p.rpb - 1) / p.rpb;
  }
  if (p.bwd_vec) {
    p.bwd_tiles = (n + (kBwdBlock / p.tpr) - 1) / (kBwdBlock / p.tpr);
    int per_cu = fm_host::get_param(fm_host::P_NORM_BWD_BLOCKS_PER_CU);
    if (per_cu <= 0) per_cu = 1;
    int64_t blocks = (int64_t)fm_host::num_cus() * per_cu;
    if (blocks > p.bwd_tiles) blocks = p.bwd_tiles;
    if (blocks < 1) blocks = 1;
    p.bwd_blocks = (int)blocks;
  } else {
    int64_t chunks = n < 256 ? n : 256;
    if (chunks < 1) chunks = 1;
    p.rows_per_chunk = (n + chunks - 1) / chunks;
    p.bwd_blocks = (int)((n + p.rows_per_chunk - 1) / (p.rows_per_chunk > 0 ? p.rows_per_chunk : 1));
    if (p.bwd_blocks < 1) p.bwd_blocks = 1;
  }
  return p;
}

#define FM_FOR_EACH_SHAPE(X) \
  X(4, 1) X(8, 1) X(16, 1) X(32, 1) X(64, 1) X(64, 2) X(64, 3) X(128, 2) X(128, 3)    \
  X(256, 2) X(256, 3) X(512, 2) X(512, 3) X(1024, 2) X(1024, 3) X(1024, 4)

// Persistent grid of the forward: every workgroup slot of the device exactly once, so the
// hardware places the same number of workgroups on every compute unit.
inline int64_t fwd_grid(const Plan& p, int occupancy) {
  int per_cu = fm_host::get_param(fm_host::P_NORM_FWD_BLOCKS_PER_CU);
  if (per_cu <= 0) per_cu = occupancy;
  int64_t g = (int64_t)fm_host::num_cus() * per_cu;
  if (g > p.tiles) g = p.tiles;
  return g < 1 ? 1 : g;
}

template <typename T, typename WT, bool ADD, bool LN>
int launch_fwd(const Plan& p, const void* x, const void* delta, const void* w, const void* bias,
               void* xn, void* y, float* mean, float* rstd, int64_t n, int64_t d, float eps,
               hipStream_t st) {
  const T* xp = static_cast<const T*>(x);
  const T* dp = static_cast<const T*>(delta);
  const WT* wp = static_cast<const WT*>(w);
  const WT* bp = static_cast<const WT*>(bias);
  T* xnp = static_cast<T*>(xn);
  T* yp = static_cast<T*>(y);
  if (p.wide) {
    FM_LAUNCH((norm_fwd_wide<T, WT, ADD, LN>), dim3((unsigned)n), dim3(kWideThreads), 0, st, xp,
                       dp, wp, bp, xnp, yp, mean, rstd, (int)d, eps);
    return FM_OK;
  }
  if (!p.vec) {
    FM_LAUNCH((norm_fwd_generic<T, WT, ADD, LN>), dim3((unsigned)n), dim3(256), 0, st, xp, dp,
                       wp, bp, xnp, yp, mean, rstd, d, eps);
    return FM_OK;
  }
  // measured on fwd + bwd pairs of a plain RMSNorm (us, streamed | kept): 128 MiB 119.6 | 116.6,
  // 256 MiB 229.8 | 219.7; the fused add at [16384,8192] bf16 loses 60 us when x is kept
  const bool keep = !ADD && n * d * (int64_t)sizeof(T) <= (256ll << 20);
#define X(TPR_, IT_)                                                                            \
  if (p.tpr == TPR_ && p.iters == IT_) {                                                        \
    constexpr int block_ = BlockOf<TPR_>::value;                                                \
    if (keep) {                                                                                 \
      constexpr auto kern_ = norm_fwd_kernel<T, WT, TPR_, IT_, ADD, LN, !ADD>;                  \
      const int occ_ = fm_host::resident_per_cu<kern_>(block_, 0);                              \
      FM_LAUNCH((norm_fwd_kernel<T, WT, TPR_, IT_, ADD, LN, !ADD>),                             \
                dim3((unsigned)fwd_grid(p, occ_)), dim3(block_), 0, st, xp, dp, wp, bp, xnp, yp, \
                mean, rstd, n, (int)d, eps, p.tiles);                                           \
    } else {                                                                                    \
      constexpr auto kern_ = norm_fwd_kernel<T, WT, TPR_, IT_, ADD, LN, false>;                 \
      const int occ_ = fm_host::resident_per_cu<kern_>(block_, 0);                              \
      FM_LAUNCH((norm_fwd_kernel<T, WT, TPR_, IT_, ADD, LN, false>),                            \
                dim3((unsigned)fwd_grid(p, occ_)), dim3(block_), 0, st, xp, dp, wp, bp, xnp, yp, \
                mean, rstd, n, (int)d, eps, p.tiles);                                           \
    }                                                                                           \
    return FM_OK;                                                                               \
  }
  FM_FOR_EACH_SHAPE(X)
#undef X
  fm_host::set_error("norm: no kernel for tpr=%d iters=%d", p.tpr, p.iters);
  return FM_ERR_UNSUPPORTED;
}

template <typename T, typename WT, bool LN>
int launch_bwd(const Plan& p, const void* x, const void* w, const float* mean, const float* rstd,
               const void* dy, const void* gxn, void* dx, void* dd, void* dw, void* db, float* partial,
               int64_t n, int64_t d, hipStream_t st) {
  const T* xp = static_cast<const T*>(x);
  const WT* wp = static_cast<const WT*>(w);
  const T* dyp = static_cast<const T*>(dy);
  const T* gp = static_cast<const T*>(gxn);
  T* dxp = static_cast<T*>(dx);
  T* ddp = static_cast<T*>(dd);
  if (dw == nullptr && db == nullptr) partial = nullptr;
  const int pcols = (int)(LN ? 2 * d : d);
  const int wide_iters = (int)((d / Elem<T>::kVec + kWideThreads - 1) / kWideThreads);
  const bool acc_fits = wide_iters * Elem<T>::kVec <= 32 && !(LN && sizeof(T) == 4 && wide_iters > 6);
  if (p.bwd_wide && acc_fits) {
    // the column sums fit the registers: one persistent kernel, a chunk of rows per workgroup
    const dim3 grid((unsigned)p.bwd_blocks);
    // dy in LDS (PARK) where it would otherwise push registers out to scratch, the next row loaded
    // under the output sweep (PIPE) where that pays; measured per form (us, RMSNorm / LayerNorm,
    // plain | PARK | PARK + PIPE): bf16 [7281,18432] 167 / 186 | 171 / 191 | 174 / 217;
    // bf16 [4096,32768] 167 / 345 | 173 / 214 | 167 / 236; fp32 [3276,20480] 173 / 257 | 160 / 202 |
    // 160 / 223; fp32 [2048,32768] 291 | 211 | 181.
    constexpr int kMaxIt = 32 / Elem<T>::kVec;
#define GOA(IT_)                                                                                  \
  do {                                                                                            \
    constexpr bool park_ = LN ? (IT_ >= 4) : (sizeof(T) == 4);                                    \
    constexpr bool pipe_ = sizeof(T) == 4 && IT_ == 8;                                            \
    constexpr int lds_ = park_ ? IT_ * kWideThreads * 16 : 0;                                     \
    if (lds_ == 0 || fm_host::grant_dynamic_lds<&norm_bwd_wide_acc<T, WT, LN, IT_, park_, pipe_>>(lds_)) \
      FM_LAUNCH((norm_bwd_wide_acc<T, WT, LN, IT_, park_, pipe_>), grid, dim3(kWideThreads), (size_t)lds_, \
                st, xp, wp, mean, rstd, dyp, gp, dxp, ddp, partial, n, (int)d, p.rows_per_chunk); \
    else                                                                                          \
      FM_LAUNCH((norm_bwd_wide_acc<T, WT, LN, IT_, false, false>), grid, dim3(kWideThreads), 0, st, xp, wp, \
                mean, rstd, dyp, gp, dxp, ddp, partial, n, (int)d, p.rows_per_chunk);             \
  } while (0)
    if (wide_iters <= 3 && kMaxIt >= 3) GOA(3);
    else if (wide_iters <= 4 || kMaxIt < 8) GOA(4);
    else if (wide_iters <= 6) {
      if constexpr (kMaxIt >= 6) GOA(6);
      else GOA(4);
    } else {
      if constexpr (kMaxIt >= 8) GOA(8);
      else GOA(4);
    }
#undef GOA
  } else if (p.bwd_wide) {
    FM_LAUNCH((norm_bwd_wide<T, WT, LN>), dim3((unsigned)n), dim3(kWideThreads), 0, st, xp, wp,
                       mean, rstd, dyp, gp, dxp, ddp, (int)d);
    if (partial != nullptr) {
      const int nvec = (int)(d / Elem<T>::kVec);
      dim3 grid((unsigned)((nvec + 63) / 64), (unsigned)p.bwd_blocks);
      hipLaunchKernelGGL((dw_wide<T, LN>), grid, dim3(256), 0, st, xp, mean, rstd, dyp, partial, n, (int)d,
                         p.rows_per_chunk);
    }
  } else if (!p.bwd_vec) {
    FM_LAUNCH((norm_bwd_generic<T, WT, LN>), dim3((unsigned)n), dim3(256), 0, st, xp, wp, mean,
                       rstd, dyp, gp, dxp, ddp, d);
    if (partial != nullptr) {
      dim3 grid((unsigned)((d + 63) / 64), (unsigned)p.bwd_blocks);
      hipLaunchKernelGGL((dw_generic<T, LN>), grid, dim3(256), 0, st, xp, mean, rstd, dyp, partial, n, d,
                         p.rows_per_chunk);
    }
  } else {
    bool done = false;
    // an x that fits the 256 MiB memory-side cache is read with cached loads (see the kernel)
    const bool x_cached = n * d * (int64_t)sizeof(T) <= (256ll << 20);
#define X(TPR_, IT_)                                                                           \
  if (!done && p.tpr == TPR_ && p.iters == IT_) {                                              \
    if (x_cached)                                                                              \
      FM_LAUNCH((norm_bwd_kernel<T, WT, TPR_, IT_, LN, true>), dim3((unsigned)p.bwd_blocks),   \
                dim3(kBwdBlock), 0, st, xp, wp, mean, rstd, dyp, gp, dxp, ddp, partial, n, (int)d, \
                p.bwd_tiles);                                                                  \
    else                                                                                       \
      FM_LAUNCH((norm_bwd_kernel<T, WT, TPR_, IT_, LN, false>), dim3((unsigned)p.bwd_blocks),  \
                dim3(kBwdBlock), 0, st, xp, wp, mean, rstd, dyp, gp, dxp, ddp, partial, n, (int)d, \
                p.bwd_tiles);                                                                  \
    done = true;                                                                               \
  }
    FM_FOR_EACH_SHAPE(X)
#undef X
    if (!done) {
      fm_host::set_error("norm_bwd: no kernel for tpr=%d iters=%d", p.tpr, p.iters);
      return FM_ERR_UNSUPPORTED;
    }
  }
  if (partial != nullptr) {
    // LayerNorm with both parameter gradients wanted: one launch, two rows of workgroups
    const bool both = LN && dw != nullptr && db != nullptr;
    void* outs[2] = {dw, LN ? db : nullptr};
    for (int which = 0; which < (LN && !both ? 2 : 1); ++which) {
      if (outs[which] == nullptr) continue;
      const float* src = partial + (int64_t)which * d;
      WT* first = static_cast<WT*>(outs[which]);
      WT* second = both ? static_cast<WT*>(db) : nullptr;
      const unsigned gy = both ? 2u : 1u;
      // narrow weights: 16 columns a workgroup, so that a column sum of few columns still spreads
      // over the device (no difference from 8192 columns on)
      if (d % 4 == 0 && d <= 4096)
        hipLaunchKernelGGL((colsum16_kernel<WT>), dim3((unsigned)((d + 15) / 16), gy), dim3(1024), 0, st, src,
                           first, p.bwd_blocks, (int)d, pcols, second);
      else if (d % 4 == 0)
        hipLaunchKernelGGL((colsum_kernel<WT>), dim3((unsigned)((d + 63) / 64), gy), dim3(1024), 0, st, src, first,
                           p.bwd_blocks, (int)d, pcols, second);
      else
        hipLaunchKernelGGL((colsum_scalar_kernel<WT>), dim3((unsigned)((d + 63) / 64), gy), dim3(1024), 0, st, src,
                           first, p.bwd_blocks, (int)d, pcols, second);
    }
  }
  return FM_OK;
}

int check_common(const char* what, int64_t n, int64_t d, int x_dtype, int w_dtype) {
  FM_CHECK_ARG(n >= 0 && d > 0, "%s: bad shape n=%lld d=%lld", what, (long long)n, (long long)d);
  FM_CHECK_ARG(x_dtype == FM_F32 || x_dtype == FM_F16 || x_dtype == FM_BF16, "%s: bad x_dtype %d",
               what, x_dtype);
  FM_CHECK_ARG(w_dtype == x_dtype || w_dtype == FM_F32,
               "%s: w_dtype must equal x_dtype or be fp32 (got x=%d w=%d)", what, x_dtype, w_dtype);
  if (n > 0x7fffffffLL || d > 0x7fffffffLL) {
    fm_host::set_error("%s: n and d must be below 2^31", what);
    return FM_ERR_UNSUPPORTED;
  }
  return FM_OK;
}

template <bool ADD, bool LN>
int fwd_entry(const char* what, const void* x, const void* delta, const void* w, const void* bias,
              void* xn, void* y, float* mean, float* rstd, int64_t n, int64_t d, int x_dtype,
              int w_dtype, float eps, fm_stream_t stream) {
  int rc = check_common(what, n, d, x_dtype, w_dtype);
  if (rc != FM_OK) return rc;
  if (n == 0) return FM_OK;
  FM_CHECK_ARG(x && w && y && rstd && (!ADD || (delta && xn)) && (!LN || mean), "%s: NULL pointer", what);
  bool al = fm_host::aligned16(x) && fm_host::aligned16(w) && fm_host::aligned16(y) &&
            fm_host::aligned16(bias);
  if (ADD) al = al && fm_host::aligned16(delta) && fm_host::aligned16(xn);
  const Plan p = make_plan(n, d, x_dtype, al);
  hipStream_t st = static_cast<hipStream_t>(stream);
#define CALL(T, WT) rc = launch_fwd<T, WT, ADD, LN>(p, x, delta, w, bias, xn, y, mean, rstd, n, d, eps, st)
  if (x_dtype == FM_F32) CALL(float, float);
  else if (x_dtype == FM_BF16 && w_dtype == FM_BF16) CALL(bf16_t, bf16_t);
  else if (x_dtype == FM_BF16) CALL(bf16_t, float);
  else if (w_dtype == FM_F16) CALL(f16_t, f16_t);
  else CALL(f16_t, float);
#undef CALL
  if (rc != FM_OK) return rc;
  FM_CHECK_LAUNCH(what);
  return FM_OK;
}

template <bool LN>
int bwd_entry(const char* what, const void* x, const void* w, const float* mean, const float* rstd,
              const void* dy, const void* gxn, void* dx, void* dd, void* dw, void* db, void* workspace,
              size_t workspace_bytes, int64_t n, int64_t d, int x_dtype, int w_dtype,
              fm_stream_t stream) {
  int rc = check_common(what, n, d, x_dtype, w_dtype);
  if (rc != FM_OK) return rc;
  FM_CHECK_ARG(w != nullptr, "%s: NULL weight", what);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (n == 0) {
    // empty batch: the parameter gradients are exactly zero. A fill kernel rather than a
    // memset node, so the call stays safe under graph capture.
    const int64_t words = ((int64_t)d * elem_size(w_dtype) + 1) / 2;
    void* outs[2] = {dw, LN ? db : nullptr};
    for (void* o : outs) {
      if (o == nullptr) continue;
      hipLaunchKernelGGL(zero_u16_kernel, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, st,
                         static_cast<uint16_t*>(o), words);
      FM_CHECK_LAUNCH(what);
    }
    return FM_OK;
  }
  FM_CHECK_ARG(x && rstd && dy && dx && (!LN || mean), "%s: NULL pointer", what);
  if (dd == dx) dd = nullptr;
  bool al = fm_host::aligned16(x) && fm_host::aligned16(w) && fm_host::aligned16(dy) &&
            fm_host::aligned16(dx) && fm_host::aligned16(gxn) && fm_host::aligned16(dd) &&
            fm_host::aligned16(workspace);
  const Plan p = make_plan(n, d, x_dtype, al);
  if (dw != nullptr || (LN && db != nullptr)) {
    const size_t need = (size_t)p.bwd_blocks * (size_t)d * sizeof(float) * (LN ? 2 : 1);
    if (workspace == nullptr || workspace_bytes < need) {
      fm_host::set_error("%s: workspace of %zu bytes needed, %zu given", what, need, workspace_bytes);
      return FM_ERR_WORKSPACE;
    }
  }
  float* partial = static_cast<float*>(workspace);
#define CALL(T, WT) \
  rc = launch_bwd<T, WT, LN>(p, x, w, mean, rstd, dy, gxn, dx, dd, dw, db, partial, n, d, st)
  if (x_dtype == FM_F32) CALL(float, float);
  else if (x_dtype == FM_BF16 && w_dtype == FM_BF16) CALL(bf16_t, bf16_t);
  else if (x_dtype == FM_BF16) CALL(bf16_t, float);
  else if (w_dtype == FM_F16) CALL(f16_t, f16_t);
  else CALL(f16_t, float);
#undef CALL
  if (rc != FM_OK) return rc;
  FM_CHECK_LAUNCH(what);
  return FM_OK;
}

// bytes of backward workspace: the larger of the two paths, so the answer does not depend on
// pointer alignment
inline size_t bwd_workspace_bytes(int64_t n, int64_t d, int x_dtype, bool ln) {
  if (n <= 0 || d <= 0) return 0;
  const Plan a = make_plan(n, d, x_dtype, true);
  const Plan b = make_plan(n, d, x_dtype, false);
  const int p = a.bwd_blocks > b.bwd_blocks ? a.bwd_blocks : b.bwd_blocks;
  return (size_t)p * (size_t)d * sizeof(float) * (ln ? 2 : 1);
}

}  // namespace
