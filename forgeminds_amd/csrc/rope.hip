// Per-head RMSNorm followed by half-split RoPE, forward and backward, for gfx950.
//
// Reference semantics: forgemind/kernels/_fallback.py:38-45 and forgemind/kernels/rope.py:46-120:
// x is [B, T, H, D]; per head r = rsqrt(mean(x^2) + eps), y = x * r * w, then with the halves
// (y1, y2) and cos/sin [T, D/2]:  out = (y1*cos - y2*sin, y1*sin + y2*cos), one rounding.
// Backward: rotate the incoming gradient back (dy1 = do1*cos + do2*sin, dy2 = -do1*sin + do2*cos),
// then the RMSNorm backward of norm.hip; dw = sum over heads of dy * xhat in fp32, written as
// one partial row per workgroup and summed in a fixed order.
//
// Heads are short (64-256 elements), so a head is owned by a group of G lanes; a lane holds one
// 16-byte vector of each half (the same columns of both), which keeps both rotation partners
// in one thread and every access 16 bytes wide. Head dims that do not split into 16-byte
// vectors per half, or unaligned buffers, use a scalar variant (four elements of each half per
// lane). Grids are persistent: the weight columns stay in registers, cos/sin rows are shared by
// the heads of a token and come from cache.
#include "fm_norm.hip.h"   // colsum_kernel / colsum_scalar_kernel: fixed-order column sums of partial rows

using namespace fm;

namespace {

constexpr int kEH = 4;        // elements per lane per half
constexpr int kBlock = 256;

// Position of a row's token in its sequence. The entry points refuse more than 2^31 - 1 rows, so the
// two divisions are 32-bit ones (a 64-bit division is some two hundred dependent instructions, paid
// by every tile of every wave).
__device__ __forceinline__ int token_of(int64_t row, int heads, int t_len) {
  return (int)(((uint32_t)row / (uint32_t)heads) % (uint32_t)t_len);
}

template <typename T, typename WT, int G, bool BWD>
__global__ __launch_bounds__(kBlock) void rope_kernel(const T* __restrict__ x, const WT* __restrict__ w,
                                                       const float* __restrict__ cosv,
                                                       const float* __restrict__ sinv,
                                                       const T* __restrict__ dout, float* __restrict__ rstd,
                                                       T* __restrict__ out, float* __restrict__ partial,
                                                       int64_t rows, int t_len, int heads, int d, float eps,
                                                       int64_t tiles) {
  constexpr int RPB = kBlock / G;
  __shared__ float fold[BWD ? RPB * G * 2 * kEH : 1];
  const int tid = threadIdx.x, rib = tid / G, l = tid % G;
  const int half = d / 2;
  float wv1[kEH], wv2[kEH], a1[kEH], a2[kEH];
#pragma unroll
  for (int e = 0; e < kEH; ++e) {
    const int j = l * kEH + e;
    wv1[e] = j < half ? Elem<WT>::load1(w + j) : 0.f;
    wv2[e] = j < half ? Elem<WT>::load1(w + half + j) : 0.f;
    a1[e] = 0.f; a2[e] = 0.f;
  }
  for (int64_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
    const int64_t row = tile * RPB + rib;
    const bool valid = row < rows;
    const int t = valid ? token_of(row, heads, t_len) : 0;
    const T* xp = x + row * (int64_t)d;
    float x1[kEH], x2[kEH], c[kEH], s[kEH];
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < kEH; ++e) {
      const int j = l * kEH + e;
      const bool on = valid && j < half;
      x1[e] = on ? Elem<T>::load1(xp + j) : 0.f;
      x2[e] = on ? Elem<T>::load1(xp + half + j) : 0.f;
      c[e] = on ? cosv[(int64_t)t * half + j] : 0.f;
      s[e] = on ? sinv[(int64_t)t * half + j] : 0.f;
      ss += x1[e] * x1[e] + x2[e] * x2[e];
    }
    if constexpr (!BWD) {
      ss = group_reduce<G, OpSum>(ss);
      const float r = rsqrtf(ss / (float)d + eps);
      if (valid && l == 0) rstd[row] = r;
      T* op = out + row * (int64_t)d;
#pragma unroll
      for (int e = 0; e < kEH; ++e) {
        const int j = l * kEH + e;
        if (valid && j < half) {
          const float y1 = (x1[e] * r) * wv1[e], y2 = (x2[e] * r) * wv2[e];
          Elem<T>::store1(op + j, y1 * c[e] - y2 * s[e]);
          Elem<T>::store1(op + half + j, y1 * s[e] + y2 * c[e]);
        }
      }
    } else {
      const float r = valid ? rstd[row] : 0.f;
      const T* gp = dout + row * (int64_t)d;
      float g1[kEH], g2[kEH];
      float dot = 0.f;
#pragma unroll
      for (int e = 0; e < kEH; ++e) {
        const int j = l * kEH + e;
        const bool on = valid && j < half;
        const float o1 = on ? Elem<T>::load1(gp + j) : 0.f;
        const float o2 = on ? Elem<T>::load1(gp + half + j) : 0.f;
        const float dy1 = o1 * c[e] + o2 * s[e], dy2 = o2 * c[e] - o1 * s[e];
        x1[e] *= r; x2[e] *= r;                       // xhat
        a1[e] += dy1 * x1[e]; a2[e] += dy2 * x2[e];
        g1[e] = dy1 * wv1[e]; g2[e] = dy2 * wv2[e];
        dot += g1[e] * x1[e] + g2[e] * x2[e];
      }
      dot = group_reduce<G, OpSum>(dot);
      const float cm = dot / (float)d;
      T* op = out + row * (int64_t)d;
#pragma unroll
      for (int e = 0; e < kEH; ++e) {
        const int j = l * kEH + e;
        if (valid && j < half) {
          Elem<T>::store1(op + j, (g1[e] - x1[e] * cm) * r);
          Elem<T>::store1(op + half + j, (g2[e] - x2[e] * cm) * r);
        }
      }
    }
  }
  if constexpr (BWD) {
    if (partial == nullptr) return;
    // fold the rows of this workgroup in row order, then write one partial row
#pragma unroll
    for (int e = 0; e < kEH; ++e) {
      fold[(rib * 2 + 0) * G * kEH + l * kEH + e] = a1[e];
      fold[(rib * 2 + 1) * G * kEH + l * kEH + e] = a2[e];
    }
    __syncthreads();
    float* prow = partial + (int64_t)blockIdx.x * d;
    for (int j = tid; j < d; j += kBlock) {
      const int hsel = j >= half ? 1 : 0, jj = j - hsel * half;
      float acc = 0.f;
      for (int rr = 0; rr < RPB; ++rr) acc += fold[(rr * 2 + hsel) * G * kEH + jj];
      prow[j] = acc;
    }
  }
}

// 16-byte loads of fp32 tables that line up with one vector of activations
template <typename T>
__device__ __forceinline__ void load_f32_cols(const float* p, float (&o)[Elem<T>::kVec]) {
  constexpr int EPV = Elem<T>::kVec;
#pragma unroll
  for (int q = 0; q < EPV / 4; ++q) {
    float a[4];
    Elem<float>::unpack(load16(p + 4 * q), a);
#pragma unroll
    for (int i = 0; i < 4; ++i) o[4 * q + i] = a[i];
  }
}

template <typename T, typename WT>
__device__ __forceinline__ void load_w_cols(const WT* p, float (&o)[Elem<T>::kVec]) {
  constexpr int EPV = Elem<T>::kVec;
#pragma unroll
  for (int e = 0; e < EPV; ++e) o[e] = Elem<WT>::load1(p + e);
}

// H consecutive heads of one token per lane group and tile: they share the token's cos / sin
// columns, which are then fetched once per H heads instead of once per head (the tables cost
// twice the bytes of x at the L1 otherwise), and a lane has H times the bytes in flight.
template <typename T, typename WT, int G, bool BWD, int H>
__global__ __launch_bounds__(kBlock) void rope_vec_kernel(const T* __restrict__ x, const WT* __restrict__ w,
                                                           const float* __restrict__ cosv,
                                                           const float* __restrict__ sinv,
                                                           const T* __restrict__ dout,
                                                           float* __restrict__ rstd, T* __restrict__ out,
                                                           float* __restrict__ partial, int64_t rows,
                                                           int t_len, int heads, int d, float eps,
                                                           int64_t tiles) {
  constexpr int EPV = Elem<T>::kVec;
  constexpr int RPB = kBlock / G;
  __shared__ float fold[BWD ? RPB * G * 2 * EPV : 1];
  const int tid = threadIdx.x, rib = tid / G, l = tid % G;
  const int half = d / 2;
  const int col = l * EPV;               // this lane's columns in each half
  const bool lane_on = col < half;
  float wv1[EPV], wv2[EPV], a1[EPV], a2[EPV];
#pragma unroll
  for (int e = 0; e < EPV; ++e) { wv1[e] = 0.f; wv2[e] = 0.f; a1[e] = 0.f; a2[e] = 0.f; }
  if (lane_on) {
    load_w_cols<T, WT>(w + col, wv1);
    load_w_cols<T, WT>(w + half + col, wv2);
  }
  for (int64_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
    // rows is a multiple of H and so is the number of heads of a token: the H rows exist
    // together and belong to one token
    const int64_t row0 = (tile * RPB + rib) * H;
    const bool live = row0 < rows;
    const bool on = lane_on && live;
    const int t = live ? token_of(row0, heads, t_len) : 0;
    float c[EPV], sn[EPV];
#pragma unroll
    for (int e = 0; e < EPV; ++e) { c[e] = 0.f; sn[e] = 0.f; }
    u32x4 r1[H], r2[H], q1[BWD ? H : 1], q2[BWD ? H : 1];
    if (on) {
#pragma unroll
      for (int j = 0; j < H; ++j) {
        const T* xp = x + (row0 + j) * (int64_t)d;
        r1[j] = load16_stream(xp + col);
        r2[j] = load16_stream(xp + half + col);
        if constexpr (BWD) {
          const T* gp = dout + (row0 + j) * (int64_t)d;
          q1[j] = load16_stream(gp + col);
          q2[j] = load16_stream(gp + half + col);
        }
      }
      load_f32_cols<T>(cosv + (int64_t)t * half + col, c);
      load_f32_cols<T>(sinv + (int64_t)t * half + col, sn);
    }
#pragma unroll
    for (int j = 0; j < H; ++j) {
      const int64_t row = row0 + j;
      float x1[EPV], x2[EPV];
#pragma unroll
      for (int e = 0; e < EPV; ++e) { x1[e] = 0.f; x2[e] = 0.f; }
      if (on) {
        Elem<T>::unpack(r1[j], x1);
        Elem<T>::unpack(r2[j], x2);
      }
      if constexpr (!BWD) {
        float ss = 0.f;
#pragma unroll
        for (int e = 0; e < EPV; ++e) ss += x1[e] * x1[e] + x2[e] * x2[e];
        ss = group_reduce<G, OpSum>(ss);
        const float r = rsqrtf(ss / (float)d + eps);
        if (live && l == 0) rstd[row] = r;
        if (on) {
          float o1[EPV], o2[EPV];
#pragma unroll
          for (int e = 0; e < EPV; ++e) {
            const float y1 = (x1[e] * r) * wv1[e], y2 = (x2[e] * r) * wv2[e];
            o1[e] = y1 * c[e] - y2 * sn[e];
            o2[e] = y1 * sn[e] + y2 * c[e];
          }
          T* op = out + row * (int64_t)d;
          store16_stream(op + col, Elem<T>::pack(o1));
          store16_stream(op + half + col, Elem<T>::pack(o2));
        }
      } else {
        const float r = live ? rstd[row] : 0.f;
        float g1[EPV], g2[EPV];
#pragma unroll
        for (int e = 0; e < EPV; ++e) { g1[e] = 0.f; g2[e] = 0.f; }
        if (on) {
          Elem<T>::unpack(q1[j], g1);
          Elem<T>::unpack(q2[j], g2);
        }
        float dot = 0.f;
#pragma unroll
        for (int e = 0; e < EPV; ++e) {
          const float dy1 = g1[e] * c[e] + g2[e] * sn[e], dy2 = g2[e] * c[e] - g1[e] * sn[e];
          x1[e] *= r; x2[e] *= r;                       // xhat
          a1[e] += dy1 * x1[e]; a2[e] += dy2 * x2[e];
          g1[e] = dy1 * wv1[e]; g2[e] = dy2 * wv2[e];
          dot += g1[e] * x1[e] + g2[e] * x2[e];
        }
        dot = group_reduce<G, OpSum>(dot);
        const float cm = dot / (float)d;
        if (on) {
          float o1[EPV], o2[EPV];
#pragma unroll
          for (int e = 0; e < EPV; ++e) {
            o1[e] = (g1[e] - x1[e] * cm) * r;
            o2[e] = (g2[e] - x2[e] * cm) * r;
          }
          T* op = out + row * (int64_t)d;
          store16_stream(op + col, Elem<T>::pack(o1));
          store16_stream(op + half + col, Elem<T>::pack(o2));
        }
      }
    }
  }
  if constexpr (BWD) {
    if (partial == nullptr) return;
    // fold the rows of this workgroup in row order, then write one partial row
#pragma unroll
    for (int e = 0; e < EPV; ++e) {
      fold[(rib * 2 + 0) * G * EPV + col + e] = a1[e];
      fold[(rib * 2 + 1) * G * EPV + col + e] = a2[e];
    }
    __syncthreads();
    float* prow = partial + (int64_t)blockIdx.x * d;
    for (int j = tid; j < d; j += kBlock) {
      const int hsel = j >= half ? 1 : 0, jj = j - hsel * half;
      float acc = 0.f;
      for (int rr = 0; rr < RPB; ++rr) acc += fold[(rr * 2 + hsel) * G * EPV + jj];
      prow[j] = acc;
    }
  }
}

// Heads of four or eight 16-byte vectors (64 bf16 / fp16 elements and below). With one vector of
// each half per lane a load instruction of the kernel above touches only half of every 128-byte
// line (the halves of such a head are 64 bytes or less). Here a head is owned by G = d / EPV lanes,
// one vector per lane, so a group's load is the head's contiguous bytes; the rotation partner
// (the same columns of the other half) lives G / 2 lanes away and is fetched with lane-permute
// instructions: the packed input vector in the forward (the partner's normalised value is then
// recomputed from it and the partner's weights), the packed incoming gradient in the backward.
// Sum over the g lanes of a group that starts at lane `base` (any g: the groups of a wave need not
// be a power of two wide), in lane order; four fetches from other lanes in flight at a time.
__device__ __forceinline__ float group_sum_any(float v, int base, int g) {
  float t = 0.f;
  const int last = base + g - 1;
  for (int i = 0; i < g; i += 4) {
    const int s0 = base + i;
    float a[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) a[u] = __shfl(v, s0 + u < last ? s0 + u : last, 64);
#pragma unroll
    for (int u = 0; u < 4; ++u) t += (i + u < g) ? a[u] : 0.f;
  }
  return t;
}

template <int HG>
__device__ __forceinline__ uint32_t lane_xor(uint32_t v) {
  static_assert(HG == 2 || HG == 4, "partner two or four lanes away");
  if constexpr (HG == 2) return (uint32_t)FM_DPP_I((int)v, kDppXor2);
  // i ^ 4 inside eight lanes: mirror the eight (i -> 7 - i), then reverse each quad (quad_perm:[3,2,1,0])
  return (uint32_t)FM_DPP_I(FM_DPP_I((int)v, kDppHalfMirror), 0x1B);
}

// G = 0: the group width comes at run time (`g_any`, any even number up to 64: heads of 6, 10, 12,
// 14, 20, 24 ... vectors, head sizes 48, 80, 96, 112, 160, 192 ... in bf16). A wave then holds
// 64 / g heads, its last 64 % g lanes stay idle, the partner is fetched with ds_bpermute and the
// sums over a head run over its lanes in order.
template <typename T, typename WT, int G, bool BWD, int H>
__global__ __launch_bounds__(kBlock) void rope_pair_kernel(const T* __restrict__ x, const WT* __restrict__ w,
                                                            const float* __restrict__ cosv,
                                                            const float* __restrict__ sinv,
                                                            const T* __restrict__ dout,
                                                            float* __restrict__ rstd, T* __restrict__ out,
                                                            float* __restrict__ partial, int64_t rows,
                                                            int t_len, int heads, int d, float eps,
                                                            int64_t tiles, int g_any) {
  constexpr int EPV = Elem<T>::kVec;
  __shared__ float fold[BWD ? kBlock * EPV : 1];
  const int tid = threadIdx.x, lane = tid & 63;
  const int g = G ? G : g_any;
  const int gpw = 64 / g;                 // heads per wave
  const int RPB = (kBlock / 64) * gpw;
  const int HG = g / 2;
  const bool used = lane < gpw * g;       // (every lane when g is a power of two)
  const int rib = (tid >> 6) * gpw + (used ? lane / g : 0), l = used ? lane % g : 0;
  const int half = d / 2;                 // == HG * EPV
  const bool first = l < HG;              // this lane holds columns of the first half
  const int col = l * EPV;                // its columns inside the head
  const int hcol = (l % HG) * EPV;        // the same columns inside a half: cos / sin
  float wo[EPV], wp[BWD ? 1 : EPV], a[BWD ? EPV : 1];
  load_w_cols<T, WT>(w + col, wo);
  if constexpr (!BWD) load_w_cols<T, WT>(w + (first ? col + half : col - half), wp);
  if constexpr (BWD) {
#pragma unroll
    for (int e = 0; e < EPV; ++e) a[e] = 0.f;
  }
  for (int64_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
    // rows is a multiple of H and so is the number of heads of a token: the H rows exist
    // together and belong to one token
    // Power-of-two groups: the H rows of a group are consecutive heads of one token and share its
    // cos / sin columns (rows and the heads of a token are multiples of H there). Other widths:
    // the H rows lie RPB apart, so that each load instruction of a wave covers consecutive rows
    // (whole 128-byte lines although a row is not a whole number of them), and every row fetches
    // the columns of its own token.
    constexpr bool SHARED = G != 0;
    int64_t rowj[H];
    bool livej[H];
#pragma unroll
    for (int j = 0; j < H; ++j) {
      rowj[j] = SHARED ? (tile * RPB + rib) * H + j : (tile * H + j) * RPB + rib;
      livej[j] = used && rowj[j] < rows;
    }
    float c[EPV], sn[EPV];
    u32x4 rx[H], rg[BWD ? H : 1];
#pragma unroll
    for (int j = 0; j < H; ++j) rx[j] = u32x4{0u, 0u, 0u, 0u};
    if constexpr (BWD) {
#pragma unroll
      for (int j = 0; j < H; ++j) rg[j] = u32x4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int j = 0; j < H; ++j) {
      if (livej[j]) {
        rx[j] = load16_stream(x + rowj[j] * (int64_t)d + col);
        if constexpr (BWD) rg[j] = load16_stream(dout + rowj[j] * (int64_t)d + col);
      }
    }
    if constexpr (SHARED) {
      const int t = livej[0] ? token_of(rowj[0], heads, t_len) : 0;
      load_f32_cols<T>(cosv + (int64_t)t * half + hcol, c);
      load_f32_cols<T>(sinv + (int64_t)t * half + hcol, sn);
    }
#pragma unroll
    for (int j = 0; j < H; ++j) {
      const int64_t row = rowj[j];
      const bool live = livej[j];
      if constexpr (!SHARED) {
        const int t = live ? token_of(row, heads, t_len) : 0;
        load_f32_cols<T>(cosv + (int64_t)t * half + hcol, c);
        load_f32_cols<T>(sinv + (int64_t)t * half + hcol, sn);
      }
      float xv[EPV], o[EPV];
      Elem<T>::unpack(rx[j], xv);
      if constexpr (!BWD) {
        float ss = 0.f;
#pragma unroll
        for (int e = 0; e < EPV; ++e) ss += xv[e] * xv[e];
        if constexpr (G != 0) ss = group_reduce<(G ? G : 2), OpSum>(ss);
        else ss = group_sum_any(ss, lane - l, g);
        const float r = rsqrtf(ss / (float)d + eps);
        if (live && l == 0) rstd[row] = r;
        u32x4 pr;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          if constexpr (G != 0) pr[q] = lane_xor<(G ? G / 2 : 2)>(rx[j][q]);
          else pr[q] = (uint32_t)__shfl((int)rx[j][q], first ? lane + HG : lane - HG, 64);
        }
        float pv[EPV];
        Elem<T>::unpack(pr, pv);
#pragma unroll
        for (int e = 0; e < EPV; ++e) {
          const float y = (xv[e] * r) * wo[e], py = (pv[e] * r) * wp[e];
          // first half: y1 * cos - y2 * sin; second half: y1 * sin + y2 * cos
          o[e] = first ? y * c[e] - py * sn[e] : py * sn[e] + y * c[e];
        }
      } else {
        const float r = live ? rstd[row] : 0.f;
        u32x4 pq;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          if constexpr (G != 0) pq[q] = lane_xor<(G ? G / 2 : 2)>(rg[j][q]);
          else pq[q] = (uint32_t)__shfl((int)rg[j][q], first ? lane + HG : lane - HG, 64);
        }
        float gv[EPV], pg[EPV];
        Elem<T>::unpack(rg[j], gv);
        Elem<T>::unpack(pq, pg);
        float dot = 0.f;
#pragma unroll
        for (int e = 0; e < EPV; ++e) {
          // rotate back: dy1 = do1 * cos + do2 * sin, dy2 = do2 * cos - do1 * sin
          const float dy = first ? gv[e] * c[e] + pg[e] * sn[e] : gv[e] * c[e] - pg[e] * sn[e];
          xv[e] *= r;                                   // xhat
          a[e] += dy * xv[e];
          o[e] = dy * wo[e];
          dot += o[e] * xv[e];
        }
        if constexpr (G != 0) dot = group_reduce<(G ? G : 2), OpSum>(dot);
        else dot = group_sum_any(dot, lane - l, g);
        const float cm = dot / (float)d;
#pragma unroll
        for (int e = 0; e < EPV; ++e) o[e] = (o[e] - xv[e] * cm) * r;
      }
      if (live) store16_stream(out + row * (int64_t)d + col, Elem<T>::pack(o));
    }
  }
  if constexpr (BWD) {
    if (partial == nullptr) return;
    // fold the rows of this workgroup in row order, then write one partial row
    if (used) {
#pragma unroll
      for (int e = 0; e < EPV; ++e) fold[rib * g * EPV + col + e] = a[e];
    }
    __syncthreads();
    float* prow = partial + (int64_t)blockIdx.x * d;
    for (int j = tid; j < d; j += kBlock) {
      float acc = 0.f;
      for (int rr = 0; rr < RPB; ++rr) acc += fold[rr * g * EPV + j];
      prow[j] = acc;
    }
  }
}

struct Shape { int g; int gv; int64_t tiles; int64_t vtiles; int blocks; };

// g: lanes per head of the scalar kernel; gv: of the vector kernel (0 when the head does not
// split into 16-byte vectors per half). blocks: persistent grid, also the number of partial rows.
bool make_shape(int64_t rows, int64_t d, int esize, Shape* s) {   // esize 0: scalar variant only
  if (d < 2 || d % 2 != 0) return false;
  const int64_t half = d / 2;
  int g = 1;
  while ((int64_t)g * kEH < half) g *= 2;
  if (g > 64) return false;
  s->g = g;
  const int epv = esize > 0 ? 16 / esize : 1;
  s->gv = 0;
  if (esize > 0 && half % epv == 0) {
    int gv = 1;
    while ((int64_t)gv * epv < half) gv *= 2;
    if (gv <= 64) s->gv = gv;
  }
  s->tiles = (rows + kBlock / g - 1) / (kBlock / g);
  s->vtiles = s->gv ? (rows + kBlock / s->gv - 1) / (kBlock / s->gv) : 0;
  // 8 workgroups of 256 threads per unit; the scalar variant never has fewer tiles than the
  // vector one, so this bound holds for both and does not depend on the dtype
  int64_t blocks = (int64_t)fm_host::num_cus() * 8;
  if (blocks > s->tiles) blocks = s->tiles;
  s->blocks = (int)(blocks < 1 ? 1 : blocks);
  return true;
}

template <typename T, typename WT, bool BWD>
int launch(const Shape& sh, bool vec, const void* x, const void* w, const float* c, const float* s,
           const void* dout, float* rstd, void* out, float* partial, int64_t rows, int t_len, int heads,
           int d, float eps, hipStream_t st) {
  // heads of one token that a lane group takes per tile (vector kernel): 2 (4 in the forward is
  // slower again: fewer waves fit), 1 when the head count is odd
  int hpg = 1;
  // heads of exactly four or eight vectors: one vector per lane, partner by lane permute
  const bool pair = vec && (sh.gv == 2 || sh.gv == 4) && (int64_t)sh.gv * 2 * Elem<T>::kVec == d;
  if (vec) {
    // the one-vector-per-lane kernel: eight-lane groups take four heads forward and two backward;
    // four-lane groups one (with more, a wave's load instruction skips between 64-byte heads)
    const int want = !pair ? 2 : (sh.gv == 2 ? 1 : (BWD ? 2 : 4));
    if (want >= 4 && (!BWD || pair) && heads % 4 == 0) hpg = 4;
    else if (want >= 2 && heads % 2 == 0) hpg = 2;
  }
  // other heads of up to fourteen vectors (head sizes 48, 80, 96, 112 in bf16): the same kernel with
  // groups of exactly that many lanes. bf16 [.., 32, d], 2^27 elements, forward / backward in TB/s,
  // against the vector kernel with the next power of two of lanes: d = 48: 3.8 / 4.4 against
  // 2.0 / 2.6; 80: 3.7 / 4.4 against 3.0 / 3.6; 96: 3.9 / 4.6 against 3.9 / 4.4; 112: 3.6 / 4.3
  // against 3.3 / 3.9; wider heads (160, 192) are faster there (4.3 / 4.3 and 4.9 / 4.9).
  const int hv = vec ? (int)(d / Elem<T>::kVec) : 0;
  const int g_any = (vec && !pair && hv <= 14 && (hv & (hv - 1)) != 0) ? hv : 0;
  if (g_any) hpg = 2;
  const int rpb = g_any ? (kBlock / 64) * (64 / g_any) : kBlock / (pair ? 2 * sh.gv : (vec ? sh.gv : sh.g));
  const int64_t tiles = (rows + (int64_t)rpb * hpg - 1) / ((int64_t)rpb * hpg);
  const int64_t blocks = sh.blocks < tiles ? sh.blocks : tiles;
  int64_t used_blocks = blocks;
  // The grid is persistent: no more workgroups than the device holds at once (a kernel whose
  // registers allow seven per compute unit, launched with eight, runs the eighth after the others
  // have finished their whole share: twice the time).
#define GO_K(K, ...)                                                                                  \
  do {                                                                                                \
    static int occupancy = 0; /* workgroups of this kernel one compute unit holds, at most 8 */       \
    if (occupancy == 0) {                                                                             \
      int o = 0;                                                                                      \
      if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&o, K, kBlock, 0) != hipSuccess || o < 1) o = 8; \
      occupancy = o > 8 ? 8 : o;                                                                      \
    }                                                                                                 \
    const int64_t fit = (int64_t)fm_host::num_cus() * occupancy;                                      \
    used_blocks = blocks < fit ? blocks : fit;                                                        \
    FM_LAUNCH(K, dim3((unsigned)used_blocks), dim3(kBlock), 0, st, __VA_ARGS__);                      \
  } while (0)
#define ARGS static_cast<const T*>(x), static_cast<const WT*>(w), c, s, static_cast<const T*>(dout), rstd, \
             static_cast<T*>(out), partial, rows, t_len, heads, d, eps, tiles
#define GO_V(G)                                                                                           \
  do {                                                                                                    \
    if (hpg == 1) GO_K((rope_vec_kernel<T, WT, G, BWD, 1>), ARGS);                                          \
    else if (hpg == 2) GO_K((rope_vec_kernel<T, WT, G, BWD, 2>), ARGS);                                     \
    else if constexpr (!BWD) GO_K((rope_vec_kernel<T, WT, G, BWD, 4>), ARGS);                               \
  } while (0)
#define GO_S(G) GO_K((rope_kernel<T, WT, G, BWD>), ARGS)
#define BY_G(GO, g)           \
  switch (g) {                \
    case 1: GO(1); break;     \
    case 2: GO(2); break;     \
    case 4: GO(4); break;     \
    case 8: GO(8); break;     \
    case 16: GO(16); break;   \
    case 32: GO(32); break;   \
    default: GO(64); break;   \
  }
  if (pair || g_any) {
#define GO_P(G, H_) GO_K((rope_pair_kernel<T, WT, G, BWD, H_>), ARGS, g_any)
#define GO_PH(G)                  \
  do {                            \
    if (hpg == 4) GO_P(G, 4);     \
    else if (hpg == 2) GO_P(G, 2);\
    else GO_P(G, 1);              \
  } while (0)
    if (g_any) GO_PH(0);
    else if (sh.gv == 2) GO_PH(4);
    else GO_PH(8);
#undef GO_PH
#undef GO_P
  } else if (vec) { BY_G(GO_V, sh.gv) } else { BY_G(GO_S, sh.g) }
#undef BY_G
#undef GO_V
#undef GO_S
#undef ARGS
#undef GO_K
  return (int)used_blocks;
}

int check(const char* what, int64_t b, int64_t t, int64_t h, int64_t d, int x_dtype, int w_dtype, Shape* sh) {
  FM_CHECK_ARG(b >= 0 && t > 0 && h > 0 && d > 0, "%s: bad shape", what);
  FM_CHECK_ARG(x_dtype == FM_F32 || x_dtype == FM_F16 || x_dtype == FM_BF16, "%s: bad x_dtype %d", what, x_dtype);
  FM_CHECK_ARG(w_dtype == x_dtype || w_dtype == FM_F32, "%s: w_dtype must equal x_dtype or be fp32", what);
  if (b * t * h > 0x7fffffffLL || !make_shape(b * t * h, d, x_dtype == FM_F32 ? 4 : 2, sh)) {
    fm_host::set_error("%s: head dim must be even and <= 512, rows < 2^31 (d=%lld)", what, (long long)d);
    return FM_ERR_UNSUPPORTED;
  }
  return FM_OK;
}

}  // namespace

extern "C" {

size_t fm_qk_norm_rope_bwd_workspace(int64_t b, int64_t t, int64_t h, int64_t d) {
  Shape sh;
  if (b <= 0 || t <= 0 || h <= 0 || !make_shape(b * t * h, d, 0, &sh)) return 0;
  return (size_t)sh.blocks * (size_t)d * sizeof(float);
}

int fm_qk_norm_rope_fwd(const void* x, const void* w, const float* cosv, const float* sinv, void* out,
                        float* rstd, int64_t b, int64_t t, int64_t h, int64_t d, int x_dtype, int w_dtype,
                        float eps, fm_stream_t stream) {
  Shape sh;
  int rc = check("fm_qk_norm_rope_fwd", b, t, h, d, x_dtype, w_dtype, &sh);
  if (rc != FM_OK) return rc;
  if (b == 0) return FM_OK;
  FM_CHECK_ARG(x && w && cosv && sinv && out && rstd, "fm_qk_norm_rope_fwd: NULL pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int64_t rows = b * t * h;
  const bool vec = sh.gv != 0 && fm_host::aligned16(x) && fm_host::aligned16(out) &&
                   fm_host::aligned16(cosv) && fm_host::aligned16(sinv);
#define CALL(T, WT) launch<T, WT, false>(sh, vec, x, w, cosv, sinv, nullptr, rstd, out, nullptr, rows, (int)t, (int)h, (int)d, eps, st)
  if (x_dtype == FM_F32) CALL(float, float);
  else if (x_dtype == FM_BF16 && w_dtype == FM_BF16) CALL(bf16_t, bf16_t);
  else if (x_dtype == FM_BF16) CALL(bf16_t, float);
  else if (w_dtype == FM_F16) CALL(f16_t, f16_t);
  else CALL(f16_t, float);
#undef CALL
  FM_CHECK_LAUNCH("fm_qk_norm_rope_fwd");
  return FM_OK;
}

int fm_qk_norm_rope_bwd(const void* x, const void* w, const float* cosv, const float* sinv,
                        const float* rstd, const void* dout, void* dx, void* dw, void* workspace,
                        size_t workspace_bytes, int64_t b, int64_t t, int64_t h, int64_t d, int x_dtype,
                        int w_dtype, fm_stream_t stream) {
  Shape sh;
  int rc = check("fm_qk_norm_rope_bwd", b, t, h, d, x_dtype, w_dtype, &sh);
  if (rc != FM_OK) return rc;
  FM_CHECK_ARG(b > 0, "fm_qk_norm_rope_bwd: empty batch");
  FM_CHECK_ARG(x && w && cosv && sinv && rstd && dout && dx, "fm_qk_norm_rope_bwd: NULL pointer");
  float* partial = nullptr;
  if (dw != nullptr) {
    const size_t need = (size_t)sh.blocks * (size_t)d * sizeof(float);
    if (workspace == nullptr || workspace_bytes < need) {
      fm_host::set_error("fm_qk_norm_rope_bwd: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
      return FM_ERR_WORKSPACE;
    }
    partial = static_cast<float*>(workspace);
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int64_t rows = b * t * h;
  const bool vec = sh.gv != 0 && fm_host::aligned16(x) && fm_host::aligned16(dx) && fm_host::aligned16(dout) &&
                   fm_host::aligned16(cosv) && fm_host::aligned16(sinv);
#define CALL(T, WT)                                                                                    \
  const int used = launch<T, WT, true>(sh, vec, x, w, cosv, sinv, dout, const_cast<float*>(rstd), dx,   \
                                       partial, rows, (int)t, (int)h, (int)d, 0.f, st);                \
  if (partial != nullptr) {                                                                            \
    if (d % 4 == 0)                                                                                    \
      hipLaunchKernelGGL((colsum_kernel<WT>), dim3((unsigned)((d + 63) / 64)), dim3(1024), 0, st,       \
                         partial, static_cast<WT*>(dw), used, (int)d, (int)d, static_cast<WT*>(nullptr));                         \
    else                                                                                               \
      hipLaunchKernelGGL((colsum_scalar_kernel<WT>), dim3((unsigned)((d + 63) / 64)), dim3(1024), 0, st, \
                         partial, static_cast<WT*>(dw), used, (int)d, (int)d, static_cast<WT*>(nullptr));                         \
  }
  if (x_dtype == FM_F32) { CALL(float, float); }
  else if (x_dtype == FM_BF16 && w_dtype == FM_BF16) { CALL(bf16_t, bf16_t); }
  else if (x_dtype == FM_BF16) { CALL(bf16_t, float); }
  else if (w_dtype == FM_F16) { CALL(f16_t, f16_t); }
  else { CALL(f16_t, float); }
#undef CALL
  FM_CHECK_LAUNCH("fm_qk_norm_rope_bwd");
  return FM_OK;
}

}  // extern "C"
