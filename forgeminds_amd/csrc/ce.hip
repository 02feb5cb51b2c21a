// Vocabulary-wide cross entropy, forward and backward, for gfx950.
//
// Reference semantics: forgemind/loss.py:54-70 (sum of per-row CE over the valid rows,
// divided by max(1, n_valid); ignored rows contribute nothing and get a zero gradient).
//
// Forward: one workgroup per row, one read of the row. Each thread runs an online
// (max, sum-exp) over its share of the row in the base-2 domain, the workgroup merges
// the pairs, and lse[row] is saved. Backward: the softmax is recomputed from lse instead of
// being stored, so the whole fwd+bwd moves 2 + 2 + 2 bytes per bf16 logit. A second form
// (ce_loss_grad_kernel) produces the loss and the gradient from one read of rows that fit the
// register file: 2 + 2 bytes per logit.
#include "fm_vocab.hip.h"

using namespace fm;

namespace {

// KEEP: the rows are read with ordinary (cached) loads instead of streaming ones. The forward of a
// training step takes it for the LAST rows, as many as the memory-side cache holds: the backward,
// which follows at once and walks the rows in the same order, then finds them there when it gets to
// them (its own loads and stores stream past that cache). A load's kind cannot be chosen at run
// time -- two loads of one address that differ only in their cache hint are merged into a plain
// one -- so the two kinds are two instantiations, launched over two row ranges (`row0`).
template <typename T, int THREADS, int UNROLL, bool KEEP>
__global__ __launch_bounds__(THREADS) void ce_fwd_kernel(const T* __restrict__ logits,
                                                          const int64_t* __restrict__ labels,
                                                          float* __restrict__ lse,
                                                          float* __restrict__ row_loss, int v,
                                                          int64_t ignore_index, bool vec_ok, int64_t row0) {
  constexpr int EPV = Elem<T>::kVec;
  constexpr int NW = THREADS / 64;
  __shared__ float smem[2 * NW];
  const int64_t row = row0 + blockIdx.x;
  const T* rp = logits + row * (int64_t)v;
  const RowSplit sp = split_row<EPV>(row, v, vec_ok);
  const int tid = threadIdx.x;

  // the label and its logit are fetched first, so the two dependent loads overlap the
  // streaming pass instead of trailing it
  int64_t y = 0;
  float ylogit = 0.f;
  if (tid == 0) {
    y = labels[row];
    if (y != ignore_index && y >= 0 && y < v) ylogit = Elem<T>::load1(rp + y);
  }

  MaxSum st{kNegBig, 0.f};
  for (int c0 = 0; c0 < sp.nvec; c0 += THREADS * UNROLL) {
    u32x4 raw[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int c = clamp_col(c0 + u * THREADS + tid, sp.nvec);
      raw[u] = KEEP ? load16(rp + sp.head + (int64_t)c * EPV) : load16_stream(rp + sp.head + (int64_t)c * EPV);
    }
    // the maximum is taken on the raw logits and scaled once per batch, so each element costs
    // one max, one fma and one exp2
    float z[UNROLL][EPV];
    float raw_max = -INFINITY;
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int c = c0 + u * THREADS + tid;
      if (c < sp.nvec) {
        Elem<T>::unpack(raw[u], z[u]);
#pragma unroll
        for (int e = 0; e < EPV; ++e) raw_max = fmaxf(raw_max, z[u][e]);
      } else {
#pragma unroll
        for (int e = 0; e < EPV; ++e) z[u][e] = -INFINITY;
      }
    }
    const float cm = fmaxf(st.m, raw_max * kLog2e);   // st.m is finite, so cm is
    float acc = st.s * fast_exp2(st.m - cm);
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
#pragma unroll
      for (int e = 0; e < EPV; ++e) acc += fast_exp2(__builtin_fmaf(z[u][e], kLog2e, -cm));
    }
    st.m = cm;
    st.s = acc;
  }
  const int ne = edge_count(sp, v);
  for (int e = tid; e < ne; e += THREADS) {
    const float z = Elem<T>::load1(rp + edge_col(sp, e)) * kLog2e;
    const float cm = fmaxf(st.m, z);
    st.s = st.s * fast_exp2(st.m - cm) + fast_exp2(z - cm);
    st.m = cm;
  }
  const MaxSum tot = block_merge<NW>(st, smem);
  if (tid == 0) {
    const float l = (tot.m + fast_log2(tot.s)) * kLn2;
    if (lse != nullptr) lse[row] = l;
    float loss = 0.f;
    if (y != ignore_index) loss = (y >= 0 && y < v) ? l - ylogit : __builtin_nanf("");
    row_loss[row] = loss;
  }
}

// loss = sum(row_loss) [/ max(1, n_valid)] in a fixed order: thread i adds rows i, i+1024, ...,
// then lanes and waves are combined in index order.
__global__ __launch_bounds__(1024) void ce_finalize_kernel(const float* __restrict__ row_loss,
                                                           const int64_t* __restrict__ labels,
                                                           int64_t n, int64_t ignore_index,
                                                           int mean, float* __restrict__ loss,
                                                           float* __restrict__ n_valid) {
  __shared__ float sf[16];
  __shared__ int si[16];
  float a = 0.f;
  int cnt = 0;
  // eight rows' loads in flight per thread; the additions keep the order stated above
  int64_t i = threadIdx.x;
  for (; i + 7 * 1024 < n; i += 8 * 1024) {
    float r[8];
    int64_t l[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) { r[u] = row_loss[i + u * 1024]; l[u] = labels[i + u * 1024]; }
#pragma unroll
    for (int u = 0; u < 8; ++u) { a += r[u]; cnt += l[u] != ignore_index ? 1 : 0; }
  }
  for (; i < n; i += 1024) {
    a += row_loss[i];
    cnt += labels[i] != ignore_index ? 1 : 0;
  }
  a = wave_sum(a);
  cnt = wave_sum_i(cnt);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) { sf[wave] = a; si[wave] = cnt; }
  __syncthreads();
  if (threadIdx.x == 0) {
    float t = sf[0];
    int c = si[0];
    for (int i = 1; i < 16; ++i) { t += sf[i]; c += si[i]; }
    const float nv = c > 0 ? (float)c : 1.f;
    *n_valid = nv;
    *loss = mean ? t / nv : t;
  }
}

template <typename T, int THREADS, int UNROLL>
__global__ __launch_bounds__(THREADS) void ce_bwd_kernel(const T* __restrict__ logits,
                                                          const int64_t* __restrict__ labels,
                                                          const float* __restrict__ lse,
                                                          const float* __restrict__ n_valid,
                                                          const float* __restrict__ grad_out,
                                                          T* __restrict__ dlogits, int v,
                                                          int64_t ignore_index, bool vec_ok, int chunks) {
  constexpr int EPV = Elem<T>::kVec;
  // chunks > 1: a workgroup takes one tile of THREADS * UNROLL vectors of a row, not the whole row
  // (the backward needs nothing from the rest of the row but the saved log-sum-exp)
  const int64_t row = chunks > 1 ? (int64_t)(blockIdx.x / (unsigned)chunks) : (int64_t)blockIdx.x;
  const int chunk = chunks > 1 ? (int)(blockIdx.x % (unsigned)chunks) : 0;
  const T* rp = logits + row * (int64_t)v;
  T* gp = dlogits + row * (int64_t)v;
  const RowSplit sp = split_row<EPV>(row, v, vec_ok);
  const int tid = threadIdx.x;
  const int64_t y64 = labels[row];
  const int ne = chunk == 0 ? edge_count(sp, v) : 0;   // the row's unaligned ends go with its first tile
  const int c_begin = chunks > 1 ? chunk * THREADS * UNROLL : 0;
  const int c_end = chunks > 1 ? (c_begin + THREADS * UNROLL < sp.nvec ? c_begin + THREADS * UNROLL : sp.nvec) : sp.nvec;

  if (y64 == ignore_index) {  // ignored row: zeros, and the logits are never read
    const u32x4 zero = {0u, 0u, 0u, 0u};
    for (int c = c_begin + tid; c < c_end; c += THREADS) store16_stream(gp + sp.head + (int64_t)c * EPV, zero);
    for (int e = tid; e < ne; e += THREADS) Elem<T>::store1(gp + edge_col(sp, e), 0.f);
    return;
  }
  const int y = (y64 >= 0 && y64 < v) ? (int)y64 : -1;
  const float scale = (grad_out != nullptr ? *grad_out : 1.f) / (n_valid != nullptr ? *n_valid : 1.f);
  const float l2 = lse[row] * kLog2e;

  for (int c0 = c_begin; c0 < c_end; c0 += THREADS * UNROLL) {
    u32x4 raw[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int c = clamp_col(c0 + u * THREADS + tid, sp.nvec);
      raw[u] = load16_stream(rp + sp.head + (int64_t)c * EPV);
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int c = c0 + u * THREADS + tid;
      touch(raw[u]);
      if (c < sp.nvec) {
        float z[EPV], o[EPV];
        Elem<T>::unpack(raw[u], z);
        const int col0 = sp.head + c * EPV;
#pragma unroll
        for (int e = 0; e < EPV; ++e) o[e] = fast_exp2(z[e] * kLog2e - l2);
        if (y >= col0 && y < col0 + EPV) {   // the one vector of the row that holds the label
#pragma unroll
          for (int e = 0; e < EPV; ++e) o[e] -= (col0 + e == y) ? 1.f : 0.f;
        }
#pragma unroll
        for (int e = 0; e < EPV; ++e) o[e] *= scale;
        store16_stream(gp + col0, Elem<T>::pack(o));
      }
    }
  }
  for (int e = tid; e < ne; e += THREADS) {
    const int col = edge_col(sp, e);
    float p = fast_exp2(Elem<T>::load1(rp + col) * kLog2e - l2);
    if (col == y) p -= 1.f;
    Elem<T>::store1(gp + col, p * scale);
  }
}

// Rows too wide for registers (or unaligned buffers), loss and gradient in ONE launch: the
// streaming log-sum-exp, the workgroup merge, then a second sweep over the same row that writes
// the gradient. The second sweep follows the first at once, so a cache that still holds the
// row serves it (the first sweep uses ordinary loads for that reason). dlogits may be the logits buffer itself:
// every element is re-read by the thread that writes it.
template <typename T, int THREADS, int UNROLL>
__global__ __launch_bounds__(THREADS) void ce_loss_grad_wide_kernel(const T* logits,
                                                                     const int64_t* __restrict__ labels,
                                                                     const float* __restrict__ n_valid,
                                                                     float* __restrict__ lse,
                                                                     float* __restrict__ row_loss,
                                                                     T* dlogits, int v,
                                                                     int64_t ignore_index, bool vec_ok) {
  constexpr int EPV = Elem<T>::kVec;
  constexpr int NW = THREADS / 64;
  __shared__ float smem[2 * NW];
  const int64_t row = blockIdx.x;
  const T* rp = logits + row * (int64_t)v;
  T* gp = dlogits + row * (int64_t)v;
  const RowSplit sp = split_row<EPV>(row, v, vec_ok);
  const int tid = threadIdx.x;
  const int ne = edge_count(sp, v);
  const int64_t y64 = labels[row];

  if (y64 == ignore_index) {  // ignored row: zeros, and the logits are never read
    const u32x4 zero = {0u, 0u, 0u, 0u};
    for (int c = tid; c < sp.nvec; c += THREADS) store16_stream(gp + sp.head + (int64_t)c * EPV, zero);
    for (int e = tid; e < ne; e += THREADS) Elem<T>::store1(gp + edge_col(sp, e), 0.f);
    if (tid == 0) {
      row_loss[row] = 0.f;
      if (lse != nullptr) lse[row] = 0.f;
    }
    return;
  }
  const int y = (y64 >= 0 && y64 < v) ? (int)y64 : -1;
  float ylogit = 0.f;
  if (tid == 0 && y >= 0) ylogit = Elem<T>::load1(rp + y);

  MaxSum st{kNegBig, 0.f};
  for (int c0 = 0; c0 < sp.nvec; c0 += THREADS * UNROLL) {
    u32x4 raw[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int c = clamp_col(c0 + u * THREADS + tid, sp.nvec);
      raw[u] = load16(rp + sp.head + (int64_t)c * EPV);
    }
    float z[UNROLL][EPV];
    float raw_max = -INFINITY;
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int c = c0 + u * THREADS + tid;
      if (c < sp.nvec) {
        Elem<T>::unpack(raw[u], z[u]);
#pragma unroll
        for (int e = 0; e < EPV; ++e) raw_max = fmaxf(raw_max, z[u][e]);
      } else {
#pragma unroll
        for (int e = 0; e < EPV; ++e) z[u][e] = -INFINITY;
      }
    }
    const float cm = fmaxf(st.m, raw_max * kLog2e);
    float acc = st.s * fast_exp2(st.m - cm);
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
#pragma unroll
      for (int e = 0; e < EPV; ++e) acc += fast_exp2(__builtin_fmaf(z[u][e], kLog2e, -cm));
    }
    st.m = cm;
    st.s = acc;
  }
  for (int e = tid; e < ne; e += THREADS) {
    const float z = Elem<T>::load1(rp + edge_col(sp, e)) * kLog2e;
    const float cm = fmaxf(st.m, z);
    st.s = st.s * fast_exp2(st.m - cm) + fast_exp2(z - cm);
    st.m = cm;
  }
  const MaxSum tot = block_merge<NW>(st, smem);
  const float l2 = tot.m + fast_log2(tot.s);
  const float scale = 1.f / (n_valid != nullptr ? *n_valid : 1.f);
  if (tid == 0) {
    const float l = l2 * kLn2;
    if (lse != nullptr) lse[row] = l;
    row_loss[row] = y >= 0 ? l - ylogit : __builtin_nanf("");
  }
  for (int c0 = 0; c0 < sp.nvec; c0 += THREADS * UNROLL) {
    u32x4 raw[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int c = clamp_col(c0 + u * THREADS + tid, sp.nvec);
      raw[u] = load16_stream(rp + sp.head + (int64_t)c * EPV);
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int c = c0 + u * THREADS + tid;
      touch(raw[u]);
      if (c < sp.nvec) {
        float z[EPV], o[EPV];
        Elem<T>::unpack(raw[u], z);
        const int col0 = sp.head + c * EPV;
#pragma unroll
        for (int e = 0; e < EPV; ++e) o[e] = fast_exp2(z[e] * kLog2e - l2);
        if (y >= col0 && y < col0 + EPV) {   // the one vector of the row that holds the label
#pragma unroll
          for (int e = 0; e < EPV; ++e) o[e] -= (col0 + e == y) ? 1.f : 0.f;
        }
#pragma unroll
        for (int e = 0; e < EPV; ++e) o[e] *= scale;
        store16_stream(gp + col0, Elem<T>::pack(o));
      }
    }
  }
  for (int e = tid; e < ne; e += THREADS) {
    const int col = edge_col(sp, e);
    float p = fast_exp2(Elem<T>::load1(rp + col) * kLog2e - l2);
    if (col == y) p -= 1.f;
    Elem<T>::store1(gp + col, p * scale);
  }
}

// Number of rows whose label is not ignore_index, as the float the gradient is divided by
// (at least 1). One workgroup; runs ahead of ce_loss_grad_kernel, which needs the count.
__global__ __launch_bounds__(1024) void ce_count_kernel(const int64_t* __restrict__ labels, int64_t n,
                                                        int64_t ignore_index,
                                                        float* __restrict__ n_valid) {
  __shared__ int si[16];
  int cnt = 0;
  int64_t i = threadIdx.x;
  for (; i + 7 * 1024 < n; i += 8 * 1024) {
    int64_t l[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) l[u] = labels[i + u * 1024];
#pragma unroll
    for (int u = 0; u < 8; ++u) cnt += l[u] != ignore_index ? 1 : 0;
  }
  for (; i < n; i += 1024) cnt += labels[i] != ignore_index ? 1 : 0;
  cnt = wave_sum_i(cnt);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) si[wave] = cnt;
  __syncthreads();
  if (threadIdx.x == 0) {
    int c = si[0];
    for (int i = 1; i < 16; ++i) c += si[i];
    *n_valid = c > 0 ? (float)c : 1.f;
  }
}

// Loss and gradient from ONE read of the logits: the row stays in registers (ITERS 16-byte
// vectors per thread) between the log-sum-exp and the gradient store, so the whole
// forward + backward of a training step moves 2 + 2 bytes per bf16 logit instead of 2 + 2 + 2.
// dlogits may be the logits buffer itself: every element is read by the thread that later
// writes it. The gradient is (softmax - onehot) * scale, scale = 1 / n_valid for the mean.
template <typename T, int THREADS, int ITERS>
__global__ __launch_bounds__(THREADS) void ce_loss_grad_kernel(const T* logits,
                                                                const int64_t* __restrict__ labels,
                                                                const float* __restrict__ n_valid,
                                                                float* __restrict__ lse,
                                                                float* __restrict__ row_loss,
                                                                T* dlogits, int v,
                                                                int64_t ignore_index) {
  constexpr int EPV = Elem<T>::kVec;
  constexpr int NW = THREADS / 64;
  __shared__ float smem[2 * NW];
  const int64_t row = blockIdx.x;
  const T* rp = logits + row * (int64_t)v;
  T* gp = dlogits + row * (int64_t)v;
  const RowSplit sp = split_row<EPV>(row, v, true);
  const int tid = threadIdx.x;
  const int ne = edge_count(sp, v);
  const int64_t y64 = labels[row];

  if (y64 == ignore_index) {  // ignored row: zeros, and the logits are never read
    const u32x4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      const int c = i * THREADS + tid;
      if (c < sp.nvec) store16_stream(gp + sp.head + (int64_t)c * EPV, zero);
    }
    for (int e = tid; e < ne; e += THREADS) Elem<T>::store1(gp + edge_col(sp, e), 0.f);
    if (tid == 0) {
      row_loss[row] = 0.f;
      if (lse != nullptr) lse[row] = 0.f;
    }
    return;
  }
  const int y = (y64 >= 0 && y64 < v) ? (int)y64 : -1;
  float ylogit = 0.f;
  if (tid == 0 && y >= 0) ylogit = Elem<T>::load1(rp + y);   // early: overlaps the row loads

  u32x4 raw[ITERS];
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
    const int c = i * THREADS + tid;
    if (c < sp.nvec) raw[i] = load16_stream(rp + sp.head + (int64_t)c * EPV);
  }
  // the unaligned ends of the row (at most EPV - 1 elements each): thread e keeps edge e
  float edge = -INFINITY;
  int edge_at = -1;
  if (tid < ne) {
    edge_at = edge_col(sp, tid);
    edge = Elem<T>::load1(rp + edge_at) * kLog2e;
  }
  // maximum first, then the sum: the data sits in registers, a second sweep costs no traffic
  float mz = fmaxf(edge, kNegBig);
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
    const int c = i * THREADS + tid;
    if (c < sp.nvec) {
      float z[EPV];
      Elem<T>::unpack(raw[i], z);
#pragma unroll
      for (int e = 0; e < EPV; ++e) mz = fmaxf(mz, z[e] * kLog2e);
    }
  }
  float ssum = edge_at >= 0 ? fast_exp2(edge - mz) : 0.f;
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
    const int c = i * THREADS + tid;
    if (c < sp.nvec) {
      float z[EPV];
      Elem<T>::unpack(raw[i], z);
#pragma unroll
      for (int e = 0; e < EPV; ++e) ssum += fast_exp2(z[e] * kLog2e - mz);
    }
  }
  const MaxSum tot = block_merge<NW>(MaxSum{mz, ssum}, smem);
  const float l2 = tot.m + fast_log2(tot.s);
  const float scale = 1.f / (n_valid != nullptr ? *n_valid : 1.f);
  if (tid == 0) {
    const float l = l2 * kLn2;
    if (lse != nullptr) lse[row] = l;
    row_loss[row] = y >= 0 ? l - ylogit : __builtin_nanf("");
  }
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
    const int c = i * THREADS + tid;
    if (c < sp.nvec) {
      float z[EPV], o[EPV];
      Elem<T>::unpack(raw[i], z);
      const int col0 = sp.head + c * EPV;
#pragma unroll
      for (int e = 0; e < EPV; ++e) o[e] = fast_exp2(z[e] * kLog2e - l2);
      if (y >= col0 && y < col0 + EPV) {
#pragma unroll
        for (int e = 0; e < EPV; ++e) o[e] -= (col0 + e == y) ? 1.f : 0.f;
      }
#pragma unroll
      for (int e = 0; e < EPV; ++e) o[e] *= scale;
      store16_stream(gp + col0, Elem<T>::pack(o));
    }
  }
  if (edge_at >= 0) {
    float p = fast_exp2(edge - l2);
    if (edge_at == y) p -= 1.f;
    Elem<T>::store1(gp + edge_at, p * scale);
  }
}

// The same for rows past eight vectors a thread that still fit the CHIP: a 1024-thread workgroup, one
// per compute unit, keeps 16 vectors a thread in registers and 8 more in 128 KB of LDS (filled straight
// from memory, every thread fetches its own slots only: no barrier for them): 24576 vectors, 196608 bf16 columns, the
// vocabularies of 100 K to 152 K entries among them. One read and one write of the row, where the two
// sweeps of ce_loss_grad_wide_kernel read it twice. What a row has beyond the 24576 vectors is streamed
// and read again (taken up to twice that width).
constexpr int kCeHeldThreads = 1024;
constexpr int kCeHeldRegs = 16;
constexpr int kCeHeldLds = 8;
constexpr int kCeHeldMaxVec = kCeHeldThreads * (kCeHeldRegs + kCeHeldLds);
template <typename T>
__global__ __launch_bounds__(kCeHeldThreads) void ce_loss_grad_held_kernel(const T* logits,
                                                                            const int64_t* __restrict__ labels,
                                                                            const float* __restrict__ n_valid,
                                                                            float* __restrict__ lse,
                                                                            float* __restrict__ row_loss,
                                                                            T* dlogits, int v,
                                                                            int64_t ignore_index) {
  constexpr int EPV = Elem<T>::kVec;
  constexpr int THREADS = kCeHeldThreads, RI = kCeHeldRegs, LI = kCeHeldLds;
  constexpr int NW = THREADS / 64;
  extern __shared__ u32x4 parked[];          // [LI][THREADS]
  __shared__ float smem[2 * NW];
  const int64_t row = blockIdx.x;
  const T* rp = logits + row * (int64_t)v;
  T* gp = dlogits + row * (int64_t)v;
  const RowSplit sp = split_row<EPV>(row, v, true);
  const int tid = threadIdx.x;
  const int ne = edge_count(sp, v);
  const int64_t y64 = labels[row];

  if (y64 == ignore_index) {  // ignored row: zeros, and the logits are never read
    const u32x4 zero = {0u, 0u, 0u, 0u};
    for (int c = tid; c < sp.nvec; c += THREADS) store16_stream(gp + sp.head + (int64_t)c * EPV, zero);
    for (int e = tid; e < ne; e += THREADS) Elem<T>::store1(gp + edge_col(sp, e), 0.f);
    if (tid == 0) {
      row_loss[row] = 0.f;
      if (lse != nullptr) lse[row] = 0.f;
    }
    return;
  }
  const int y = (y64 >= 0 && y64 < v) ? (int)y64 : -1;
  float ylogit = 0.f;
  if (tid == 0 && y >= 0) ylogit = Elem<T>::load1(rp + y);   // early: overlaps the row loads

  // the row's unaligned ends first (at most EPV - 1 elements each, thread e keeps edge e): a wait
  // for them then waits for nothing that was issued behind them
  float edge = -INFINITY;
  int edge_at = -1;
  if (tid < ne) {
    edge_at = edge_col(sp, tid);
    edge = Elem<T>::load1(rp + edge_at) * kLog2e;
  }
  // every register load of the thread is issued before the first is used (clamped columns: no load
  // sits behind a branch)
  u32x4 raw[RI];
#pragma unroll
  for (int i = 0; i < RI; ++i)
    raw[i] = load16_stream(rp + sp.head + (int64_t)clamp_col(i * THREADS + tid, sp.nvec) * EPV);
  // Running (maximum, sum), one vector at a time IN THE ORDER THE LOADS WERE ISSUED: the wait before
  // vector i counts the loads issued after it, so the arithmetic on the first vectors runs while
  // the later ones are still on their way. The loads into LDS are issued only behind that: while
  // one of them is outstanding the compiler waits for ALL vector-memory operations wherever it
  // has to wait for one (it takes loads into registers and into LDS to complete in any order),
  // which would hold the first vector back until the last has arrived ([4096,128256] bf16: 424 us
  // with the LDS share requested up front, 391 us this way, 428 us with a maximum pass and a sum
  // pass over data that had all been waited for).
  MaxSum run{fmaxf(edge, kNegBig), 0.f};
  if (edge_at >= 0) run.s = fast_exp2(edge - run.m);
  auto fold = [&](const u32x4& r) {
    float z[EPV];
    Elem<T>::unpack(r, z);
    float cm = run.m;
#pragma unroll
    for (int e = 0; e < EPV; ++e) { z[e] *= kLog2e; cm = fmaxf(cm, z[e]); }
    float acc = run.s * fast_exp2(run.m - cm);
#pragma unroll
    for (int e = 0; e < EPV; ++e) acc += fast_exp2(z[e] - cm);
    run.m = cm;
    run.s = acc;
  };
#pragma unroll
  for (int i = 0; i < RI; ++i) {
    if (i * THREADS + tid < sp.nvec) fold(raw[i]);
  }
  {
    const int wave_first = __builtin_amdgcn_readfirstlane(tid & ~63);
#pragma unroll
    for (int j = 0; j < LI; ++j)
      load16_stream_to_lds(rp + sp.head + (int64_t)clamp_col((RI + j) * THREADS + tid, sp.nvec) * EPV,
                           parked + j * THREADS + wave_first);
  }
  wait_vmem_all();   // those loads name no register the compiler could wait on
#pragma unroll
  for (int j = 0; j < LI; ++j) {
    if ((RI + j) * THREADS + tid < sp.nvec) fold(parked[j * THREADS + tid]);
  }
  // vectors past what the chip holds: streamed into the same running pair, read again below
  for (int c0 = kCeHeldMaxVec; c0 < sp.nvec; c0 += THREADS * 2) {
    u32x4 more[2];
#pragma unroll
    for (int u = 0; u < 2; ++u)
      more[u] = load16(rp + sp.head + (int64_t)clamp_col(c0 + u * THREADS + tid, sp.nvec) * EPV);
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      touch(more[u]);
      if (c0 + u * THREADS + tid < sp.nvec) {
        float z[EPV];
        Elem<T>::unpack(more[u], z);
        float cm = run.m;
#pragma unroll
        for (int e = 0; e < EPV; ++e) { z[e] *= kLog2e; cm = fmaxf(cm, z[e]); }
        float acc = run.s * fast_exp2(run.m - cm);
#pragma unroll
        for (int e = 0; e < EPV; ++e) acc += fast_exp2(z[e] - cm);
        run.m = cm;
        run.s = acc;
      }
    }
  }
  const MaxSum tot = block_merge<NW>(run, smem);
  const float l2 = tot.m + fast_log2(tot.s);
  const float scale = 1.f / (n_valid != nullptr ? *n_valid : 1.f);
  if (tid == 0) {
    const float l = l2 * kLn2;
    if (lse != nullptr) lse[row] = l;
    row_loss[row] = y >= 0 ? l - ylogit : __builtin_nanf("");
  }
#pragma unroll
  for (int i = 0; i < RI + LI; ++i) {
    const int c = i * THREADS + tid;
    if (c < sp.nvec) {
      u32x4 r;
      if (i < RI) { touch_whole(raw[i < RI ? i : 0]); r = raw[i < RI ? i : 0]; }
      else r = parked[(i - RI) * THREADS + tid];
      float z[EPV], o[EPV];
      Elem<T>::unpack(r, z);
      const int col0 = sp.head + c * EPV;
#pragma unroll
      for (int e = 0; e < EPV; ++e) o[e] = fast_exp2(z[e] * kLog2e - l2);
      if (y >= col0 && y < col0 + EPV) {
#pragma unroll
        for (int e = 0; e < EPV; ++e) o[e] -= (col0 + e == y) ? 1.f : 0.f;
      }
#pragma unroll
      for (int e = 0; e < EPV; ++e) o[e] *= scale;
      store16_stream(gp + col0, Elem<T>::pack(o));
    }
  }
  for (int c0 = kCeHeldMaxVec; c0 < sp.nvec; c0 += THREADS * 2) {
    u32x4 more[2];
#pragma unroll
    for (int u = 0; u < 2; ++u)
      more[u] = load16_stream(rp + sp.head + (int64_t)clamp_col(c0 + u * THREADS + tid, sp.nvec) * EPV);
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int c = c0 + u * THREADS + tid;
      touch(more[u]);
      if (c < sp.nvec) {
        float z[EPV], o[EPV];
        Elem<T>::unpack(more[u], z);
        const int col0 = sp.head + c * EPV;
#pragma unroll
        for (int e = 0; e < EPV; ++e) o[e] = fast_exp2(z[e] * kLog2e - l2);
        if (y >= col0 && y < col0 + EPV) {
#pragma unroll
          for (int e = 0; e < EPV; ++e) o[e] -= (col0 + e == y) ? 1.f : 0.f;
        }
#pragma unroll
        for (int e = 0; e < EPV; ++e) o[e] *= scale;
        store16_stream(gp + col0, Elem<T>::pack(o));
      }
    }
  }
  if (edge_at >= 0) {
    float p = fast_exp2(edge - l2);
    if (edge_at == y) p -= 1.f;
    Elem<T>::store1(gp + edge_at, p * scale);
  }
}

// x *= *factor in place, skipped altogether when the factor is exactly 1 (the usual upstream
// gradient of a loss): the gradient written by ce_loss_grad_kernel then costs no second pass.
template <typename T>
__global__ __launch_bounds__(1024) void scale_inplace_kernel(T* x, const float* __restrict__ factor,
                                                             int64_t count, bool vec_ok) {
  constexpr int EPV = Elem<T>::kVec;
  const float f = *factor;
  if (f == 1.f) return;
  const int64_t nvec = vec_ok ? count / EPV : 0;
  const int64_t stride = (int64_t)gridDim.x * 1024;
  for (int64_t c = (int64_t)blockIdx.x * 1024 + threadIdx.x; c < nvec; c += stride) {
    float z[EPV];
    Elem<T>::unpack(load16_stream(x + c * EPV), z);
#pragma unroll
    for (int e = 0; e < EPV; ++e) z[e] *= f;
    store16_stream(x + c * EPV, Elem<T>::pack(z));
  }
  for (int64_t i = nvec * EPV + (int64_t)blockIdx.x * 1024 + threadIdx.x; i < count; i += stride)
    Elem<T>::store1(x + i, Elem<T>::load1(x + i) * f);
}

// Narrow rows (up to 1024 logits, e.g. classification heads): a row is owned by TPR lanes of a
// wave, each holding ITERS elements (t, t + TPR, ...), several rows per workgroup. LOSS writes
// lse / row_loss, GRAD writes (softmax - onehot) * scale with scale = grad_out / n_valid (each
// NULL pointer counts as 1). Any alignment, one element per load.
template <typename T, int TPR, int ITERS, bool LOSS, bool GRAD>
__global__ __launch_bounds__(256) void ce_rows_kernel(const T* logits, const int64_t* __restrict__ labels,
                                                      const float* __restrict__ n_valid,
                                                      const float* __restrict__ grad_out,
                                                      float* __restrict__ lse, float* __restrict__ row_loss,
                                                      T* dlogits, int64_t n, int v, int64_t ignore_index) {
  constexpr int RPB = 256 / TPR;
  const int tid = threadIdx.x;
  const int rib = tid / TPR;
  const int t = tid % TPR;
  const int64_t row = (int64_t)blockIdx.x * RPB + rib;
  const bool valid = row < n;
  const int64_t base = row * (int64_t)v;
  const int64_t y64 = valid ? labels[row] : ignore_index;
  const bool ignored = y64 == ignore_index;
  const int y = (y64 >= 0 && y64 < v) ? (int)y64 : -1;
  float z[ITERS];
  float m = kNegBig;
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
    const int c = i * TPR + t;
    // an ignored row of the gradient-only form is not read at all
    z[i] = (valid && c < v && (LOSS || !ignored)) ? Elem<T>::load1(logits + base + c) * kLog2e : -INFINITY;
    m = fmaxf(m, z[i]);
  }
  m = group_reduce<TPR, OpMax>(m);
  float ssum = 0.f;
  float ylogit2 = 0.f;          // the label's logit (times log2 e), found among the lane's elements
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
    if (i * TPR + t == y) ylogit2 = z[i];
    z[i] = fast_exp2(z[i] - m);
    ssum += z[i];
  }
  ssum = group_reduce<TPR, OpSum>(ssum);
  const float l2 = m + fast_log2(ssum);
  if constexpr (LOSS) {
    ylogit2 = group_reduce<TPR, OpSum>(ylogit2);     // one lane holds it, the others add 0
    if (valid && t == 0) {
      const float l = l2 * kLn2;
      if (lse != nullptr) lse[row] = l;
      row_loss[row] = ignored ? 0.f : (y >= 0 ? l - ylogit2 * kLn2 : __builtin_nanf(""));
    }
  }
  if constexpr (GRAD) {
    const float scale = (grad_out != nullptr ? *grad_out : 1.f) / (n_valid != nullptr ? *n_valid : 1.f);
    const float inv = 1.f / ssum;
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      const int c = i * TPR + t;
      if (valid && c < v) {
        float p = ignored ? 0.f : z[i] * inv;
        if (c == y && !ignored) p -= 1.f;
        Elem<T>::store1(dlogits + base + c, ignored ? 0.f : p * scale);
      }
    }
  }
}

// The same lane groups with 16-byte accesses, for rows that are a whole number of aligned
// vectors: lane t of a row's TPR lanes holds vectors t, t + TPR, ... packed, and unpacks them
// once per pass (maximum, sum, gradient). The gradient may overwrite the logits: the label's
// logit is taken from the registers, and a lane stores only what it loaded.
template <typename T, int TPR, int ITERS, bool LOSS, bool GRAD>
__global__ __launch_bounds__(256) void ce_vrows_kernel(const T* logits, const int64_t* __restrict__ labels,
                                                       const float* __restrict__ n_valid,
                                                       const float* __restrict__ grad_out,
                                                       float* __restrict__ lse, float* __restrict__ row_loss,
                                                       T* dlogits, int64_t n, int v, int64_t ignore_index) {
  constexpr int EPV = Elem<T>::kVec;
  constexpr int RPB = 256 / TPR;
  const int tid = threadIdx.x;
  const int rib = tid / TPR;
  const int t = tid % TPR;
  const int64_t row = (int64_t)blockIdx.x * RPB + rib;
  const bool valid = row < n;
  const int64_t base = row * (int64_t)v;
  const int nvec = v / EPV;
  const int64_t y64 = valid ? labels[row] : ignore_index;
  const bool ignored = y64 == ignore_index;
  const int y = (y64 >= 0 && y64 < v) ? (int)y64 : -1;
  // an ignored row of the gradient-only form is not read at all
  const bool read = valid && (LOSS || !ignored);
  u32x4 r[ITERS];
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
    const int c = i * TPR + t;
    if (read && c < nvec) r[i] = load16_stream(logits + base + (int64_t)c * EPV);
  }
  float m = kNegBig;
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
    if (read && i * TPR + t < nvec) {
      float f[EPV];
      unpack_again<T, (ITERS >= 8)>(r[i], f);
#pragma unroll
      for (int e = 0; e < EPV; ++e) m = fmaxf(m, f[e] * kLog2e);
    }
  }
  m = group_reduce<TPR, OpMax>(m);
  // a NaN anywhere must reach the whole row: fmaxf drops it, so it is carried in the sum
  float ssum = 0.f;
  float ylogit2 = 0.f;          // the label's logit (times log2 e), found among the lane's elements
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
    const int c = i * TPR + t;
    if (read && c < nvec) {
      float f[EPV];
      unpack_again<T, (ITERS >= 8)>(r[i], f);
#pragma unroll
      for (int e = 0; e < EPV; ++e) {
        const float z = f[e] * kLog2e;
        if (LOSS && c * EPV + e == y) ylogit2 = z;
        ssum += fast_exp2(z - m);
      }
    }
  }
  ssum = group_reduce<TPR, OpSum>(ssum);
  const float l2 = m + fast_log2(ssum);
  if constexpr (LOSS) {
    ylogit2 = group_reduce<TPR, OpSum>(ylogit2);     // one lane holds it, the others add 0
    if (valid && t == 0) {
      const float l = l2 * kLn2;
      if (lse != nullptr) lse[row] = l;
      row_loss[row] = ignored ? 0.f : (y >= 0 ? l - ylogit2 * kLn2 : __builtin_nanf(""));
    }
  }
  if constexpr (GRAD) {
    const float scale = (grad_out != nullptr ? *grad_out : 1.f) / (n_valid != nullptr ? *n_valid : 1.f);
    const float inv = 1.f / ssum;
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      const int c = i * TPR + t;
      if (valid && c < nvec) {
        float f[EPV], o[EPV];
        if (!ignored) unpack_again<T, (ITERS >= 8)>(r[i], f);
#pragma unroll
        for (int e = 0; e < EPV; ++e) {
          float p = ignored ? 0.f : fast_exp2(f[e] * kLog2e - m) * inv;
          if (c * EPV + e == y && !ignored) p -= 1.f;
          o[e] = ignored ? 0.f : p * scale;
        }
        store16_stream(dlogits + base + (int64_t)c * EPV, Elem<T>::pack(o));
      }
    }
  }
}

// Widest row, in 16-byte vectors, of the vector lane-group kernel (the forward alone takes twice
// the width of the forms that write a gradient).
constexpr int kVRowsMaxVec = 512;

bool vrows_fits(int v, int esize, bool bf16, const void* logits, const void* dlogits, bool loss, bool grad) {
  const int epv = 16 / esize;
  // eight vectors per lane only pay for bf16 (the other types then run at a quarter of the occupancy)
  const int lim = loss && !grad ? kVRowsMaxVec : kVRowsMaxVec / 2;
  return v % epv == 0 && v / epv <= lim && fm_host::aligned16(logits) && (!grad || fm_host::aligned16(dlogits));
}

template <typename T, bool LOSS, bool GRAD>
bool launch_vrows(const void* logits, const int64_t* labels, const float* n_valid, const float* grad_out,
                  float* lse, float* row_loss, void* dlogits, int64_t n, int v, int64_t ignore_index,
                  hipStream_t st) {
  constexpr int EPV = Elem<T>::kVec;
  if (!vrows_fits(v, (int)sizeof(T), std::is_same<T, bf16_t>::value, logits, dlogits, LOSS, GRAD)) return false;
  // four vectors a lane where the row has them: a wave then keeps 4 KiB in flight, and narrow
  // rows share it (a 512-element bf16 row takes 16 lanes, not 64)
  const int nvec = v / EPV;
  int tpr = 4;
  while (tpr < 64 && tpr * 4 < nvec) tpr *= 2;
  int iters = 1;
  while (tpr * iters < nvec) iters *= 2;
  const dim3 grid((unsigned)((n + 256 / tpr - 1) / (256 / tpr)));
#define GOV(TPR_, IT_)                                                                              \
  if (tpr == TPR_ && iters == IT_) {                                                                \
    FM_LAUNCH((ce_vrows_kernel<T, TPR_, IT_, LOSS, GRAD>), grid, dim3(256), 0, st,         \
                       static_cast<const T*>(logits), labels, n_valid, grad_out, lse, row_loss,     \
                       static_cast<T*>(dlogits), n, v, ignore_index);                               \
    return true;                                                                                    \
  }
  GOV(4, 1) GOV(4, 2) GOV(4, 4) GOV(8, 4) GOV(16, 4) GOV(32, 4) GOV(64, 4)
  if constexpr (LOSS && !GRAD) { GOV(64, 8) }
#undef GOV
  return false;
}

// rows of up to 1024 logits go to ce_rows_kernel; returns false for wider rows
// Widest row the lane-group kernel takes.
inline int rows_max_v() { return 64 * 16; }

template <typename T, bool LOSS, bool GRAD>
bool launch_rows(const void* logits, const int64_t* labels, const float* n_valid, const float* grad_out,
                 float* lse, float* row_loss, void* dlogits, int64_t n, int v, int64_t ignore_index,
                 hipStream_t st) {
  if (launch_vrows<T, LOSS, GRAD>(logits, labels, n_valid, grad_out, lse, row_loss, dlogits, n, v, ignore_index, st))
    return true;
  if (v > rows_max_v()) return false;
  // fp32 gradients of rows past 512 classes go faster through the workgroup-per-row kernels
  if (GRAD && sizeof(T) == 4 && v > 512) return false;
  const int tpr = v <= 16 * 16 ? 16 : 64;
  int iters = 1;
  while (tpr * iters < v) iters *= 2;
  const dim3 grid((unsigned)((n + 256 / tpr - 1) / (256 / tpr)));
#define GOR(TPR_, IT_)                                                                              \
  if (tpr == TPR_ && iters == IT_) {                                                                \
    FM_LAUNCH((ce_rows_kernel<T, TPR_, IT_, LOSS, GRAD>), grid, dim3(256), 0, st,          \
                       static_cast<const T*>(logits), labels, n_valid, grad_out, lse, row_loss,     \
                       static_cast<T*>(dlogits), n, v, ignore_index);                               \
    return true;                                                                                    \
  }
  GOR(16, 1) GOR(16, 2) GOR(16, 4) GOR(16, 8) GOR(16, 16) GOR(64, 8) GOR(64, 16)
#undef GOR
  return false;
}

#define FM_CE_BY_DTYPE(dtype, CALL)              \
  do {                                           \
    if ((dtype) == FM_F32) { CALL(float); }      \
    else if ((dtype) == FM_BF16) { CALL(bf16_t); } \
    else { CALL(f16_t); }                        \
  } while (0)

// What the memory-side cache of the part holds (MI355X: 256 MiB): the forward that expects a backward
// reads that much of its input, the last rows, with cached loads. [8192,32000] bf16 forward + backward:
// 250.0 us with streaming loads throughout, 242.9 with the last 50 % of the rows (262 MB) cached,
// 248.1 / 246.5 / 247.0 with the last 40 / 60 / 70 %, 244.8 with all of them, 245.6 with the FIRST
// half, 252.9 with the backward walking the rows in reverse (the forward alone is 12 % slower on the
// rows it reads with cached loads).
constexpr int64_t kKeepBytes = 256ll << 20;

template <typename T>
int launch_fwd(const void* logits, const int64_t* labels, float* lse, float* row_loss, int64_t n,
               int v, int64_t ignore_index, bool vec_ok, bool backward_follows, hipStream_t st) {
  const T* lp = static_cast<const T*>(logits);
  // the forward alone keeps 256 threads up to 24 KiB rows (16 KiB rows: 50 against 65 us per 256 MiB)
  const fm_host::VocabShape sh = fm_host::vocab_shape(v, sizeof(T), 512, 4, 24 * 1024);
  int64_t kept = backward_follows ? kKeepBytes / ((int64_t)v * (int64_t)sizeof(T)) : 0;
  if (kept > n) kept = n;
  const int64_t streamed = n - kept;
#define LAUNCH(TH, UN)                                                                          \
  do {                                                                                          \
    if (streamed > 0)                                                                           \
      FM_LAUNCH((ce_fwd_kernel<T, TH, UN, false>), dim3((unsigned)streamed), dim3(TH), 0, st, lp, labels, lse, \
                row_loss, v, ignore_index, vec_ok, (int64_t)0);                                 \
    if (kept > 0)                                                                               \
      FM_LAUNCH((ce_fwd_kernel<T, TH, UN, true>), dim3((unsigned)kept), dim3(TH), 0, st, lp, labels, lse, \
                row_loss, v, ignore_index, vec_ok, streamed);                                   \
  } while (0)
  FM_VOCAB_DISPATCH(sh, LAUNCH);
#undef LAUNCH
  return FM_OK;
}

template <typename T>
int launch_bwd(const void* logits, const int64_t* labels, const float* lse, const float* n_valid,
               const float* grad_out, void* dlogits, int64_t n, int v, int64_t ignore_index,
               bool vec_ok, hipStream_t st) {
  const T* lp = static_cast<const T*>(logits);
  T* gp = static_cast<T*>(dlogits);
  const fm_host::VocabShape sh = fm_host::vocab_shape(v, sizeof(T), 1024, 4);
  // rows longer than one tile (threads x unroll vectors): a workgroup per tile
  const int64_t tile = (int64_t)sh.threads * sh.unroll;
  int64_t chunks = (v / Elem<T>::kVec + 1 + tile - 1) / tile;
  if (chunks < 1 || n * chunks > 0x7fffffffLL) chunks = 1;
  const dim3 grid((unsigned)(n * chunks));
#define LAUNCH(TH, UN)                                                                         \
  FM_LAUNCH((ce_bwd_kernel<T, TH, UN>), grid, dim3(TH), 0, st, lp, labels, lse, n_valid, \
                     grad_out, gp, v, ignore_index, vec_ok, (int)chunks)
  FM_VOCAB_DISPATCH(sh, LAUNCH);
#undef LAUNCH
  return FM_OK;
}

int check_shape(const char* what, int64_t n, int64_t v, int dtype) {
  FM_CHECK_ARG(n >= 0 && v > 0, "%s: bad shape n=%lld v=%lld", what, (long long)n, (long long)v);
  FM_CHECK_ARG(dtype == FM_F32 || dtype == FM_F16 || dtype == FM_BF16, "%s: bad dtype %d", what,
               dtype);
  if (n > 0x7fffffffLL || v > 0x7fffffffLL) {
    fm_host::set_error("%s: n and v must be below 2^31", what);
    return FM_ERR_UNSUPPORTED;
  }
  return FM_OK;
}

}  // namespace

extern "C" {

int fm_ce_fwd(const void* logits, const int64_t* labels, float* lse, float* row_loss, float* loss,
              float* n_valid, int64_t n, int64_t v, int dtype, int64_t ignore_index, int reduction,
              fm_stream_t stream) {
  int rc = check_shape("fm_ce_fwd", n, v, dtype);
  if (rc != FM_OK) return rc;
  FM_CHECK_ARG(reduction == FM_REDUCE_SUM || reduction == FM_REDUCE_MEAN,
               "fm_ce_fwd: reduction must be sum or mean (got %d)", reduction);
  FM_CHECK_ARG(loss && n_valid, "fm_ce_fwd: NULL scalar output");
  FM_CHECK_ARG(n == 0 || (logits && labels && row_loss), "fm_ce_fwd: NULL pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  bool narrow = false;
  if (n > 0) {
#define CALL(T) narrow = launch_rows<T, true, false>(logits, labels, nullptr, nullptr, lse, row_loss, nullptr, n, (int)v, ignore_index, st)
    FM_CE_BY_DTYPE(dtype, CALL);
#undef CALL
  }
  if (n > 0 && !narrow) {
    const bool vec_ok = fm_host::aligned16(logits);
    const bool bwd = lse != nullptr;   // the saved log-sum-exps are what a backward needs: no lse, no backward
    if (dtype == FM_F32) launch_fwd<float>(logits, labels, lse, row_loss, n, (int)v, ignore_index, vec_ok, bwd, st);
    else if (dtype == FM_BF16) launch_fwd<bf16_t>(logits, labels, lse, row_loss, n, (int)v, ignore_index, vec_ok, bwd, st);
    else launch_fwd<f16_t>(logits, labels, lse, row_loss, n, (int)v, ignore_index, vec_ok, bwd, st);
  }
  if (n > 0) FM_CHECK_LAUNCH("fm_ce_fwd");
  hipLaunchKernelGGL(ce_finalize_kernel, dim3(1), dim3(1024), 0, st, row_loss, labels, n,
                     ignore_index, reduction == FM_REDUCE_MEAN ? 1 : 0, loss, n_valid);
  FM_CHECK_LAUNCH("fm_ce_fwd(finalize)");
  return FM_OK;
}

int fm_ce_bwd(const void* logits, const int64_t* labels, const float* lse, const float* n_valid,
              const float* grad_out, void* dlogits, int64_t n, int64_t v, int dtype,
              int64_t ignore_index, fm_stream_t stream) {
  int rc = check_shape("fm_ce_bwd", n, v, dtype);
  if (rc != FM_OK) return rc;
  if (n == 0) return FM_OK;
  FM_CHECK_ARG(logits && labels && lse && dlogits, "fm_ce_bwd: NULL pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  bool narrow = false;
#define CALL(T) narrow = launch_rows<T, false, true>(logits, labels, n_valid, grad_out, nullptr, nullptr, dlogits, n, (int)v, ignore_index, st)
  FM_CE_BY_DTYPE(dtype, CALL);
#undef CALL
  if (narrow) {
    FM_CHECK_LAUNCH("fm_ce_bwd");
    return FM_OK;
  }
  const bool vec_ok = fm_host::aligned16(logits) && fm_host::aligned16(dlogits);
  if (dtype == FM_F32) launch_bwd<float>(logits, labels, lse, n_valid, grad_out, dlogits, n, (int)v, ignore_index, vec_ok, st);
  else if (dtype == FM_BF16) launch_bwd<bf16_t>(logits, labels, lse, n_valid, grad_out, dlogits, n, (int)v, ignore_index, vec_ok, st);
  else launch_bwd<f16_t>(logits, labels, lse, n_valid, grad_out, dlogits, n, (int)v, ignore_index, vec_ok, st);
  FM_CHECK_LAUNCH("fm_ce_bwd");
  return FM_OK;
}

int fm_ce_loss_grad(const void* logits, const int64_t* labels, float* lse, float* row_loss,
                    float* loss, float* n_valid, void* dlogits, int64_t n, int64_t v, int dtype,
                    int64_t ignore_index, int reduction, fm_stream_t stream) {
  int rc = check_shape("fm_ce_loss_grad", n, v, dtype);
  if (rc != FM_OK) return rc;
  FM_CHECK_ARG(reduction == FM_REDUCE_SUM || reduction == FM_REDUCE_MEAN,
               "fm_ce_loss_grad: reduction must be sum or mean (got %d)", reduction);
  FM_CHECK_ARG(loss && n_valid, "fm_ce_loss_grad: NULL scalar output");
  FM_CHECK_ARG(n == 0 || (logits && labels && row_loss && dlogits), "fm_ce_loss_grad: NULL pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int esize = dtype == FM_F32 ? 4 : 2;
  const int64_t nvec = v / (16 / esize);
  if (n > 0 && (vrows_fits((int)v, esize, dtype == FM_BF16, logits, dlogits, true, true) ||
                (v <= rows_max_v() && !(esize == 4 && v > 512)))) {   // narrow rows: lane groups, in place allowed
    const bool mean_ = reduction == FM_REDUCE_MEAN;
    if (mean_) {
      hipLaunchKernelGGL(ce_count_kernel, dim3(1), dim3(1024), 0, st, labels, n, ignore_index, n_valid);
      FM_CHECK_LAUNCH("fm_ce_loss_grad(count)");
    }
    bool done = false;
#define CALL(T) done = launch_rows<T, true, true>(logits, labels, mean_ ? n_valid : nullptr, nullptr, lse, row_loss, dlogits, n, (int)v, ignore_index, st)
    FM_CE_BY_DTYPE(dtype, CALL);
#undef CALL
    if (done) {
      FM_CHECK_LAUNCH("fm_ce_loss_grad");
      hipLaunchKernelGGL(ce_finalize_kernel, dim3(1), dim3(1024), 0, st, row_loss, labels, n, ignore_index,
                         mean_ ? 1 : 0, loss, n_valid);
      FM_CHECK_LAUNCH("fm_ce_loss_grad(finalize)");
      return FM_OK;
    }
  }
  const bool one_pass = n > 0 && fm_host::aligned16(logits) && fm_host::aligned16(dlogits) &&
                        nvec <= 8 * 1024;
  // wider, up to what a compute unit holds: the row stays on the chip (needs 128 KB of LDS granted)
  if (!one_pass && n > 0 && fm_host::aligned16(logits) && fm_host::aligned16(dlogits) &&
      nvec <= 2 * kCeHeldMaxVec) {
    bool granted = false;
#define GRANT(T) granted = fm_host::grant_dynamic_lds<&ce_loss_grad_held_kernel<T>>(kCeHeldLds * kCeHeldThreads * 16)
    FM_CE_BY_DTYPE(dtype, GRANT);
#undef GRANT
    if (granted) {
      const bool mean_ = reduction == FM_REDUCE_MEAN;
      if (mean_) {
        hipLaunchKernelGGL(ce_count_kernel, dim3(1), dim3(1024), 0, st, labels, n, ignore_index, n_valid);
        FM_CHECK_LAUNCH("fm_ce_loss_grad(count)");
      }
#define HELD(T)                                                                                    \
  FM_LAUNCH((ce_loss_grad_held_kernel<T>), dim3((unsigned)n), dim3(kCeHeldThreads),                \
            (size_t)kCeHeldLds * kCeHeldThreads * 16, st, static_cast<const T*>(logits), labels,    \
            mean_ ? n_valid : nullptr, lse, row_loss, static_cast<T*>(dlogits), (int)v, ignore_index)
      FM_CE_BY_DTYPE(dtype, HELD);
#undef HELD
      FM_CHECK_LAUNCH("fm_ce_loss_grad");
      hipLaunchKernelGGL(ce_finalize_kernel, dim3(1), dim3(1024), 0, st, row_loss, labels, n, ignore_index,
                         mean_ ? 1 : 0, loss, n_valid);
      FM_CHECK_LAUNCH("fm_ce_loss_grad(finalize)");
      return FM_OK;
    }
  }
  if (!one_pass) {
    // rows too wide for the register file (or unaligned buffers): two sweeps in one launch
    if (n > 0) {
      const bool mean_ = reduction == FM_REDUCE_MEAN;
      if (mean_) {
        hipLaunchKernelGGL(ce_count_kernel, dim3(1), dim3(1024), 0, st, labels, n, ignore_index, n_valid);
        FM_CHECK_LAUNCH("fm_ce_loss_grad(count)");
      }
      const bool vec_ok = fm_host::aligned16(logits) && fm_host::aligned16(dlogits);
      const dim3 wgrid((unsigned)n);
#define WIDE(T)                                                                                   \
  FM_LAUNCH((ce_loss_grad_wide_kernel<T, 1024, 2>), wgrid, dim3(1024), 0, st,            \
                     static_cast<const T*>(logits), labels, mean_ ? n_valid : nullptr, lse, row_loss, \
                     static_cast<T*>(dlogits), (int)v, ignore_index, vec_ok)
      FM_CE_BY_DTYPE(dtype, WIDE);
#undef WIDE
      FM_CHECK_LAUNCH("fm_ce_loss_grad");
    }
    hipLaunchKernelGGL(ce_finalize_kernel, dim3(1), dim3(1024), 0, st, row_loss, labels, n, ignore_index,
                       reduction == FM_REDUCE_MEAN ? 1 : 0, loss, n_valid);
    FM_CHECK_LAUNCH("fm_ce_loss_grad(finalize)");
    return FM_OK;
  }
  const bool mean = reduction == FM_REDUCE_MEAN;
  const int pref = fm_host::get_param(fm_host::P_VOCAB_THREADS);
  if (mean) {
    hipLaunchKernelGGL(ce_count_kernel, dim3(1), dim3(1024), 0, st, labels, n, ignore_index, n_valid);
    FM_CHECK_LAUNCH("fm_ce_loss_grad(count)");
  }
  const float* nv = mean ? n_valid : nullptr;
  const dim3 grid((unsigned)n);
#define LAUNCH(T, TH, IT)                                                                        \
  FM_LAUNCH((ce_loss_grad_kernel<T, TH, IT>), grid, dim3(TH), 0, st,                    \
                     static_cast<const T*>(logits), labels, nv, lse, row_loss,                   \
                     static_cast<T*>(dlogits), (int)v, ignore_index)
#define BY_ITERS(T, TH)                        \
  do {                                         \
    if (iters == 2) LAUNCH(T, TH, 2);          \
    else if (iters == 4) LAUNCH(T, TH, 4);     \
    else if (iters == 8) LAUNCH(T, TH, 8);     \
    else LAUNCH(T, TH, 16);                    \
  } while (0)
#define BY_SHAPE(T)                            \
  do {                                         \
    if (threads == 256) BY_ITERS(T, 256);      \
    else if (threads == 512) BY_ITERS(T, 512); \
    else if (iters == 2) LAUNCH(T, 1024, 2);   \
    else if (iters == 4) LAUNCH(T, 1024, 4);   \
    else LAUNCH(T, 1024, 8);                   \
  } while (0)
  // the fewest threads that hold the row in at most 8 vectors each: small workgroups keep
  // several rows per compute unit in different phases (loading, reducing, storing). fp16 and
  // fp32 rows stop at 4 vectors below 1024 threads: with 8 the compiler keeps the converted
  // values of all of them alive (over 220 registers, one workgroup per unit).
  const int per_thread = dtype == FM_BF16 ? 8 : 4;
  int threads = pref == 256 || pref == 512 || pref == 1024 ? pref : 256;
  while (threads < 1024 && nvec > (int64_t)threads * per_thread) threads *= 2;
  int iters = 2;
  while ((int64_t)threads * iters < nvec) iters *= 2;
  if (dtype == FM_F32) BY_SHAPE(float);
  else if (dtype == FM_BF16) BY_SHAPE(bf16_t);
  else BY_SHAPE(f16_t);
#undef BY_ITERS
#undef BY_SHAPE
#undef LAUNCH
  FM_CHECK_LAUNCH("fm_ce_loss_grad");
  hipLaunchKernelGGL(ce_finalize_kernel, dim3(1), dim3(1024), 0, st, row_loss, labels, n,
                     ignore_index, mean ? 1 : 0, loss, n_valid);
  FM_CHECK_LAUNCH("fm_ce_loss_grad(finalize)");
  return FM_OK;
}

int fm_scale_inplace(void* x, const float* factor, int64_t count, int dtype, fm_stream_t stream) {
  FM_CHECK_ARG(count >= 0, "fm_scale_inplace: bad count %lld", (long long)count);
  FM_CHECK_ARG(dtype == FM_F32 || dtype == FM_F16 || dtype == FM_BF16, "fm_scale_inplace: bad dtype %d",
               dtype);
  if (count == 0) return FM_OK;
  FM_CHECK_ARG(x && factor, "fm_scale_inplace: NULL pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool vec_ok = fm_host::aligned16(x);
  const int64_t per_block = 1024 * 8 * 4;   // elements a workgroup covers per sweep, roughly
  int64_t blocks = (count + per_block - 1) / per_block;
  const int64_t cap = (int64_t)fm_host::num_cus() * 8;
  if (blocks > cap) blocks = cap;
  const dim3 grid((unsigned)blocks);
  if (dtype == FM_F32) hipLaunchKernelGGL(scale_inplace_kernel<float>, grid, dim3(1024), 0, st, static_cast<float*>(x), factor, count, vec_ok);
  else if (dtype == FM_BF16) hipLaunchKernelGGL(scale_inplace_kernel<bf16_t>, grid, dim3(1024), 0, st, static_cast<bf16_t*>(x), factor, count, vec_ok);
  else hipLaunchKernelGGL(scale_inplace_kernel<f16_t>, grid, dim3(1024), 0, st, static_cast<f16_t*>(x), factor, count, vec_ok);
  FM_CHECK_LAUNCH("fm_scale_inplace");
  return FM_OK;
}

}  // extern "C"
