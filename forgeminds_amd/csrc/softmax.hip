// Row softmax over the last dimension for gfx950.
//
// Reference semantics: forgemind/kernels/softmax.py:27-80 (y = exp(x - max) / sum, fp32
// math, stored in x's dtype; NaN propagates, a row of -inf yields NaN like torch).
// Rows of up to 128 KiB whose width is a whole number of 16-byte vectors stay in registers:
// a row is owned by TPR threads (a lane group, a wave or the waves of one workgroup, several
// rows per workgroup when they are narrow), read once, reduced (maximum, then sum) and written.
// Aligned rows from 8192 vectors on stay on the chip instead (registers and LDS of one workgroup
// per compute unit; what a row has beyond that is streamed and read again).
// Other rows take one workgroup each: an online (max, sum-exp) pass, then a second pass over
// the row (served by L2 for rows that fit) that writes exp2(z - m) / s.
//
// Backward (forgemind/kernels/softmax.py:108-115: dx = (dy - sum(dy * y)) * y): the same three
// shapes over two inputs, fp32 math on the stored y and dy, one rounding at the store.
#include "fm_vocab.hip.h"

using namespace fm;

namespace {

template <typename T, int THREADS, int UNROLL>
__global__ __launch_bounds__(THREADS) void softmax_kernel(const T* __restrict__ x, T* __restrict__ y,
                                                           int v, bool vec_ok) {
  constexpr int EPV = Elem<T>::kVec;
  constexpr int NW = THREADS / 64;
  __shared__ float smem[2 * NW];
  const int64_t row = blockIdx.x;
  const T* rp = x + row * (int64_t)v;
  T* op = y + row * (int64_t)v;
  const RowSplit sp = split_row<EPV>(row, v, vec_ok);
  const int tid = threadIdx.x;
  const int ne = edge_count(sp, v);

  MaxSum st{kNegBig, 0.f};
  for (int c0 = 0; c0 < sp.nvec; c0 += THREADS * UNROLL) {
    u32x4 raw[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int c = clamp_col(c0 + u * THREADS + tid, sp.nvec);
      raw[u] = load16(rp + sp.head + (int64_t)c * EPV);
    }
    float z[UNROLL][EPV];
    float cm = st.m;
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int c = c0 + u * THREADS + tid;
      if (c < sp.nvec) {
        Elem<T>::unpack(raw[u], z[u]);
#pragma unroll
        for (int e = 0; e < EPV; ++e) { z[u][e] *= kLog2e; cm = fmaxf(cm, z[u][e]); }
      } else {
#pragma unroll
        for (int e = 0; e < EPV; ++e) z[u][e] = -INFINITY;
      }
    }
    float acc = st.s * fast_exp2(st.m - cm);
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
#pragma unroll
      for (int e = 0; e < EPV; ++e) acc += fast_exp2(z[u][e] - cm);
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
  // a row whose maximum is -inf has sum 0: 0 * inf = NaN, which is what torch returns
  const float inv = 1.f / tot.s;
  for (int c0 = 0; c0 < sp.nvec; c0 += THREADS * UNROLL) {
    u32x4 raw[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int c = clamp_col(c0 + u * THREADS + tid, sp.nvec);
      raw[u] = load16(rp + sp.head + (int64_t)c * EPV);
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int c = c0 + u * THREADS + tid;
      touch(raw[u]);
      if (c < sp.nvec) {
        float z[EPV], o[EPV];
        Elem<T>::unpack(raw[u], z);
#pragma unroll
        for (int e = 0; e < EPV; ++e) o[e] = fast_exp2(z[e] * kLog2e - tot.m) * inv;
        store16_stream(op + sp.head + (int64_t)c * EPV, Elem<T>::pack(o));
      }
    }
  }
  for (int e = tid; e < ne; e += THREADS) {
    const int col = edge_col(sp, e);
    Elem<T>::store1(op + col, fast_exp2(Elem<T>::load1(rp + col) * kLog2e - tot.m) * inv);
  }
}

template <int TPR> struct RowBlock { static constexpr int value = TPR > 256 ? TPR : 256; };

template <typename T, int TPR, int ITERS>
__global__ __launch_bounds__(RowBlock<TPR>::value) void softmax_rows_kernel(const T* __restrict__ x,
                                                                             T* __restrict__ y, int64_t n,
                                                                             int v) {
  constexpr int EPV = Elem<T>::kVec;
  constexpr int BLOCK = RowBlock<TPR>::value;
  constexpr int RPB = BLOCK / TPR;
  __shared__ float smem[RPB * (TPR > 64 ? TPR / 64 : 1)];
  const int tid = threadIdx.x;
  const int rib = tid / TPR;
  const int t = tid % TPR;
  const int64_t row = (int64_t)blockIdx.x * RPB + rib;
  const bool valid = row < n;
  const int nvec = v / EPV;
  const int64_t base = row * (int64_t)v;

  float z[ITERS][EPV];
  float m = kNegBig;
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
    const int c = i * TPR + t;
    if (valid && c < nvec) {
      Elem<T>::unpack(load16_stream(x + base + (int64_t)c * EPV), z[i]);
#pragma unroll
      for (int e = 0; e < EPV; ++e) { z[i][e] *= kLog2e; m = fmaxf(m, z[i][e]); }
    } else {
#pragma unroll
      for (int e = 0; e < EPV; ++e) z[i][e] = -INFINITY;
    }
  }
  // a NaN anywhere must reach the whole row: fmaxf drops it, so it is carried in the sum
  m = row_reduce<TPR, OpMax>(m, smem, rib, t);
  float ssum = 0.f;
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
#pragma unroll
    for (int e = 0; e < EPV; ++e) {
      z[i][e] = fast_exp2(z[i][e] - m);
      ssum += z[i][e];
    }
  }
  ssum = row_reduce<TPR, OpSum>(ssum, smem, rib, t);
  // a row whose maximum is -inf has sum 0: 0 * inf = NaN, which is what torch returns
  const float inv = 1.f / ssum;
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
    const int c = i * TPR + t;
    if (valid && c < nvec) {
      float o[EPV];
#pragma unroll
      for (int e = 0; e < EPV; ++e) o[e] = z[i][e] * inv;
      store16_stream(y + base + (int64_t)c * EPV, Elem<T>::pack(o));
    }
  }
}

// Narrow rows whose width is not a whole number of 16-byte vectors (or whose buffers are not
// 16-byte aligned): the same scheme with one element per load. Lane t of a row's TPR lanes holds
// elements t, t + TPR, ...
template <typename T, int TPR, int ITERS>
__global__ __launch_bounds__(256) void softmax_rows_scalar_kernel(const T* __restrict__ x,
                                                                  T* __restrict__ y, int64_t n, int v) {
  constexpr int RPB = 256 / TPR;
  const int tid = threadIdx.x;
  const int rib = tid / TPR;
  const int t = tid % TPR;
  const int64_t row = (int64_t)blockIdx.x * RPB + rib;
  const bool valid = row < n;
  const int64_t base = row * (int64_t)v;
  float z[ITERS];
  float m = kNegBig;
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
    const int c = i * TPR + t;
    z[i] = (valid && c < v) ? Elem<T>::load1(x + base + c) * kLog2e : -INFINITY;
    m = fmaxf(m, z[i]);
  }
  m = group_reduce<TPR, OpMax>(m);
  float ssum = 0.f;
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
    z[i] = fast_exp2(z[i] - m);
    ssum += z[i];
  }
  ssum = group_reduce<TPR, OpSum>(ssum);
  const float inv = 1.f / ssum;
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
    const int c = i * TPR + t;
    if (valid && c < v) Elem<T>::store1(y + base + c, z[i] * inv);
  }
}


// ---------------------------------------------------------------- backward
template <typename T, int THREADS, int UNROLL>
__global__ __launch_bounds__(THREADS) void softmax_bwd_kernel(const T* __restrict__ y,
                                                               const T* __restrict__ dy,
                                                               T* __restrict__ dx, int v, bool vec_ok) {
  constexpr int EPV = Elem<T>::kVec;
  constexpr int NW = THREADS / 64;
  __shared__ float smem[NW];
  const int64_t row = blockIdx.x;
  const T* yp = y + row * (int64_t)v;
  const T* gp = dy + row * (int64_t)v;
  T* op = dx + row * (int64_t)v;
  const RowSplit sp = split_row<EPV>(row, v, vec_ok);
  const int tid = threadIdx.x;
  const int ne = edge_count(sp, v);
  float dot = 0.f;
  for (int c0 = 0; c0 < sp.nvec; c0 += THREADS * UNROLL) {
    u32x4 ry[UNROLL], rg[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int c = clamp_col(c0 + u * THREADS + tid, sp.nvec);
      ry[u] = load16(yp + sp.head + (int64_t)c * EPV);
      rg[u] = load16(gp + sp.head + (int64_t)c * EPV);
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int c = c0 + u * THREADS + tid;
      if (c < sp.nvec) {
        float a[EPV], b[EPV];
        Elem<T>::unpack(ry[u], a);
        Elem<T>::unpack(rg[u], b);
#pragma unroll
        for (int e = 0; e < EPV; ++e) dot += a[e] * b[e];
      }
    }
  }
  for (int e = tid; e < ne; e += THREADS) {
    const int col = edge_col(sp, e);
    dot += Elem<T>::load1(yp + col) * Elem<T>::load1(gp + col);
  }
  dot = block_sum<NW>(dot, smem);
  for (int c0 = 0; c0 < sp.nvec; c0 += THREADS * UNROLL) {
    u32x4 ry[UNROLL], rg[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int c = clamp_col(c0 + u * THREADS + tid, sp.nvec);
      ry[u] = load16(yp + sp.head + (int64_t)c * EPV);
      rg[u] = load16(gp + sp.head + (int64_t)c * EPV);
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int c = c0 + u * THREADS + tid;
      touch(ry[u]);
      touch(rg[u]);
      if (c < sp.nvec) {
        float a[EPV], b[EPV], o[EPV];
        Elem<T>::unpack(ry[u], a);
        Elem<T>::unpack(rg[u], b);
#pragma unroll
        for (int e = 0; e < EPV; ++e) o[e] = (b[e] - dot) * a[e];
        store16_stream(op + sp.head + (int64_t)c * EPV, Elem<T>::pack(o));
      }
    }
  }
  for (int e = tid; e < ne; e += THREADS) {
    const int col = edge_col(sp, e);
    Elem<T>::store1(op + col, (Elem<T>::load1(gp + col) - dot) * Elem<T>::load1(yp + col));
  }
}

template <typename T, int TPR, int ITERS>
__global__ __launch_bounds__(RowBlock<TPR>::value) void softmax_bwd_rows_kernel(const T* __restrict__ y,
                                                                                 const T* __restrict__ dy,
                                                                                 T* __restrict__ dx,
                                                                                 int64_t n, int v) {
  constexpr int EPV = Elem<T>::kVec;
  constexpr int BLOCK = RowBlock<TPR>::value;
  constexpr int RPB = BLOCK / TPR;
  __shared__ float smem[RPB * (TPR > 64 ? TPR / 64 : 1)];
  const int tid = threadIdx.x;
  const int rib = tid / TPR;
  const int t = tid % TPR;
  const int64_t row = (int64_t)blockIdx.x * RPB + rib;
  const bool valid = row < n;
  const int nvec = v / EPV;
  const int64_t base = row * (int64_t)v;
  u32x4 ry[ITERS], rg[ITERS];      // both rows stay packed between the dot product and the store
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
    const int c = i * TPR + t;
    if (valid && c < nvec) {
      ry[i] = load16_stream(y + base + (int64_t)c * EPV);
      rg[i] = load16_stream(dy + base + (int64_t)c * EPV);
    } else {
      ry[i] = u32x4{0u, 0u, 0u, 0u};
      rg[i] = u32x4{0u, 0u, 0u, 0u};
    }
  }
  float dot = 0.f;
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
    float a[EPV], b[EPV];
    Elem<T>::unpack(ry[i], a);
    Elem<T>::unpack(rg[i], b);
#pragma unroll
    for (int e = 0; e < EPV; ++e) dot += a[e] * b[e];
  }
  dot = row_reduce<TPR, OpSum>(dot, smem, rib, t);
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
    const int c = i * TPR + t;
    if (valid && c < nvec) {
      float a[EPV], b[EPV], o[EPV];
      Elem<T>::unpack(ry[i], a);
      Elem<T>::unpack(rg[i], b);
#pragma unroll
      for (int e = 0; e < EPV; ++e) o[e] = (b[e] - dot) * a[e];
      store16_stream(dx + base + (int64_t)c * EPV, Elem<T>::pack(o));
    }
  }
}

template <typename T, int TPR, int ITERS>
__global__ __launch_bounds__(256) void softmax_bwd_rows_scalar_kernel(const T* __restrict__ y,
                                                                      const T* __restrict__ dy,
                                                                      T* __restrict__ dx, int64_t n, int v) {
  constexpr int RPB = 256 / TPR;
  const int tid = threadIdx.x;
  const int rib = tid / TPR;
  const int t = tid % TPR;
  const int64_t row = (int64_t)blockIdx.x * RPB + rib;
  const bool valid = row < n;
  const int64_t base = row * (int64_t)v;
  float a[ITERS], b[ITERS];
  float dot = 0.f;
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
    const int c = i * TPR + t;
    const bool in = valid && c < v;
    a[i] = in ? Elem<T>::load1(y + base + c) : 0.f;
    b[i] = in ? Elem<T>::load1(dy + base + c) : 0.f;
    dot += a[i] * b[i];
  }
  dot = group_reduce<TPR, OpSum>(dot);
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
    const int c = i * TPR + t;
    if (valid && c < v) Elem<T>::store1(dx + base + c, (b[i] - dot) * a[i]);
  }
}

#define FM_SOFTMAX_SHAPES(X) \
  X(1, 1) X(2, 1) X(4, 1) X(8, 1) X(16, 1) X(32, 1) X(64, 1) X(64, 2) X(128, 2) X(256, 2) X(256, 4) X(512, 4) X(512, 8) X(1024, 8)

// threads per row and vectors per thread for a row of nvec 16-byte vectors; false: too wide
bool rows_plan(int64_t nvec, int* tpr, int* iters) {
  static const int kPlans[][3] = {{1, 1, 1},     {2, 2, 1},      {4, 4, 1},     {8, 8, 1},      {16, 16, 1},    {32, 32, 1},
                                  {64, 64, 1},   {128, 64, 2},   {256, 128, 2},  {512, 256, 2},
                                  {1024, 256, 4}, {2048, 512, 4}, {4096, 512, 8}, {8192, 1024, 8}};
  for (auto& pl : kPlans) {
    if (nvec <= pl[0]) { *tpr = pl[1]; *iters = pl[2]; return true; }
  }
  return false;
}

// lanes per row and elements per lane of the scalar lane-group kernels (v <= 1024): about
// Rows past the register kernels that still fit the CHIP, one workgroup per compute unit, the row
// read once. Forward: 1024 threads keep 16 vectors each in registers and 8 more in 128 KB of LDS
// (24576 vectors, 196608 bf16 columns); the three passes (maximum, sum, output) unpack the packed
// vectors afresh. Backward (two rows, y and dy): 512 threads with twice the registers each, 24 + 8
// vector pairs a thread (16384 pairs). Every thread parks and fetches its own LDS slots only, so
// the passes need no barrier for them.
constexpr int kHeldFwdThreads = 1024, kHeldFwdRegs = 16, kHeldFwdLds = 8;
constexpr int kHeldFwdMaxVec = kHeldFwdThreads * (kHeldFwdRegs + kHeldFwdLds);
constexpr int kHeldBwdThreads = 512, kHeldBwdRegs = 24, kHeldBwdLds = 8;
constexpr int kHeldBwdMaxVec = kHeldBwdThreads * (kHeldBwdRegs + kHeldBwdLds);

template <typename T>
__global__ __launch_bounds__(kHeldFwdThreads) void softmax_held_kernel(const T* __restrict__ x,
                                                                        T* __restrict__ y, int v) {
  constexpr int EPV = Elem<T>::kVec;
  constexpr int THREADS = kHeldFwdThreads, RI = kHeldFwdRegs, LI = kHeldFwdLds;
  constexpr int NW = THREADS / 64;
  extern __shared__ u32x4 parked[];          // [LI][THREADS]
  __shared__ float smem[2 * NW];
  const int64_t row = blockIdx.x;
  const T* rp = x + row * (int64_t)v;
  T* op = y + row * (int64_t)v;
  const RowSplit sp = split_row<EPV>(row, v, true);
  const int tid = threadIdx.x;
  const int ne = edge_count(sp, v);
  // the unaligned ends of the row first (at most EPV - 1 elements each, thread e keeps edge e): a
  // wait for them then waits for nothing that was issued behind them
  float edge = -INFINITY;
  int edge_at = -1;
  if (tid < ne) {
    edge_at = edge_col(sp, tid);
    edge = Elem<T>::load1(rp + edge_at) * kLog2e;
  }
  u32x4 raw[RI];
#pragma unroll
  for (int i = 0; i < RI; ++i)
    raw[i] = load16_stream(rp + sp.head + (int64_t)clamp_col(i * THREADS + tid, sp.nvec) * EPV);
  auto vec = [&](int i) -> u32x4 {
    if (i < RI) { touch(raw[i < RI ? i : 0]); return raw[i < RI ? i : 0]; }
    return parked[(i - RI) * THREADS + tid];
  };
  // Running (maximum, sum), one vector at a time in the order the loads were issued: the wait
  // before vector i counts the loads issued after it, so the arithmetic on the first vectors runs
  // while the later ones are still on their way. The LDS share is filled straight from memory, and
  // requested only behind that (with a load into LDS outstanding the compiler waits for ALL
  // vector-memory operations wherever it has to wait for one). A NaN anywhere must reach the whole
  // row: fmaxf drops it, the sum carries it.
  MaxSum st{fmaxf(edge, kNegBig), 0.f};
  if (edge_at >= 0) st.s = fast_exp2(edge - st.m);
  auto fold = [&](const u32x4& r) {
    float z[EPV];
    Elem<T>::unpack(r, z);
    float cm = st.m;
#pragma unroll
    for (int e = 0; e < EPV; ++e) { z[e] *= kLog2e; cm = fmaxf(cm, z[e]); }
    float acc = st.s * fast_exp2(st.m - cm);
#pragma unroll
    for (int e = 0; e < EPV; ++e) acc += fast_exp2(z[e] - cm);
    st.m = cm;
    st.s = acc;
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
  for (int c0 = kHeldFwdMaxVec; c0 < sp.nvec; c0 += THREADS * 2) {
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
        float cm = st.m;
#pragma unroll
        for (int e = 0; e < EPV; ++e) { z[e] *= kLog2e; cm = fmaxf(cm, z[e]); }
        float acc = st.s * fast_exp2(st.m - cm);
#pragma unroll
        for (int e = 0; e < EPV; ++e) acc += fast_exp2(z[e] - cm);
        st.m = cm;
        st.s = acc;
      }
    }
  }
  const MaxSum tot = block_merge<NW>(st, smem);
  // a row whose maximum is -inf has sum 0: 0 * inf = NaN, which is what torch returns
  const float inv = 1.f / tot.s;
#pragma unroll
  for (int i = 0; i < RI + LI; ++i) {
    const int c = i * THREADS + tid;
    if (c < sp.nvec) {
      float z[EPV], o[EPV];
      Elem<T>::unpack(vec(i), z);
#pragma unroll
      for (int e = 0; e < EPV; ++e) o[e] = fast_exp2(z[e] * kLog2e - tot.m) * inv;
      store16_stream(op + sp.head + (int64_t)c * EPV, Elem<T>::pack(o));
    }
  }
  for (int c0 = kHeldFwdMaxVec; c0 < sp.nvec; c0 += THREADS * 2) {
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
#pragma unroll
        for (int e = 0; e < EPV; ++e) o[e] = fast_exp2(z[e] * kLog2e - tot.m) * inv;
        store16_stream(op + sp.head + (int64_t)c * EPV, Elem<T>::pack(o));
      }
    }
  }
  if (edge_at >= 0) Elem<T>::store1(op + edge_at, fast_exp2(edge - tot.m) * inv);
}

template <typename T>
__global__ __launch_bounds__(kHeldBwdThreads) void softmax_bwd_held_kernel(const T* __restrict__ y,
                                                                            const T* __restrict__ dy,
                                                                            T* __restrict__ dx, int v) {
  constexpr int EPV = Elem<T>::kVec;
  constexpr int THREADS = kHeldBwdThreads, RI = kHeldBwdRegs, LI = kHeldBwdLds;
  constexpr int NW = THREADS / 64;
  extern __shared__ u32x4 parked[];          // [LI][2][THREADS]
  __shared__ float smem[NW];
  const int64_t row = blockIdx.x;
  const T* yp = y + row * (int64_t)v;
  const T* gp = dy + row * (int64_t)v;
  T* op = dx + row * (int64_t)v;
  const RowSplit sp = split_row<EPV>(row, v, true);
  const int tid = threadIdx.x;
  const int ne = edge_count(sp, v);
  u32x4 ry[RI], rg[RI];
#pragma unroll
  for (int i = 0; i < RI; ++i) {
    const int c = clamp_col(i * THREADS + tid, sp.nvec);
    ry[i] = load16_stream(yp + sp.head + (int64_t)c * EPV);
    rg[i] = load16_stream(gp + sp.head + (int64_t)c * EPV);
  }
#pragma unroll
  for (int j = 0; j < LI; j += 2) {
    u32x4 ly[2], lg[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int c = clamp_col((RI + j + u) * THREADS + tid, sp.nvec);
      ly[u] = load16_stream(yp + sp.head + (int64_t)c * EPV);
      lg[u] = load16_stream(gp + sp.head + (int64_t)c * EPV);
    }
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      parked[((j + u) * 2 + 0) * THREADS + tid] = ly[u];
      parked[((j + u) * 2 + 1) * THREADS + tid] = lg[u];
    }
  }
  float ey = 0.f, eg = 0.f;   // thread e keeps edge e of both rows
  int edge_at = -1;
  if (tid < ne) {
    edge_at = edge_col(sp, tid);
    ey = Elem<T>::load1(yp + edge_at);
    eg = Elem<T>::load1(gp + edge_at);
  }
  float dot = ey * eg;
#pragma unroll
  for (int i = 0; i < RI + LI; ++i) {
    if (i * THREADS + tid < sp.nvec) {
      u32x4 a4, b4;
      if (i < RI) {
        touch(ry[i < RI ? i : 0]);
        touch(rg[i < RI ? i : 0]);
        a4 = ry[i < RI ? i : 0]; b4 = rg[i < RI ? i : 0];
      } else {
        a4 = parked[((i - RI) * 2 + 0) * THREADS + tid]; b4 = parked[((i - RI) * 2 + 1) * THREADS + tid];
      }
      float a[EPV], b[EPV];
      Elem<T>::unpack(a4, a);
      Elem<T>::unpack(b4, b);
#pragma unroll
      for (int e = 0; e < EPV; ++e) dot += a[e] * b[e];
    }
  }
  // vector pairs past what the chip holds: streamed here, read again below
  for (int c0 = kHeldBwdMaxVec; c0 < sp.nvec; c0 += THREADS * 2) {
    u32x4 my[2], mg[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int c = clamp_col(c0 + u * THREADS + tid, sp.nvec);
      my[u] = load16(yp + sp.head + (int64_t)c * EPV);
      mg[u] = load16(gp + sp.head + (int64_t)c * EPV);
    }
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      touch(my[u]);
      if (c0 + u * THREADS + tid < sp.nvec) {
        float a[EPV], b[EPV];
        Elem<T>::unpack(my[u], a);
        Elem<T>::unpack(mg[u], b);
#pragma unroll
        for (int e = 0; e < EPV; ++e) dot += a[e] * b[e];
      }
    }
  }
  dot = row_reduce<THREADS, OpSum>(dot, smem, 0, tid);
#pragma unroll
  for (int i = 0; i < RI + LI; ++i) {
    const int c = i * THREADS + tid;
    if (c < sp.nvec) {
      u32x4 a4, b4;
      if (i < RI) {
        touch(ry[i < RI ? i : 0]);
        touch(rg[i < RI ? i : 0]);
        a4 = ry[i < RI ? i : 0]; b4 = rg[i < RI ? i : 0];
      } else {
        a4 = parked[((i - RI) * 2 + 0) * THREADS + tid]; b4 = parked[((i - RI) * 2 + 1) * THREADS + tid];
      }
      float a[EPV], b[EPV], o[EPV];
      Elem<T>::unpack(a4, a);
      Elem<T>::unpack(b4, b);
#pragma unroll
      for (int e = 0; e < EPV; ++e) o[e] = (b[e] - dot) * a[e];
      store16_stream(op + sp.head + (int64_t)c * EPV, Elem<T>::pack(o));
    }
  }
  for (int c0 = kHeldBwdMaxVec; c0 < sp.nvec; c0 += THREADS * 2) {
    u32x4 my[2], mg[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int c = clamp_col(c0 + u * THREADS + tid, sp.nvec);
      my[u] = load16_stream(yp + sp.head + (int64_t)c * EPV);
      mg[u] = load16_stream(gp + sp.head + (int64_t)c * EPV);
    }
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int c = c0 + u * THREADS + tid;
      touch(my[u]);
      if (c < sp.nvec) {
        float a[EPV], b[EPV], o[EPV];
        Elem<T>::unpack(my[u], a);
        Elem<T>::unpack(mg[u], b);
#pragma unroll
        for (int e = 0; e < EPV; ++e) o[e] = (b[e] - dot) * a[e];
        store16_stream(op + sp.head + (int64_t)c * EPV, Elem<T>::pack(o));
      }
    }
  }
  if (edge_at >= 0) Elem<T>::store1(op + edge_at, (eg - dot) * ey);
}

// four elements a lane for the narrowest rows, so that rows of a few elements do not idle
// most of a 16-lane group
void scalar_plan(int v, int* tpr, int* iters) {
  int t = 1;
  while (t < 16 && 4 * t < v) t *= 2;
  if (v > 16 * 16) t = 64;
  int it = 1;
  while (t * it < v) it *= 2;
  if (t >= 16 && it < 4) it = 4;      // the instantiated shapes
  *tpr = t;
  *iters = it;
}

template <typename T>
void launch(const void* x, void* y, int64_t n, int v, bool vec_ok, hipStream_t st) {
  const T* xp = static_cast<const T*>(x);
  T* yp = static_cast<T*>(y);
  constexpr int EPV = Elem<T>::kVec;
  int tpr = 0, iters = 0;
  if (vec_ok && v % EPV == 0 && rows_plan(v / EPV, &tpr, &iters)) {
#define X(TPR_, IT_)                                                                               \
  if (tpr == TPR_ && iters == IT_) {                                                               \
    constexpr int RPB = RowBlock<TPR_>::value / TPR_;                                              \
    FM_LAUNCH((softmax_rows_kernel<T, TPR_, IT_>), dim3((unsigned)((n + RPB - 1) / RPB)), \
                       dim3(RowBlock<TPR_>::value), 0, st, xp, yp, n, v);                          \
    return;                                                                                        \
  }
    FM_SOFTMAX_SHAPES(X)
#undef X
  }
  if (v <= 64 * 16) {   // narrow, not vectorisable: lane groups with one element per load
    int tpr, iters;
    scalar_plan(v, &tpr, &iters);
    const dim3 sgrid((unsigned)((n + 256 / tpr - 1) / (256 / tpr)));
#define GOS(TPR_, IT_)                                                                             \
  if (tpr == TPR_ && iters == IT_) {                                                               \
    FM_LAUNCH((softmax_rows_scalar_kernel<T, TPR_, IT_>), sgrid, dim3(256), 0, st, xp, yp, n, v); \
    return;                                                                                        \
  }
    GOS(1, 1) GOS(1, 2) GOS(1, 4) GOS(2, 4) GOS(4, 4) GOS(8, 4)
    GOS(16, 4) GOS(16, 8) GOS(16, 16) GOS(64, 8) GOS(64, 16)
#undef GOS
  }
  // (from 8192 vectors on: below that the streaming form, several rows a compute unit, is as fast
  // or faster -- bf16 [5120,50257] 218 against 229 us, [3840,65544] 218 against 211)
  if (vec_ok && v / EPV <= 2 * kHeldFwdMaxVec && v / EPV >= 8192 &&
      fm_host::grant_dynamic_lds<&softmax_held_kernel<T>>(kHeldFwdLds * kHeldFwdThreads * 16)) {
    FM_LAUNCH((softmax_held_kernel<T>), dim3((unsigned)n), dim3(kHeldFwdThreads),
              (size_t)kHeldFwdLds * kHeldFwdThreads * 16, st, xp, yp, v);
    return;
  }
  const fm_host::VocabShape sh = fm_host::vocab_shape(v, sizeof(T), 1024, 4);
  const dim3 grid((unsigned)n);
#define LAUNCH(TH, UN) \
  FM_LAUNCH((softmax_kernel<T, TH, UN>), grid, dim3(TH), 0, st, xp, yp, v, vec_ok)
  FM_VOCAB_DISPATCH(sh, LAUNCH);
#undef LAUNCH
}

template <typename T>
void launch_bwd(const void* y, const void* dy, void* dx, int64_t n, int v, bool vec_ok, hipStream_t st) {
  const T* yp = static_cast<const T*>(y);
  const T* gp = static_cast<const T*>(dy);
  T* op = static_cast<T*>(dx);
  constexpr int EPV = Elem<T>::kVec;
  int tpr = 0, iters = 0;
  // two packed rows in registers, on the plans of the forward; half types stop at 64 KiB rows
  // (their unpacked copies would not fit the 128 registers of a 1024-thread workgroup)
  if (vec_ok && v % EPV == 0 && v / EPV <= (sizeof(T) == 4 ? 8192 : 4096) &&
      rows_plan(v / EPV, &tpr, &iters)) {
#define X(TPR_, IT_)                                                                               \
  if (tpr == TPR_ && iters == IT_) {                                                               \
    constexpr int RPB = RowBlock<TPR_>::value / TPR_;                                              \
    FM_LAUNCH((softmax_bwd_rows_kernel<T, TPR_, IT_>), dim3((unsigned)((n + RPB - 1) / RPB)), \
                       dim3(RowBlock<TPR_>::value), 0, st, yp, gp, op, n, v);                      \
    return;                                                                                        \
  }
    FM_SOFTMAX_SHAPES(X)
#undef X
  }
  if (v <= 64 * 16) {
    int tpr, iters;
    scalar_plan(v, &tpr, &iters);
    const dim3 sgrid((unsigned)((n + 256 / tpr - 1) / (256 / tpr)));
#define GOS(TPR_, IT_)                                                                             \
  if (tpr == TPR_ && iters == IT_) {                                                               \
    FM_LAUNCH((softmax_bwd_rows_scalar_kernel<T, TPR_, IT_>), sgrid, dim3(256), 0, st, yp, gp, op, n, v); \
    return;                                                                                        \
  }
    GOS(1, 1) GOS(1, 2) GOS(1, 4) GOS(2, 4) GOS(4, 4) GOS(8, 4)
    GOS(16, 4) GOS(16, 8) GOS(16, 16) GOS(64, 8) GOS(64, 16)
#undef GOS
  }
  // (16-bit rows only when they fill most of what the chip holds: bf16 [2560,100000] 373 us streamed
  // against 386 held, [2048,128256] 388 against 352; fp32 [3328,40000] 376 against 274)
  if (vec_ok && v / EPV <= 2 * kHeldBwdMaxVec && v / EPV >= 8192 &&
      fm_host::grant_dynamic_lds<&softmax_bwd_held_kernel<T>>(kHeldBwdLds * 2 * kHeldBwdThreads * 16)) {
    FM_LAUNCH((softmax_bwd_held_kernel<T>), dim3((unsigned)n), dim3(kHeldBwdThreads),
              (size_t)kHeldBwdLds * 2 * kHeldBwdThreads * 16, st, yp, gp, op, v);
    return;
  }
  const fm_host::VocabShape sh = fm_host::vocab_shape(v, sizeof(T), 1024, 4);
  const dim3 grid((unsigned)n);
#define LAUNCH(TH, UN) \
  FM_LAUNCH((softmax_bwd_kernel<T, TH, UN>), grid, dim3(TH), 0, st, yp, gp, op, v, vec_ok)
  FM_VOCAB_DISPATCH(sh, LAUNCH);
#undef LAUNCH
}

}  // namespace

extern "C" int fm_softmax_fwd(const void* x, void* y, int64_t n, int64_t v, int dtype,
                              fm_stream_t stream) {
  FM_CHECK_ARG(n >= 0 && v > 0, "fm_softmax_fwd: bad shape n=%lld v=%lld", (long long)n, (long long)v);
  FM_CHECK_ARG(dtype == FM_F32 || dtype == FM_F16 || dtype == FM_BF16, "fm_softmax_fwd: bad dtype %d",
               dtype);
  if (n > 0x7fffffffLL || v > 0x7fffffffLL) {
    fm_host::set_error("fm_softmax_fwd: n and v must be below 2^31");
    return FM_ERR_UNSUPPORTED;
  }
  if (n == 0) return FM_OK;
  FM_CHECK_ARG(x && y, "fm_softmax_fwd: NULL pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool vec_ok = fm_host::aligned16(x) && fm_host::aligned16(y);
  if (dtype == FM_F32) launch<float>(x, y, n, (int)v, vec_ok, st);
  else if (dtype == FM_BF16) launch<bf16_t>(x, y, n, (int)v, vec_ok, st);
  else launch<f16_t>(x, y, n, (int)v, vec_ok, st);
  FM_CHECK_LAUNCH("fm_softmax_fwd");
  return FM_OK;
}

extern "C" int fm_softmax_bwd(const void* y, const void* dy, void* dx, int64_t n, int64_t v, int dtype,
                              fm_stream_t stream) {
  FM_CHECK_ARG(n >= 0 && v > 0, "fm_softmax_bwd: bad shape n=%lld v=%lld", (long long)n, (long long)v);
  FM_CHECK_ARG(dtype == FM_F32 || dtype == FM_F16 || dtype == FM_BF16, "fm_softmax_bwd: bad dtype %d",
               dtype);
  if (n > 0x7fffffffLL || v > 0x7fffffffLL) {
    fm_host::set_error("fm_softmax_bwd: n and v must be below 2^31");
    return FM_ERR_UNSUPPORTED;
  }
  if (n == 0) return FM_OK;
  FM_CHECK_ARG(y && dy && dx, "fm_softmax_bwd: NULL pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool vec_ok = fm_host::aligned16(y) && fm_host::aligned16(dy) && fm_host::aligned16(dx);
  if (dtype == FM_F32) launch_bwd<float>(y, dy, dx, n, (int)v, vec_ok, st);
  else if (dtype == FM_BF16) launch_bwd<bf16_t>(y, dy, dx, n, (int)v, vec_ok, st);
  else launch_bwd<f16_t>(y, dy, dx, n, (int)v, vec_ok, st);
  FM_CHECK_LAUNCH("fm_softmax_bwd");
  return FM_OK;
}
