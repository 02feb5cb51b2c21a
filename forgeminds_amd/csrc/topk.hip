// Exact, deterministic top-k over the last dimension for gfx950.
//
// Reference semantics: forgemind/kernels/topk.py:13-19, 273-297 -- output sorted by value
// descending, index ascending inside ties; at the k-th value the smallest indices win; NaN is
// the largest value and the original NaN is what lands in `values`; -0.0 ties with +0.0.
//
// One workgroup per row, one streaming read of the row from HBM:
//   A  every thread folds each 16-byte vector it reads to one maximum and keeps those vector
//      maxima (not the data) in registers; their maximum is the thread's "group maximum";
//   T  each wave finds the ceil(k / waves)-th largest of its 64 group maxima with a ballot
//      search; the minimum over the waves, tau, can never be above the true k-th value,
//      because at least k group maxima are >= tau;
//   B  only vectors whose maximum is >= tau can hold candidates -- a few hundred out of
//      16k -- so their indices go to a work list, the workgroup re-reads just those vectors
//      (one parallel round trip, served by cache) and every element >= tau becomes a
//      candidate (key, index) in LDS; candidates are ranked by counting how many others beat
//      them under (key descending, index ascending); rank r < k is output slot r.
// Keeping maxima instead of the row keeps the kernel at 64 registers, so two 1024-thread
// workgroups share a compute unit and one streams while the other selects.
// Rows with too many candidates (long runs of equal values) take an exact path instead: a
// bitwise search for the k-th key over the whole row, then an index-ordered scan that admits
// the first (k - #greater) ties. Rows wider than the register budget make two full passes.
// Keys are order-preserving integer images of the fp32 value, so no float is ever summed and
// the result is bit-reproducible.
#include "fm_vocab.cuh"

using namespace fm;

namespace {

constexpr int kCap = 1024;  // candidate slots in LDS
constexpr int kMaxK = 512;

__device__ __forceinline__ uint32_t key_of(float f) {
  if (f != f) return 0xFFFFFFFFu;          // every NaN ties at the top
  f = f + 0.0f;                            // -0.0 -> +0.0, so the two zeros tie
  const uint32_t b = __builtin_bit_cast(uint32_t, f);
  return b ^ ((uint32_t)((int32_t)b >> 31) | 0x80000000u);
}
__device__ __forceinline__ float float_of_key(uint32_t k) {
  const uint32_t b = (k & 0x80000000u) ? (k ^ 0x80000000u) : ~k;
  return __builtin_bit_cast(float, b);
}

__device__ __forceinline__ int block_sum_int(int v, int* smem, int nw) {
  v = wave_sum_i(v);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) smem[wave] = v;
  __syncthreads();
  int s = 0;
  for (int i = 0; i < nw; ++i) s += smem[i];
  __syncthreads();
  return s;
}

// Exclusive scan of a small per-thread count in thread order; *total gets the block sum.
__device__ __forceinline__ int block_excl_scan(int v, int* smem, int nw, int* total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int inc = v;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int t = __shfl_up(inc, o, 64);
    if (lane >= o) inc += t;
  }
  if (lane == 63) smem[wave] = inc;
  __syncthreads();
  int before = 0, tot = 0;
  for (int i = 0; i < nw; ++i) {
    const int w = smem[i];
    if (i < wave) before += w;
    tot += w;
  }
  __syncthreads();
  *total = tot;
  return before + inc - v;
}

constexpr int kWorkCap = 2048;  // vectors that may be revisited in phase B

template <typename T, int THREADS, int ITERS>
__global__ __launch_bounds__(THREADS, (ITERS > 0 && ITERS <= 16 && THREADS == 1024) ? 8 : 1)
void topk_kernel(const T* __restrict__ x, T* __restrict__ values, int32_t* __restrict__ idx32,
                 int64_t* __restrict__ idx64, int v, int k, bool vec_ok) {
  constexpr int EPV = Elem<T>::kVec;
  constexpr int NW = THREADS / 64;
  constexpr bool VMAX = ITERS > 0;   // vector maxima live in registers
  constexpr uint32_t KMASK = sizeof(T) == 2 ? 0xFFFF0000u : 0xFFFFFFFFu;
  __shared__ unsigned long long ccomp[kCap];  // (key << 32) | ~index : larger is better
  __shared__ int crank[kCap];
  __shared__ int work[VMAX ? kWorkCap : 1];
  __shared__ int s_int[NW];
  __shared__ uint32_t s_tau[NW];
  __shared__ int s_count, s_nwork;

  const int64_t row = blockIdx.x;
  const T* rp = x + row * (int64_t)v;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const RowSplit sp = split_row<EPV>(row, v, vec_ok);
  const int ne = edge_count(sp, v);
  float vmax[VMAX ? ITERS : 1];

  // maximum of one vector; NaN if the vector holds a NaN (NaN outranks everything)
  auto fold = [&](const u32x4& raw) {
    float f[EPV];
    Elem<T>::unpack(raw, f);
    float m = f[0];
    bool bad = f[0] != f[0];
#pragma unroll
    for (int e = 1; e < EPV; ++e) { m = fmaxf(m, f[e]); bad |= (f[e] != f[e]); }
    return bad ? __builtin_nanf("") : m;
  };

  int C = 0;
  bool overflow = false;
  if (v <= kCap) {
    // short row: every element is a candidate
    for (int j = tid; j < v; j += THREADS)
      ccomp[j] = ((unsigned long long)key_of(Elem<T>::load1(rp + j)) << 32) | (uint32_t)(~j);
    C = v;
    __syncthreads();
  } else {
    // ---- phase A: vector maxima and the thread's group maximum
    float fm = -INFINITY;
    bool has_nan = false;
    if constexpr (VMAX) {
#pragma unroll
      for (int i0 = 0; i0 < ITERS; i0 += 4) {
        u32x4 raw[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int c = (i0 + u) * THREADS + tid;
          if (c < sp.nvec) raw[u] = load16_stream(rp + sp.head + (int64_t)c * EPV);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int c = (i0 + u) * THREADS + tid;
          float m = -INFINITY;
          if (c < sp.nvec) m = fold(raw[u]);
          vmax[i0 + u] = m;
          fm = fmaxf(fm, m);
          has_nan |= (m != m);
        }
      }
    } else {
      for (int c = tid; c < sp.nvec; c += THREADS) {
        const float m = fold(load16(rp + sp.head + (int64_t)c * EPV));
        fm = fmaxf(fm, m);
        has_nan |= (m != m);
      }
    }
    for (int e = tid; e < ne; e += THREADS) {
      const float f = Elem<T>::load1(rp + edge_col(sp, e));
      fm = fmaxf(fm, f);
      has_nan |= (f != f);
    }
    const bool has = tid < sp.nvec || tid < ne;
    const uint32_t mykey = !has ? 0u : (has_nan ? 0xFFFFFFFFu : key_of(fm));

    // ---- phase T: per-wave j-th largest group maximum, then the minimum over waves
    const int j = (k + NW - 1) / NW;
    uint32_t tw = 0u;
    if (j <= 64) {
      for (int bit = 31; bit >= 0; --bit) {
        const uint32_t trial = tw | (1u << bit);
        const int cnt = __builtin_popcountll(__ballot(mykey >= trial));
        if (cnt >= j) tw = trial;
      }
    }
    if (lane == 0) s_tau[wave] = tw;
    if (tid == 0) { s_count = 0; s_nwork = 0; }
    __syncthreads();
    uint32_t tau = s_tau[0];
#pragma unroll
    for (int i = 1; i < NW; ++i) tau = tau < s_tau[i] ? tau : s_tau[i];
    // float image of tau; keys at or below key(-inf) admit everything, the NaN key only NaNs
    const float tau_f = tau <= 0x007FFFFFu ? -INFINITY
                                           : (tau == 0xFFFFFFFFu ? __builtin_nanf("") : float_of_key(tau));
    const bool only_nan = tau == 0xFFFFFFFFu;
    auto take_of = [&](float f) { return only_nan ? (f != f) : !(f < tau_f); };

    // ---- phase B: candidates
    auto consider = [&](float f, int col) {
      if (take_of(f)) {
        const int slot = atomicAdd(&s_count, 1);
        if (slot < kCap) ccomp[slot] = ((unsigned long long)key_of(f) << 32) | (uint32_t)(~col);
      }
    };
    auto scan_vec = [&](const u32x4& raw, int c) {
      float f[EPV];
      Elem<T>::unpack(raw, f);
      bool any = false;
#pragma unroll
      for (int e = 0; e < EPV; ++e) any |= take_of(f[e]);
      if (any) {
#pragma unroll
        for (int e = 0; e < EPV; ++e) consider(f[e], sp.head + c * EPV + e);
      }
    };
    if constexpr (VMAX) {
      // B1: vectors that can hold a candidate go to the work list
#pragma unroll
      for (int i = 0; i < ITERS; ++i) {
        const int c = i * THREADS + tid;
        if (c < sp.nvec && take_of(vmax[i])) {
          const int slot = atomicAdd(&s_nwork, 1);
          if (slot < kWorkCap) work[slot] = c;
        }
      }
      __syncthreads();
      const int nwork = s_nwork;
      overflow = nwork > kWorkCap;
      // B2: revisit only those vectors, spread over the whole workgroup
      if (!overflow) {
        for (int w = tid; w < nwork; w += THREADS) {
          const int c = work[w];
          scan_vec(load16(rp + sp.head + (int64_t)c * EPV), c);
        }
      }
    } else {
      for (int c = tid; c < sp.nvec; c += THREADS) scan_vec(load16(rp + sp.head + (int64_t)c * EPV), c);
    }
    for (int e = tid; e < ne; e += THREADS) {
      const int col = edge_col(sp, e);
      consider(Elem<T>::load1(rp + col), col);
    }
    __syncthreads();
    C = s_count;
    __syncthreads();
    if (overflow) C = kCap + 1;

    if (C > kCap) {
      // ---- exact path: k-th key by bitwise search over the whole row
      auto count_if = [&](auto pred) {
        int cnt = 0;
        for (int c = tid; c < sp.nvec; c += THREADS) {
          float f[EPV];
          Elem<T>::unpack(load16(rp + sp.head + (int64_t)c * EPV), f);
#pragma unroll
          for (int e = 0; e < EPV; ++e) cnt += pred(key_of(f[e]) & KMASK) ? 1 : 0;
        }
        for (int e = tid; e < ne; e += THREADS)
          cnt += pred(key_of(Elem<T>::load1(rp + edge_col(sp, e))) & KMASK) ? 1 : 0;
        return block_sum_int(cnt, s_int, NW);
      };
      uint32_t kth = 0u;
      for (int bit = 31; bit >= (sizeof(T) == 2 ? 16 : 0); --bit) {
        const uint32_t trial = kth | (1u << bit);
        const int cnt = count_if([&](uint32_t key) { return key >= trial; });
        if (cnt >= k) kth = trial;
      }
      const int c_gt = count_if([&](uint32_t key) { return key > kth; });
      const int need = k - c_gt;  // ties admitted, in ascending index order
      if (tid == 0) s_count = 0;
      __syncthreads();
      // strictly greater: any slot (they are ranked afterwards); ties: index-ordered scan
      int base = 0;  // ties admitted so far (uniform)
      auto emit_gt = [&](float f, int col) {
        const uint32_t key = key_of(f);
        if ((key & KMASK) > kth) {
          const int slot = atomicAdd(&s_count, 1);
          ccomp[slot] = ((unsigned long long)key << 32) | (uint32_t)(~col);
        }
      };
      // columns are visited in ascending order: head edge, vectors by iteration, tail edge
      {
        int mine = 0;
        float f0 = 0.f;
        const int col = tid;
        if (tid < sp.head) {
          f0 = Elem<T>::load1(rp + col);
          emit_gt(f0, col);
          mine = ((key_of(f0) & KMASK) == kth) ? 1 : 0;
        }
        int tot;
        const int ex = block_excl_scan(mine, s_int, NW, &tot);
        if (mine && base + ex < need)
          ccomp[c_gt + base + ex] = ((unsigned long long)key_of(f0) << 32) | (uint32_t)(~col);
        base += tot;
      }
      const int niter = (sp.nvec + THREADS - 1) / THREADS;
      for (int i = 0; i < niter; ++i) {
        const int c = i * THREADS + tid;
        float f[EPV];
        int mine = 0;
        if (c < sp.nvec) {
          Elem<T>::unpack(load16(rp + sp.head + (int64_t)c * EPV), f);
#pragma unroll
          for (int e = 0; e < EPV; ++e) {
            emit_gt(f[e], sp.head + c * EPV + e);
            mine += ((key_of(f[e]) & KMASK) == kth) ? 1 : 0;
          }
        }
        int tot;
        int pos = base + block_excl_scan(mine, s_int, NW, &tot);
        if (mine && pos < need) {
#pragma unroll
          for (int e = 0; e < EPV; ++e) {
            if ((key_of(f[e]) & KMASK) == kth) {
              if (pos < need)
                ccomp[c_gt + pos] = ((unsigned long long)key_of(f[e]) << 32) | (uint32_t)(~(sp.head + c * EPV + e));
              ++pos;
            }
          }
        }
        base += tot;
      }
      {
        // tail edge (and, when vectors are off, the whole row): ascending columns per step
        const int ntail = v - sp.tail0;
        for (int t0 = 0; t0 < ntail; t0 += THREADS) {
          const int col = sp.tail0 + t0 + tid;
          int mine = 0;
          float f0 = 0.f;
          if (col < v) {
            f0 = Elem<T>::load1(rp + col);
            emit_gt(f0, col);
            mine = ((key_of(f0) & KMASK) == kth) ? 1 : 0;
          }
          int tot;
          const int ex = block_excl_scan(mine, s_int, NW, &tot);
          if (mine && base + ex < need)
            ccomp[c_gt + base + ex] = ((unsigned long long)key_of(f0) << 32) | (uint32_t)(~col);
          base += tot;
        }
      }
      __syncthreads();
      C = k;
    }
  }

  // ---- rank the C candidates by counting; rank r < k goes to output slot r
  int cpad = 64;
  while (cpad < C) cpad <<= 1;
  const int parts = THREADS / cpad > 1 ? THREADS / cpad : 1;
  for (int jx = tid; jx < C; jx += THREADS) crank[jx] = 0;
  __syncthreads();
  const int per = (C + parts - 1) / parts;
  for (int wk = tid; wk < cpad * parts; wk += THREADS) {
    const int jx = wk % cpad, part = wk / cpad;
    if (jx < C) {
      const unsigned long long me = ccomp[jx];
      const int i0 = part * per;
      const int i1 = i0 + per < C ? i0 + per : C;
      int r = 0;
      for (int i = i0; i < i1; ++i) r += ccomp[i] > me ? 1 : 0;
      if (parts == 1) crank[jx] = r; else atomicAdd(&crank[jx], r);
    }
  }
  __syncthreads();
  for (int jx = tid; jx < C; jx += THREADS) {
    const int r = crank[jx];
    if (r < k) {
      const int col = (int)(~(uint32_t)(ccomp[jx] & 0xFFFFFFFFull));
      const int64_t o = row * (int64_t)k + r;
      if (idx32 != nullptr) idx32[o] = col;
      if (idx64 != nullptr) idx64[o] = col;
      if (values != nullptr) values[o] = rp[col];
    }
  }
}

template <typename T>
int launch(const void* x, void* values, void* indices, int64_t n, int v, int k, int index_bits,
           bool vec_ok, hipStream_t st) {
  const T* xp = static_cast<const T*>(x);
  T* vp = static_cast<T*>(values);
  int32_t* i32 = index_bits == 32 ? static_cast<int32_t*>(indices) : nullptr;
  int64_t* i64 = index_bits == 64 ? static_cast<int64_t*>(indices) : nullptr;
  constexpr int EPV = Elem<T>::kVec;
  const int64_t nvec = (v + EPV - 1) / EPV + 1;  // upper bound on whole vectors of any row
  const dim3 grid((unsigned)n);
#define GO(TH, IT)                                                                               \
  hipLaunchKernelGGL((topk_kernel<T, TH, IT>), grid, dim3(TH), 0, st, xp, vp, i32, i64, v, k, vec_ok)
  const int variant = fm_host::get_param(fm_host::P_TOPK_VARIANT);
  if (variant == 1 && v > kCap) GO(1024, 0);
  else if (v <= kCap || nvec <= 256 * 4) GO(256, 4);
  else if (nvec <= 1024 * 4) GO(1024, 4);
  else if (nvec <= 1024 * 16) GO(1024, 16);
  else if (nvec <= 1024 * 32) GO(1024, 32);
  else GO(1024, 0);
#undef GO
  return FM_OK;
}

}  // namespace

extern "C" int fm_topk(const void* x, void* values, void* indices, int64_t n, int64_t v, int k,
                       int dtype, int index_bits, fm_stream_t stream) {
  FM_CHECK_ARG(n >= 0 && v > 0, "fm_topk: bad shape n=%lld v=%lld", (long long)n, (long long)v);
  FM_CHECK_ARG(dtype == FM_F32 || dtype == FM_F16 || dtype == FM_BF16, "fm_topk: bad dtype %d", dtype);
  FM_CHECK_ARG(index_bits == 32 || index_bits == 64, "fm_topk: index_bits must be 32 or 64");
  FM_CHECK_ARG(k >= 1 && k <= v, "fm_topk: selected index k out of range (got %d vs %lld)", k,
               (long long)v);
  if (k > kMaxK || n > 0x7fffffffLL || v > 0x7fffffffLL) {
    fm_host::set_error("fm_topk: k <= %d and n, v < 2^31 required (k=%d)", kMaxK, k);
    return FM_ERR_UNSUPPORTED;
  }
  if (n == 0) return FM_OK;
  FM_CHECK_ARG(x && indices, "fm_topk: NULL pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool vec_ok = fm_host::aligned16(x);
  if (dtype == FM_F32) launch<float>(x, values, indices, n, (int)v, k, index_bits, vec_ok, st);
  else if (dtype == FM_BF16) launch<bf16_t>(x, values, indices, n, (int)v, k, index_bits, vec_ok, st);
  else launch<f16_t>(x, values, indices, n, (int)v, k, index_bits, vec_ok, st);
  FM_CHECK_LAUNCH("fm_topk");
  return FM_OK;
}
