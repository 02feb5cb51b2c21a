// Exact, deterministic top-k over the last dimension for gfx950.
//
// Reference semantics: forgemind/kernels/topk.py:13-19, 273-297 -- output sorted by value
// descending, index ascending inside ties; at the k-th value the smallest indices win; NaN is
// the largest value and the original NaN is what lands in `values`; -0.0 ties with +0.0.
//
// One workgroup per row, one streaming read of the row from HBM:
//   A  every thread folds each 16-byte vector it reads to one maximum and leaves a 16-bit
//      prefix of that maximum's key in LDS (2 bytes per 16 bytes of row); the maximum over
//      its vectors is the thread's "group maximum". Rows are never unpacked to fp32 for
//      this: packed 16-bit integer instructions turn two bf16 / fp16 elements at a time into
//      16-bit keys, three integer instructions an fp32 element into a 32-bit key (about 20
//      instructions per vector instead of 70 / 40; the pass is otherwise bound by instruction
//      issue as much as by the read);
//   T  each full wave finds the ceil(k / waves)-th largest of its 64 group maxima with a
//      ballot search; the minimum over the waves, tau, can never be above the true k-th
//      value, because at least k group maxima are >= tau;
//   B  only vectors whose prefix reaches tau's can hold candidates -- a few hundred out of
//      16k -- so their indices go to a work list, the workgroup re-reads just those vectors
//      (one parallel round trip, served by cache) and every element >= tau becomes a
//      candidate (key, index) in LDS; candidates are ranked by counting how many others beat
//      them under (key descending, index ascending); rank r < k is output slot r.
// Keeping prefixes instead of the row keeps registers and LDS small, so several workgroups
// share a compute unit and one streams while another selects.
// Rows with too many candidates (long runs of equal values) take an exact path instead: a
// bitwise search for the k-th key over the whole row, then an index-ordered scan that admits
// the first (k - #greater) ties. Rows wider than the LDS budget keep the vector maxima in
// registers (up to 32 per thread) or make two full passes.
// Keys are order-preserving integer images of the fp32 value, so no float is ever summed and
// the result is bit-reproducible.
#include <type_traits>

#include "fm_topk.hip.h"

using namespace fm;

namespace {

template <typename T, int THREADS, int ITERS, int BIG>
__global__ __launch_bounds__(THREADS, (ITERS > 0 && ITERS <= 16 && THREADS == 1024) ? 8 : 1)
void topk_kernel(const T* __restrict__ x, T* __restrict__ values, int32_t* __restrict__ idx32,
                 int64_t* __restrict__ idx64, int v, int k, bool vec_ok) {
  constexpr int EPV = Elem<T>::kVec;
  constexpr bool VMAX = ITERS > 0;   // vector maxima live in registers
  constexpr int NV = VMAX ? ITERS : 1;
  __shared__ TopkShared<THREADS, VMAX ? kVecMaxRegs : kVecMaxNone, BIG> sh;

  const int64_t row = blockIdx.x;
  const T* rp = x + row * (int64_t)v;
  const int tid = threadIdx.x;
  const RowSplit sp = split_row<EPV>(row, v, vec_ok);
  const int ne = edge_count(sp, v);
  float vmax[NV];
  float fm = -INFINITY;
  bool has_nan = false;
  if (v > TopkShared<THREADS, VMAX ? kVecMaxRegs : kVecMaxNone, BIG>::kSlots) {
    // ---- phase A: vector maxima and the thread's group maximum
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
          if (c < sp.nvec) m = fold_vector_max<T>(raw[u]);
          vmax[i0 + u] = m;
          fm = fmaxf(fm, m);
          has_nan |= (m != m);
        }
      }
    } else {
      vmax[0] = 0.f;
      for (int c = tid; c < sp.nvec; c += THREADS) {
        const float m = fold_vector_max<T>(load16(rp + sp.head + (int64_t)c * EPV));
        fm = fmaxf(fm, m);
        has_nan |= (m != m);
      }
    }
    for (int e = tid; e < ne; e += THREADS) {
      const float f = Elem<T>::load1(rp + edge_col(sp, e));
      fm = fmaxf(fm, f);
      has_nan |= (f != f);
    }
  } else {
#pragma unroll
    for (int i = 0; i < NV; ++i) vmax[i] = 0.f;
  }
  topk_finish<T, THREADS, NV, VMAX ? kVecMaxRegs : kVecMaxNone, BIG>(rp, sp, v, k, vmax, nullptr, fm, has_nan, sh,
                                                                row, values, idx32, idx64, nullptr, 0.f, 0.f);
}

// Variant that leaves a 16-bit key prefix of every vector's maximum in LDS instead of the
// maxima in registers: few registers, so several workgroups share a compute unit and one
// row's selection overlaps the next row's streaming read.
template <typename T, int THREADS, int UNROLL, int BIG>
__global__ __launch_bounds__(THREADS, THREADS >= 256 ? 8 : 1) void topk_lds_kernel(const T* __restrict__ x, T* __restrict__ values,
                                                           int32_t* __restrict__ idx32,
                                                           int64_t* __restrict__ idx64, int v, int k,
                                                           bool vec_ok) {
  constexpr int EPV = Elem<T>::kVec;
  constexpr bool SK = SKey<T>::ok;   // bf16 / fp16: vhi holds 16-bit stream keys
  constexpr bool SK32 = Elem<T>::kDtype == FM_F32;   // fp32: prefixes of 32-bit stream keys
  __shared__ TopkShared<THREADS, kVecMaxLds, BIG> sh;
  extern __shared__ __align__(16) uint16_t vhi[];
  const int64_t row = blockIdx.x;
  const T* rp = x + row * (int64_t)v;
  const int tid = threadIdx.x;
  const RowSplit sp = split_row<EPV>(row, v, vec_ok);
  float fm = -INFINITY;
  bool has_nan = false;
  if (v > TopkShared<THREADS, kVecMaxLds, BIG>::kSlots) {
    {  // zero the padding of the last quad of prefixes
      const int p = ((sp.nvec + 3) & ~3) - 1 - tid;
      if (tid < 3 && p >= sp.nvec) vhi[p] = 0;
    }
    // Integer stream keys, no unpacking to fp32: bf16 / fp16 two elements at a time with packed
    // 16-bit instructions (the LDS keeps the vector's key), fp32 three instructions an element
    // (the LDS keeps the upper half of the vector's key, rounded up).
    static_assert(SK || SK32, "rows are bf16, fp16 or fp32");
    uint32_t sm = 0u;   // the key of -inf
    auto tile = [&](int c0, auto full) {
      u32x4 raw[UNROLL];
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const int c = decltype(full)::value ? c0 + u * THREADS + tid : clamp_col(c0 + u * THREADS + tid, sp.nvec);
        raw[u] = load16_stream(rp + sp.head + (int64_t)c * EPV);
      }
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const int c = c0 + u * THREADS + tid;
        if (decltype(full)::value || c < sp.nvec) {
          uint32_t m;
          if constexpr (SK) {
            m = skey_vector_max<T>(raw[u]);
            vhi[c] = (uint16_t)m;
          } else {
            m = skey32_vector_max(raw[u]);
            vhi[c] = (uint16_t)skey32_prefix(m);
          }
          sm = m > sm ? m : sm;
        }
      }
    };
    int c0 = 0;
    for (; c0 + THREADS * UNROLL <= sp.nvec; c0 += THREADS * UNROLL) tile(c0, std::true_type{});
    if (c0 < sp.nvec) tile(c0, std::false_type{});
    if constexpr (SK) {
      if (sm > SKeyC<T>::kNanAbove) has_nan = true;
      else fm = float_of_skey<T>(sm);
    } else {
      if (sm > kSKey32NanAbove) has_nan = true;
      else fm = float_of_skey32(sm);
    }
    const int ne = edge_count(sp, v);
    for (int e = tid; e < ne; e += THREADS) {
      const float f = Elem<T>::load1(rp + edge_col(sp, e));
      fm = fmaxf(fm, f);
      has_nan |= (f != f);
    }
  }
  const float none[1] = {0.f};
  topk_finish<T, THREADS, 1, kVecMaxLds, BIG, SK ? kVhiStream16 : (SK32 ? kVhiStream32 : kVhiPrefix)>(rp, sp, v, k, none, vhi, fm, has_nan, sh, row, values, idx32,
                                                  idx64, nullptr, 0.f, 0.f);
}

// Rows of up to 2048 elements: one wave per row (a 64-thread workgroup each), the whole row as
// keys in registers (EPL per lane; 16-byte loads when the rows are aligned, else lane-strided
// scalars). No step depends on the order of the registers:
//   1. tau = the k-th largest of the lanes' group maxima (ballot search, one to four compares a
//      bit) -- at least k elements reach it;
//   2. elements >= tau become candidates (key, kWaveMaxV - column) in LDS; when at most
//      64 exist each lane takes one and they are ranked by counting, which ends the row; up to
//      kWaveCand are reloaded, four a lane, and searched instead of the row (otherwise the
//      row's own registers are searched: heavy ties, or k too large for step 1);
//   3. wave_select: bitwise search for the k-th key, then, when more ties exist than places,
//      a bitwise search over the reversed column for the last tie admitted (lowest columns
//      win); winners take LDS slots and are ranked by counting among themselves.
constexpr int kWaveMaxV = 2048;
constexpr int kWaveCand = 256;

template <typename T, int NR>
__device__ __forceinline__ void wave_select(const uint32_t (&key)[NR], const uint32_t (&rc)[NR], int nreg,
                                            int k, unsigned long long* buf, const T* rp, int64_t row,
                                            T* __restrict__ values, int32_t* __restrict__ idx32,
                                            int64_t* __restrict__ idx64) {
  const int lane = threadIdx.x;
  const unsigned long long below = (1ull << lane) - 1ull;
  uint32_t kth = 0u;
  for (int bit = 31; bit >= KeyBits<T>::low; --bit) {
    const uint32_t trial = kth | (1u << bit);
    int cnt = 0;
#pragma unroll
    for (int e = 0; e < NR; ++e)
      if (e < nreg) cnt += __builtin_popcountll(__ballot(key[e] >= trial));
    if (cnt >= k) kth = trial;
  }
  int c_gt = 0, c_eq = 0;
#pragma unroll
  for (int e = 0; e < NR; ++e)
    if (e < nreg) {
      c_gt += __builtin_popcountll(__ballot(key[e] > kth));
      c_eq += __builtin_popcountll(__ballot(key[e] == kth));
    }
  const int need = k - c_gt;          // places left for the c_eq ties (kth > 0: empty slots never tie)
  uint32_t cth = 0u;                  // ties whose reversed column reaches cth are admitted
  if (need < c_eq) {
    for (int bit = 11; bit >= 0; --bit) {   // reversed columns are 1..kWaveMaxV = 1 << 11
      const uint32_t trial = cth | (1u << bit);
      int cnt = 0;
#pragma unroll
      for (int e = 0; e < NR; ++e)
        if (e < nreg) cnt += __builtin_popcountll(__ballot(key[e] == kth && rc[e] >= trial));
      if (cnt >= need) cth = trial;
    }
  }
  __syncthreads();                    // the candidates in buf have been read
  int base = 0;
#pragma unroll
  for (int e = 0; e < NR; ++e)
    if (e < nreg) {
      const bool win = key[e] > kth || (key[e] == kth && rc[e] >= cth);
      const unsigned long long m = __ballot(win);
      if (win) buf[base + __builtin_popcountll(m & below)] = ((unsigned long long)key[e] << 32) | rc[e];
      base += __builtin_popcountll(m);
    }
  __syncthreads();
  if (k > 64) {
    // many winners: a bitonic sort of the slots (padded with zeros, which sort last) costs
    // log^2 steps where counting costs k reads per winner
    int kp = 128;
    while (kp < k) kp <<= 1;
    for (int s = k + lane; s < kp; s += 64) buf[s] = 0ull;
    __syncthreads();
    for (int size = 2; size <= kp; size <<= 1) {
      for (int stride = size >> 1; stride > 0; stride >>= 1) {
        for (int t = lane; t < kp / 2; t += 64) {
          const int lo = 2 * t - (t & (stride - 1));
          const int hi = lo + stride;
          const bool desc = (lo & size) == 0;
          const unsigned long long a = buf[lo], b = buf[hi];
          if ((a < b) == desc) { buf[lo] = b; buf[hi] = a; }
        }
        __syncthreads();
      }
    }
    for (int s = lane; s < k; s += 64) {
      const unsigned long long me = buf[s];
      const int col = kWaveMaxV - (int)(uint32_t)(me & 0xFFFFFFFFull);
      const int64_t o = row * (int64_t)k + s;
      if (idx32 != nullptr) idx32[o] = col;
      if (idx64 != nullptr) idx64[o] = col;
      if (values != nullptr) values[o] = rp[col];
    }
    return;
  }
  for (int s = lane; s < k; s += 64) {
    const unsigned long long me = buf[s];
    int r = 0;
    for (int i = 0; i < k; ++i) r += buf[i] > me ? 1 : 0;
    const int col = kWaveMaxV - (int)(uint32_t)(me & 0xFFFFFFFFull);
    const int64_t o = row * (int64_t)k + r;
    if (idx32 != nullptr) idx32[o] = col;
    if (idx64 != nullptr) idx64[o] = col;
    if (values != nullptr) values[o] = rp[col];
  }
}

template <typename T, int EPL, bool VEC>
__global__ __launch_bounds__(64) void topk_wave_kernel(const T* __restrict__ x, T* __restrict__ values,
                                                        int32_t* __restrict__ idx32,
                                                        int64_t* __restrict__ idx64, int v, int k) {
  __shared__ unsigned long long buf[kMaxK];
  constexpr uint32_t KMASK = KeyBits<T>::mask;
  constexpr int EPV = Elem<T>::kVec;
  static_assert(!VEC || EPL % EPV == 0, "whole vectors per lane");
  const int lane = threadIdx.x;
  const int64_t row = blockIdx.x;
  const T* rp = x + row * (int64_t)v;
  auto col_of = [&](int e) { return VEC ? ((e / EPV) * 64 + lane) * EPV + (e % EPV) : lane + 64 * e; };
  // 0 is below the key of every value (-inf maps to 0x007FFFFF), so empty slots never win
  uint32_t mk[EPL];
  if constexpr (VEC) {
#pragma unroll
    for (int g = 0; g < EPL / EPV; ++g) {
      const int c0 = (g * 64 + lane) * EPV;
      if (c0 < v) {
        float f[EPV];
        Elem<T>::unpack(load16_stream(rp + c0), f);
#pragma unroll
        for (int i = 0; i < EPV; ++i) mk[g * EPV + i] = key_of(f[i]) & KMASK;
      } else {
#pragma unroll
        for (int i = 0; i < EPV; ++i) mk[g * EPV + i] = 0u;
      }
    }
  } else {
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
      const int col = lane + 64 * e;
      mk[e] = col < v ? (key_of(Elem<T>::load1(rp + col)) & KMASK) : 0u;
    }
  }
  // step 1: group maxima (one group per lane for small k, up to four otherwise)
  constexpr int GM = EPL < 4 ? EPL : 4;
  uint32_t gm[GM];
#pragma unroll
  for (int g = 0; g < GM; ++g) gm[g] = 0u;
#pragma unroll
  for (int e = 0; e < EPL; ++e) gm[e % GM] = gm[e % GM] > mk[e] ? gm[e % GM] : mk[e];
  int groups = GM;
  if (k <= 16) {
#pragma unroll
    for (int g = 1; g < GM; ++g) {
      gm[0] = gm[0] > gm[g] ? gm[0] : gm[g];
      gm[g] = 0u;
    }
    groups = 1;
  }
  uint32_t tau = 0u;
  if (k <= 64 * groups) {
    for (int bit = 31; bit >= KeyBits<T>::low; --bit) {
      const uint32_t trial = tau | (1u << bit);
      int cnt = 0;
#pragma unroll
      for (int g = 0; g < GM; ++g)
        if (g < groups) cnt += __builtin_popcountll(__ballot(gm[g] >= trial));
      if (cnt >= k) tau = trial;
    }
  }
  // step 2: candidates
  const unsigned long long below = (1ull << lane) - 1ull;
  int ncand = 0;
  uint32_t rc[EPL];
#pragma unroll
  for (int e = 0; e < EPL; ++e) {
    rc[e] = (uint32_t)(kWaveMaxV - col_of(e));
    const bool c = mk[e] >= tau && mk[e] != 0u;
    const unsigned long long m = __ballot(c);
    if (m == 0ull) continue;          // most registers hold no candidate
    if (c) {
      const int s = ncand + __builtin_popcountll(m & below);
      if (s < kWaveCand) buf[s] = ((unsigned long long)mk[e] << 32) | rc[e];
    }
    ncand += __builtin_popcountll(m);
  }
  __syncthreads();
  if (ncand <= 64) {
    // at most one candidate a lane: rank them all by counting; ranks below k are the output
    const unsigned long long me = lane < ncand ? buf[lane] : 0ull;
    int r = 0;
    int i = 0;
    for (; i + 8 <= ncand; i += 8) {
      unsigned long long o[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) o[u] = buf[i + u];
#pragma unroll
      for (int u = 0; u < 8; ++u) r += o[u] > me ? 1 : 0;
    }
    for (; i < ncand; ++i) r += buf[i] > me ? 1 : 0;
    if (lane < ncand && r < k) {
      const int col = kWaveMaxV - (int)(uint32_t)(me & 0xFFFFFFFFull);
      const int64_t o = row * (int64_t)k + r;
      if (idx32 != nullptr) idx32[o] = col;
      if (idx64 != nullptr) idx64[o] = col;
      if (values != nullptr) values[o] = rp[col];
    }
  } else if (ncand <= kWaveCand) {
    constexpr int CR = kWaveCand / 64;
    uint32_t ck[CR], cc[CR];
#pragma unroll
    for (int j = 0; j < CR; ++j) {
      const int s = lane + 64 * j;
      const unsigned long long item = s < ncand ? buf[s] : 0ull;
      ck[j] = (uint32_t)(item >> 32);
      cc[j] = (uint32_t)(item & 0xFFFFFFFFull);
    }
    wave_select<T, CR>(ck, cc, (ncand + 63) / 64, k, buf, rp, row, values, idx32, idx64);
  } else {
    wave_select<T, EPL>(mk, rc, EPL, k, buf, rp, row, values, idx32, idx64);
  }
}

// Rows of at most 512 elements with k <= 8: L lanes per row (8, 16, 32 or 64), eight
// neighbouring elements per lane, so a wave works on 64 / L rows at once and reads whole rows
// with 16-byte loads (VEC: v a multiple of eight, aligned buffer). Each of the k picks is a
// lane-local first maximum, a group maximum over the keys and a group minimum over the indices
// that hold it -- the canonical order (value descending, index ascending) by construction.
constexpr int kGroupMaxV = 512;
constexpr int kGroupMaxK = 8;
constexpr int kGroupRows = 2;   // rows a lane group works on together (independent chains)

template <typename T, int L, bool VEC>
__global__ __launch_bounds__(256) void topk_group_kernel(const T* __restrict__ x, T* __restrict__ values,
                                                         int32_t* __restrict__ idx32,
                                                         int64_t* __restrict__ idx64, int64_t n, int v,
                                                         int k) {
  constexpr int GE = 8;
  constexpr int GPW = 64 / L;
  constexpr int R = kGroupRows;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane / L, l = lane % L;
  const int c0 = l * GE;
  const int64_t first = ((int64_t)blockIdx.x * 4 + wave) * (GPW * R);
  int64_t row[R];
  bool live[R];
  uint32_t key[R][GE];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    row[r] = first + r * GPW + g;
    live[r] = row[r] < n;
    float f[GE];
    if constexpr (VEC) {
      constexpr int EPV = Elem<T>::kVec;
      if (live[r] && c0 < v) {
#pragma unroll
        for (int h = 0; h < GE / EPV; ++h) {
          float part[EPV];
          Elem<T>::unpack(load16_stream(x + row[r] * (int64_t)v + c0 + h * EPV), part);
#pragma unroll
          for (int q = 0; q < EPV; ++q) f[h * EPV + q] = part[q];
        }
      } else {
#pragma unroll
        for (int q = 0; q < GE; ++q) f[q] = 0.f;
      }
    } else {
#pragma unroll
      for (int q = 0; q < GE; ++q) f[q] = (live[r] && c0 + q < v) ? Elem<T>::load1(x + row[r] * (int64_t)v + c0 + q) : 0.f;
    }
#pragma unroll
    for (int q = 0; q < GE; ++q) key[r][q] = (live[r] && c0 + q < v) ? key_of(f[q]) : 0u;   // 0: below every real key
  }
  int mine[R];
#pragma unroll
  for (int r = 0; r < R; ++r) mine[r] = 0;
#pragma unroll
  for (int j = 0; j < kGroupMaxK; ++j) {
    if (j < k) {
      uint32_t bk[R], gk[R];
      int bq[R], gi[R];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        bk[r] = key[r][0];
        bq[r] = 0;
#pragma unroll
        for (int q = 1; q < GE; ++q) {
          if (key[r][q] > bk[r]) { bk[r] = key[r][q]; bq[r] = q; }
        }
      }
#pragma unroll
      for (int r = 0; r < R; ++r) gk[r] = group_max_u<L>(bk[r]);
#pragma unroll
      for (int r = 0; r < R; ++r) gi[r] = group_min_i<L>((bk[r] == gk[r]) ? c0 + bq[r] : 0x7fffffff);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int wl = gi[r] >> 3, wq = gi[r] & 7;
#pragma unroll
        for (int q = 0; q < GE; ++q) {
          if (l == wl && q == wq) key[r][q] = 0u;
        }
        if (l == j) mine[r] = gi[r];
      }
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    if (live[r] && l < k) {
      const int64_t o = row[r] * (int64_t)k + l;
      if (idx32 != nullptr) idx32[o] = mine[r];
      if (idx64 != nullptr) idx64[o] = mine[r];
      if (values != nullptr) values[o] = x[row[r] * (int64_t)v + mine[r]];
    }
  }
}

// widest row (in 16-byte vectors) whose key prefixes fit the LDS budget
constexpr int kLdsMaxVec = 20480;
// largest k the 128-thread form takes: the threshold of two full waves then still leaves the
// candidates within its 512 slots
constexpr int kSmallMaxK = 72;

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
#define GO(TH, IT, BIG_)                                                                         \
  FM_LAUNCH((topk_kernel<T, TH, IT, BIG_>), grid, dim3(TH), 0, st, xp, vp, i32, i64, v, k, vec_ok)
#define GOL(TH, UN, BIG_)                                                                        \
  FM_LAUNCH((topk_lds_kernel<T, TH, UN, BIG_>), grid, dim3(TH), (size_t)(nvec + 8) * 2, st, xp, vp, \
                     i32, i64, v, k, vec_ok)
  const bool big = k > 256;               // twice the candidate slots (1024-thread forms only)
  // 512 threads up to 140 K bf16 columns: three such workgroups share a compute unit, and while one
  // is in its selection phases two keep the loads going (top-64 of [4096,128256]: 163 against 166.5 us
  // with 1024 threads, k = 256: 215 against 254; at 152 K columns only two fit and 1024 threads win)
  int variant = nvec <= 3072 ? 1 : (nvec <= 17600 ? 2 : 3);
  {
    // The threshold search needs k <= 63 x (full waves of the row); more threads give more of
    // them while the row has a vector for each, and it pays while k stays within half of that
    // bound (past it the candidates mostly overflow anyway). Otherwise the exact path runs for
    // certain: the smallest workgroup whose threads can keep the row's keys in registers
    // (four vectors each), else the largest.
    const int64_t whole = v / EPV;
    auto cap = [&](int threads) { return (int)(std::min<int64_t>(threads, whole) / 64) * 63; };
    auto pays = [&](int threads) { return 2 * k <= cap(threads) + 8; };
    const int threads_of[4] = {0, 256, 512, 1024};
    if (k > cap(threads_of[variant])) {
      int pick = 0;
      for (int cand = variant + 1; cand <= 3 && pick == 0; ++cand)
        if (cap(threads_of[cand]) > cap(threads_of[cand - 1]) && pays(threads_of[cand])) pick = cand;
      if (pick == 0) {
        pick = 3;
        for (int cand = 3; cand >= 1; --cand)
          if (whole <= (int64_t)threads_of[cand] * 4) pick = cand;
      }
      variant = pick;
    }
    // Rows of up to 48 KiB with a small k are bound by the latency of the phases after the
    // read, not by the read: two waves per row and half the LDS put fourteen rows on a compute
    // unit instead of eight (1.2-1.8x on rows of 2-24 K elements; even by 64 KiB rows).
    if (whole <= 3072 && k <= kSmallMaxK) variant = 4;
  }
  // narrow rows, few picks: lane groups. A pick costs a lane group as much as it costs the
  // wave-per-row kernel, which pays it once per candidate set instead: past 256 columns that is
  // cheaper from the third pick on.
  if (v <= kGroupMaxV && k <= (v <= 256 ? kGroupMaxK : 2)) {
    const bool gvec = vec_ok && v % 8 == 0;
#define GOG(L_)                                                                                    \
  do {                                                                                             \
    constexpr int rows_per_block = 4 * (64 / L_) * kGroupRows;                                     \
    const dim3 ggrid((unsigned)((n + rows_per_block - 1) / rows_per_block));                       \
    if (gvec) FM_LAUNCH((topk_group_kernel<T, L_, true>), ggrid, dim3(256), 0, st, xp, vp, i32, i64, n, v, k); \
    else FM_LAUNCH((topk_group_kernel<T, L_, false>), ggrid, dim3(256), 0, st, xp, vp, i32, i64, n, v, k);     \
  } while (0)
    if (v <= 64) GOG(8);
    else if (v <= 128) GOG(16);
    else if (v <= 256) GOG(32);
    else GOG(64);
#undef GOG
  }
  else if (v <= kWaveMaxV) {       // short rows: a wave per row
    int epl = 1;
    while (64 * epl < v) epl *= 2;
    const bool wvec = vec_ok && v % EPV == 0 && epl >= EPV;
#define GOW(EPL_, VEC_)                                                                            \
  FM_LAUNCH((topk_wave_kernel<T, EPL_, VEC_>), grid, dim3(64), 0, st, xp, vp, i32, i64, v, k)
#define GOWV(EPL_)                                                                                 \
  if constexpr (EPL_ % EPV == 0) {                                                                 \
    if (wvec) GOW(EPL_, true);                                                                     \
    else GOW(EPL_, false);                                                                         \
  } else {                                                                                         \
    GOW(EPL_, false);                                                                              \
  }
    if (epl == 1) { GOWV(1) }
    else if (epl == 2) { GOWV(2) }
    else if (epl == 4) { GOWV(4) }
    else if (epl == 8) { GOWV(8) }
    else if (epl == 16) { GOWV(16) }
    else { GOWV(32) }
#undef GOWV
#undef GOW
  }
  else if (nvec > kLdsMaxVec && nvec <= fm_host::kLdsWideMaxVec && !big &&
           fm_host::allow_wide_lds<&topk_lds_kernel<T, 1024, 4, kTopkNormal>>()) GOL(1024, 4, false);
  else if (nvec > kLdsMaxVec && nvec <= fm_host::kLdsWideMaxVec && big &&
           fm_host::allow_wide_lds<&topk_lds_kernel<T, 1024, 4, kTopkBig>>()) GOL(1024, 4, true);
  else if (nvec > kLdsMaxVec) {
    if (nvec <= 1024 * 32) {
      if (big) GO(1024, 32, true);
      else GO(1024, 32, false);
    } else {
      if (big) GO(1024, 0, true);
      else GO(1024, 0, false);
    }
  } else if (variant == 4) GOL(128, 4, kTopkSmall);
  else if (variant == 1) GOL(256, 4, false);
  else if (variant == 2) GOL(512, 4, false);
  else if (big) GOL(1024, 4, true);
  else GOL(1024, 4, false);
#undef GO
#undef GOL
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
