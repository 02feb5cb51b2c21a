// Selection phases of the exact top-k, shared by the stand-alone kernel (topk.hip) and the
// KL forward that also returns the teacher's top-k (kl.hip).
//
// The caller streams the row once and hands over the maxima of the 16-byte vectors it read
// (per thread in registers, or for the whole row as 16-bit key prefixes in LDS), each thread's
// overall maximum (`fm`) and whether it saw a NaN. topk_finish then
//   T  finds, per wave, the ceil(k / waves)-th largest group maximum with a ballot search and
//      takes the minimum over the waves as tau -- never above the true k-th value;
//   B  lists the vectors whose maximum is >= tau, re-reads just those (served by cache) and
//      turns every element >= tau into a candidate (key, index) in LDS;
//   R  ranks candidates by counting how many others beat them under (key descending, index
//      ascending); rank r < k is output slot r.
// Rows with too many candidates (long runs of equal values) take an exact path: a bitwise
// search for the k-th key over the whole row, then an index-ordered scan that admits the
// first (k - #greater) ties. Keys are order-preserving integer images of the fp32 value.
#pragma once

#include <atomic>

#include "fm_vocab.hip.h"

namespace fm {

constexpr int kCap = 1024;  // candidate slots in LDS (twice that for 1024-thread workgroups)
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

// Bits of the key that a value of type T can set (the rest are all-zero or, for negative
// values, all-one): bf16 keeps 16, fp16 19 (sign, fp32 exponent, 10 mantissa bits), fp32 all.
template <typename T> struct KeyBits { static constexpr uint32_t mask = 0xFFFFFFFFu; static constexpr int low = 0; };
template <> struct KeyBits<bf16_t> { static constexpr uint32_t mask = 0xFFFF0000u; static constexpr int low = 16; };
template <> struct KeyBits<f16_t> { static constexpr uint32_t mask = 0xFFFFE000u; static constexpr int low = 13; };

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

// Sum of a 64-bit value over the workgroup (smem: nw words).
__device__ __forceinline__ unsigned long long block_sum_u64(unsigned long long v, unsigned long long* smem, int nw) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) smem[wave] = v;
  __syncthreads();
  unsigned long long s = 0ull;
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
constexpr int kSortFrom = 128;  // candidate counts above this are sorted instead of counted ...
constexpr int kRankSlots = 512; // ... when C * C > 256 * threads, so counting never sees more than this

// Where the vector maxima of the streaming pass live.
enum VecMax { kVecMaxNone = 0, kVecMaxRegs = 1, kVecMaxLds = 2 };

// 16-bit prefix of a key, rounded up: key >= tau implies key_prefix(key) >= (tau >> 16).
__device__ __forceinline__ uint32_t key_prefix(uint32_t key) {
  const uint32_t p = (key >> 16) + ((key & 0xFFFFu) != 0u ? 1u : 0u);
  return p > 0xFFFFu ? 0xFFFFu : p;
}

// BIG doubles the candidate slots: for k above 256 the threshold of a 1024-thread workgroup
// admits one to two thousand elements, which then still avoid the exact path. It is a separate
// instantiation because it costs the ordinary case (k = 64: 280 against 190 us per launch).
// SMALL halves slots and work list instead: 11 KB of LDS per workgroup, so that fourteen
// 128-thread workgroups share a compute unit (rows of a few thousand elements, k <= 64).
enum TopkSize { kTopkNormal = 0, kTopkBig = 1, kTopkSmall = 2 };
template <int THREADS, int VMAX, int SZ = kTopkNormal>
struct TopkShared {
  static constexpr int kSlots = SZ == kTopkBig ? 2 * kCap : (SZ == kTopkSmall ? kCap / 2 : kCap);
  static constexpr int kWork = SZ == kTopkSmall ? kWorkCap / 2 : kWorkCap;
  unsigned long long ccomp[kSlots];  // (key << 32) | ~index : larger is better
  int crank[kRankSlots];   // counting ranks at most this many candidates (more are sorted)
  int work[VMAX ? kWork : 1];
  int s_int[THREADS / 64];
  uint32_t s_tau[THREADS / 64];
  int s_count, s_nwork;
};

// maximum of one vector; NaN if the vector holds a NaN (NaN outranks everything)
template <typename T>
__device__ __forceinline__ float fold_vector_max(const u32x4& raw) {
  constexpr int EPV = Elem<T>::kVec;
  float f[EPV];
  Elem<T>::unpack(raw, f);
  float m = f[0];
  bool bad = f[0] != f[0];
#pragma unroll
  for (int e = 1; e < EPV; ++e) { m = fmaxf(m, f[e]); bad |= (f[e] != f[e]); }
  return bad ? __builtin_nanf("") : m;
}

// ---- 16-bit stream keys of the half types.
// The streaming pass of a bf16 / fp16 row needs only the maximum of each 16-byte vector, so it
// never unpacks to fp32: two elements at a time, the sign-magnitude bit patterns are turned into
// unsigned 16-bit keys with packed integer instructions and reduced with packed maxima.
//   skey(b) = (b ^ (b < 0 ? 0x7FFF : 0)) + 0x8000 - off   (mod 2^16),  off = 0x7FFF - bits(+inf)
// is monotone in the value, puts -inf at 0 and +inf at kNanAbove, and -- because the subtraction
// wraps -- both NaN signs above kNanAbove. -0.0 lands one below +0.0 (the two tie in the final
// order), which skey_threshold makes up for.
template <typename T> struct SKey { static constexpr bool ok = false; };
template <> struct SKey<bf16_t> { static constexpr bool ok = true; static constexpr uint32_t inf = 0x7F80u; };
template <> struct SKey<f16_t> { static constexpr bool ok = true; static constexpr uint32_t inf = 0x7C00u; };
template <typename T> struct SKeyC {
  static constexpr uint32_t off = 0x7FFFu - SKey<T>::inf;
  static constexpr uint32_t add = (0x8000u - off) & 0xFFFFu;
  static constexpr uint32_t kNanAbove = (0x8000u + SKey<T>::inf - off) & 0xFFFFu;
};

typedef unsigned short u16x2_t __attribute__((ext_vector_type(2)));
typedef short i16x2_t __attribute__((ext_vector_type(2)));

// keys of the two elements packed in one 32-bit word
template <typename T>
__device__ __forceinline__ u16x2_t skey_pair(uint32_t two) {
  const i16x2_t sgn = __builtin_bit_cast(i16x2_t, two) >> (short)15;
  const uint32_t t = two ^ (__builtin_bit_cast(uint32_t, sgn) & 0x7FFF7FFFu);
  const u16x2_t a = {(unsigned short)SKeyC<T>::add, (unsigned short)SKeyC<T>::add};
  return __builtin_bit_cast(u16x2_t, t) + a;
}
// largest key of a 16-byte vector
template <typename T>
__device__ __forceinline__ uint32_t skey_vector_max(const u32x4& raw) {
  const u16x2_t a = __builtin_elementwise_max(skey_pair<T>(raw[0]), skey_pair<T>(raw[1]));
  const u16x2_t b = __builtin_elementwise_max(skey_pair<T>(raw[2]), skey_pair<T>(raw[3]));
  const u16x2_t m = __builtin_elementwise_max(a, b);
  const uint32_t lo = m[0], hi = m[1];
  return lo > hi ? lo : hi;
}
template <typename T>
__device__ __forceinline__ uint32_t skey_of_bits(uint32_t b) {
  return ((b ^ ((b & 0x8000u) ? 0x7FFFu : 0u)) + SKeyC<T>::add) & 0xFFFFu;
}
// value of a key that is not above kNanAbove
template <typename T>
__device__ __forceinline__ float float_of_skey(uint32_t s) {
  const uint32_t t = (s - SKeyC<T>::add) & 0xFFFFu;
  const uint32_t b = t ^ ((t & 0x8000u) ? 0x7FFFu : 0u);
  if constexpr (Elem<T>::kDtype == FM_BF16) return bf16_bits_to_float((uint16_t)b);
  else return (float)__builtin_bit_cast(_Float16, (uint16_t)b);
}
// Smallest stream key a vector maximum can have when the vector holds an element whose fp32 key
// reaches tau (tau_f is tau's float image): the key of tau_f rounded DOWN to T. Zero admits -0.0.
template <typename T>
__device__ __forceinline__ uint32_t skey_threshold(uint32_t tau, float tau_f, bool only_nan) {
  // the NaN key, whole or cut down to the bits T can set: vectors that hold a NaN
  if (only_nan || tau > 0xFF800000u) return SKeyC<T>::kNanAbove + 1u;
  if (tau <= 0x007FFFFFu) return 0u;   // at or below -inf: everything
  uint32_t b;
  float back;
  if constexpr (Elem<T>::kDtype == FM_BF16) {
    b = pack_bf16(tau_f, 0.f) & 0xFFFFu;
    back = bf16_bits_to_float((uint16_t)b);
  } else {
    const _Float16 h = (_Float16)tau_f;
    b = __builtin_bit_cast(uint16_t, h);
    back = (float)h;
  }
  if ((b & 0x7FFFu) == 0u) return skey_of_bits<T>(0x8000u);
  uint32_t s = skey_of_bits<T>(b);
  if (back > tau_f && s > 0u) s -= 1u;   // keys are dense in the values: one key down is one value down
  return s;
}

// The same for fp32 rows: 32-bit stream keys (three integer instructions an element), of which the
// LDS keeps the upper 16 bits rounded up.
constexpr uint32_t kSKey32Add = 0x7F800001u;        // 0x80000000 - (0x7FFFFFFF - bits(+inf))
constexpr uint32_t kSKey32NanAbove = 0xFF000001u;   // the key of +inf
__device__ __forceinline__ uint32_t skey32(uint32_t b) {
  return (b ^ ((uint32_t)((int32_t)b >> 31) & 0x7FFFFFFFu)) + kSKey32Add;
}
__device__ __forceinline__ uint32_t skey32_vector_max(const u32x4& raw) {
  const uint32_t a = skey32(raw[0]), b = skey32(raw[1]), c = skey32(raw[2]), d = skey32(raw[3]);
  const uint32_t ab = a > b ? a : b, cd = c > d ? c : d;
  return ab > cd ? ab : cd;
}
// upper 16 bits, rounded up: s >= t implies skey32_prefix(s) >= skey32_prefix(t)
__device__ __forceinline__ uint32_t skey32_prefix(uint32_t s) {
  const uint32_t c = s < 0xFFFF0000u ? s : 0xFFFF0000u;
  return (c + 0xFFFFu) >> 16;
}
__device__ __forceinline__ float float_of_skey32(uint32_t s) {
  const uint32_t t = s - kSKey32Add;
  return __builtin_bit_cast(float, t ^ ((uint32_t)((int32_t)t >> 31) & 0x7FFFFFFFu));
}
__device__ __forceinline__ uint32_t skey32_threshold(uint32_t tau, float tau_f, bool only_nan) {
  if (only_nan) return skey32_prefix(kSKey32NanAbove + 1u);
  if (tau <= 0x007FFFFFu) return 0u;   // at or below -inf: everything
  const uint32_t b = __builtin_bit_cast(uint32_t, tau_f);
  return skey32_prefix(skey32((b & 0x7FFFFFFFu) == 0u ? 0x80000000u : b));   // zero admits -0.0
}

// how the 16-bit entries of `vhi` were made
enum VhiKind { kVhiPrefix = 0, kVhiStream16 = 1, kVhiStream32 = 2 };

// Everything after the streaming read. With kVecMaxRegs `vmax` holds NV vector maxima per
// thread (vector i * THREADS + tid in slot i); with kVecMaxLds `vhi[c]` holds key_prefix of
// vector c's maximum for the whole row, padded with zeros to a multiple of four entries and
// 8-byte aligned (with SKEY: the 16-bit stream key of vector c's maximum, or the prefix of its
// 32-bit stream key, instead); with
// kVecMaxNone the row is walked a second time. Outputs go to row `orow` of the [rows, k] arrays;
// `probs` (optional) receives exp2(x * c1 - lse2) of the selected elements.
template <typename T, int THREADS, int NV, int VMAX, int BIG = kTopkNormal, int SKEY = kVhiPrefix>
__device__ __forceinline__ void topk_finish(const T* __restrict__ rp, const RowSplit& sp, int v, int k,
                                            const float (&vmax)[NV], const uint16_t* vhi, float fm,
                                            bool has_nan,
                                            TopkShared<THREADS, VMAX, BIG>& sh, int64_t orow,
                                            T* __restrict__ values, int32_t* __restrict__ idx32,
                                            int64_t* __restrict__ idx64, float* __restrict__ probs,
                                            float c1, float lse2) {
  constexpr int EPV = Elem<T>::kVec;
  constexpr int NW = THREADS / 64;
  constexpr int ITERS = NV;
  constexpr uint32_t KMASK = KeyBits<T>::mask;
  constexpr int CAP = TopkShared<THREADS, VMAX, BIG>::kSlots;
  constexpr int WORK = TopkShared<THREADS, VMAX, BIG>::kWork;
  unsigned long long* ccomp = sh.ccomp;
  int* crank = sh.crank;
  int* work = sh.work;
  int* s_int = sh.s_int;
  uint32_t* s_tau = sh.s_tau;
  int& s_count = sh.s_count;
  int& s_nwork = sh.s_nwork;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int ne = edge_count(sp, v);
  const int64_t row = orow;

  // Sorting or ranking of the C candidates in ccomp and the output of the best k.
  auto rank_and_write = [&](int C) {
  // ---- many candidates for the size of the workgroup: a bitonic sort of the slots (key
  // descending, then column ascending; zero padding sorts last) puts output slot r at position
  // r for log^2 steps of work, where counting costs one read of every candidate per candidate
  if (C > kSortFrom && C * C > 256 * THREADS) {
    int cp = 2 * kSortFrom;
    while (cp < C) cp <<= 1;
    for (int s = C + tid; s < cp; s += THREADS) ccomp[s] = 0ull;
    __syncthreads();
    for (int size = 2; size <= cp; size <<= 1) {
      for (int stride = size >> 1; stride > 0; stride >>= 1) {
        for (int t = tid; t < cp / 2; t += THREADS) {
          const int lo = 2 * t - (t & (stride - 1));
          const int hi = lo + stride;
          const bool desc = (lo & size) == 0;
          const unsigned long long a = ccomp[lo], b = ccomp[hi];
          if ((a < b) == desc) { ccomp[lo] = b; ccomp[hi] = a; }
        }
        __syncthreads();
      }
    }
    for (int r = tid; r < k; r += THREADS) {
      const int col = (int)(~(uint32_t)(ccomp[r] & 0xFFFFFFFFull));
      const int64_t o = row * (int64_t)k + r;
      if (idx32 != nullptr) idx32[o] = col;
      if (idx64 != nullptr) idx64[o] = col;
      if (values != nullptr) values[o] = rp[col];
      if (probs != nullptr) probs[o] = fast_exp2(Elem<T>::load1(rp + col) * c1 - lse2);
    }
    return;
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
      // every lane reads the same candidate (an LDS broadcast); eight reads in flight hide
      // the LDS latency that a one-at-a-time loop would pay per candidate
      int r = 0;
      int i = i0;
      for (; i + 8 <= i1; i += 8) {
        unsigned long long o[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) o[u] = ccomp[i + u];
#pragma unroll
        for (int u = 0; u < 8; ++u) r += o[u] > me ? 1 : 0;
      }
      for (; i < i1; ++i) r += ccomp[i] > me ? 1 : 0;
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
      if (probs != nullptr) probs[o] = fast_exp2(Elem<T>::load1(rp + col) * c1 - lse2);
    }
  }
  };

  int C = 0;
  bool overflow = false;
  if (v <= CAP) {
    // short row: every element is a candidate
    for (int j = tid; j < v; j += THREADS)
      ccomp[j] = ((unsigned long long)key_of(Elem<T>::load1(rp + j)) << 32) | (uint32_t)(~j);
    C = v;
    __syncthreads();
  } else {
    const bool has = tid < sp.nvec || tid < ne;
    const uint32_t mykey = !has ? 0u : (has_nan ? 0xFFFFFFFFu : key_of(fm));

    // ---- phase T: per-wave j-th largest group maximum, then the minimum over waves.
    // Only waves whose 64 lanes all hold data vote: nfull of them with j maxima each bound
    // at least k elements from below; a part-filled wave would drag tau to the bottom.
    const int active = (sp.nvec > ne ? sp.nvec : ne) < THREADS ? (sp.nvec > ne ? sp.nvec : ne) : THREADS;
    const int nfull = active >> 6;
    const int j = nfull > 0 ? (k + nfull - 1) / nfull : 65;
    if (j > 64) {
      // no full wave can bound the k-th value from below (k beyond 63 per full wave): every
      // element would become a candidate, so the exact path is taken at once
      C = CAP + 1;
    } else {
      // Only the bits a value of type T can set are searched (the masked key is a lower bound
      // of the key with nothing representable in between), two bits per step: three ballots
      // that do not depend on each other instead of two dependent rounds.
      uint32_t tw = 0u;
      if (j <= 64 && wave < nfull) {
        const uint32_t mk = mykey & KMASK;
        int bit = 31;
        for (; bit - 1 >= KeyBits<T>::low; bit -= 2) {
          const int shift = bit - 1;
          const int c1 = __builtin_popcountll(__ballot(mk >= (tw | (1u << shift))));
          const int c2 = __builtin_popcountll(__ballot(mk >= (tw | (2u << shift))));
          const int c3 = __builtin_popcountll(__ballot(mk >= (tw | (3u << shift))));
          const uint32_t dgt = c3 >= j ? 3u : (c2 >= j ? 2u : (c1 >= j ? 1u : 0u));
          tw |= dgt << shift;
        }
        if (bit >= KeyBits<T>::low) {   // an odd number of key bits leaves one
          const uint32_t trial = tw | (1u << bit);
          if (__builtin_popcountll(__ballot(mk >= trial)) >= j) tw = trial;
        }
      }
      if (lane == 0) s_tau[wave] = (wave < nfull || j > 64) ? tw : 0xFFFFFFFFu;
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
          if (slot < CAP) ccomp[slot] = ((unsigned long long)key_of(f) << 32) | (uint32_t)(~col);
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
      if constexpr (VMAX != kVecMaxNone) {
        // B1: vectors that can hold a candidate go to the work list
        // (once the list has overflowed the row goes to the exact path anyway: the remaining
        // vectors are not appended, which spares a row of equal values 16 K atomics on one word)
        auto list = [&](int c) {
          const int slot = atomicAdd(&s_nwork, 1);
          if (slot < WORK) work[slot] = c;
        };
        if constexpr (VMAX == kVecMaxRegs) {
  #pragma unroll
          for (int i = 0; i < ITERS; ++i) {
            const int c = i * THREADS + tid;
            if (c < sp.nvec && take_of(vmax[i])) list(c);
          }
        } else {
          uint32_t tau_hi = tau >> 16;
          if constexpr (SKEY == kVhiStream16) tau_hi = skey_threshold<T>(tau, tau_f, only_nan);
          if constexpr (SKEY == kVhiStream32) tau_hi = skey32_threshold(tau, tau_f, only_nan);
          const uint64_t* quad = reinterpret_cast<const uint64_t*>(vhi);
          bool full = false;   // this thread has seen the list overflow: the row takes the exact path
          for (int q = tid; q * 4 < sp.nvec && !full; q += THREADS) {   // anyway, and a row of equal values
            const uint64_t four = quad[q];                              // is spared 16 K atomics on one word
  #pragma unroll
            for (int e = 0; e < 4; ++e) {
              const int c = q * 4 + e;
              if (c < sp.nvec && (uint32_t)((four >> (16 * e)) & 0xFFFFu) >= tau_hi) {
                const int slot = atomicAdd(&s_nwork, 1);
                if (slot < WORK) work[slot] = c;
                else full = true;
              }
            }
          }
        }
        __syncthreads();
        const int nwork = s_nwork;
        overflow = nwork > WORK;
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
      if (overflow) C = CAP + 1;

    }
    // ---- runs of equal values at the k-th place, rows whose vector maxima sit in LDS as exact
    // 16-bit keys (bf16 / fp16): the k-th largest VECTOR maximum, tau_v, is found by a bit search
    // over those 2 bytes per vector in LDS, no row read. At least k vectors hold an element
    // >= tau_v, and elements > tau_v can only sit in the fewer than k vectors whose maximum is
    // above it: those are revisited through the work list. Either they are k or more -- then the
    // top k are among them -- or the k-th value IS tau_v and the remaining places go to the first
    // elements equal to it in column order, which a scan of the row's head finds (it stops as soon
    // as it has them: with long runs that is the first few thousand columns).
    if constexpr (VMAX == kVecMaxLds && SKEY == kVhiStream16) {
      if (C > CAP && sp.nvec >= k) {
        constexpr uint32_t NANK = SKeyC<T>::kNanAbove + 1u;
        const uint32_t negz = skey_of_bits<T>(0x8000u);
        auto nsk = [&](int c) -> uint32_t {   // -0.0 ties with +0.0, every NaN with every other
          uint32_t sk = vhi[c];
          sk = sk == negz ? sk + 1u : sk;
          return sk < NANK ? sk : NANK;
        };
        uint32_t tsk = 0u;
        for (int shift = 14; shift >= 0; shift -= 2) {   // two bits a step: three counts, one reduction
          int c1 = 0, c2 = 0, c3 = 0;
          const uint32_t t1 = tsk | (1u << shift), t2 = tsk | (2u << shift), t3 = tsk | (3u << shift);
          for (int c = tid; c < sp.nvec; c += THREADS) {
            const uint32_t sk = nsk(c);
            c1 += sk >= t1 ? 1 : 0;
            c2 += sk >= t2 ? 1 : 0;
            c3 += sk >= t3 ? 1 : 0;
          }
          // counts are below 2^20 (a row holds at most 2^16.1 vectors): three fit one 64-bit sum
          const unsigned long long packed = block_sum_u64(((unsigned long long)c3 << 42) |
                                                          ((unsigned long long)c2 << 21) | (unsigned long long)c1,
                                                          reinterpret_cast<unsigned long long*>(ccomp), NW);
          const int n1 = (int)(packed & 0x1FFFFFull), n2 = (int)((packed >> 21) & 0x1FFFFFull), n3 = (int)(packed >> 42);
          tsk = n3 >= k ? t3 : (n2 >= k ? t2 : (n1 >= k ? t1 : tsk));
        }
        const uint32_t kth_c = tsk >= NANK ? (0xFFFFFFFFu & KMASK) : (key_of(float_of_skey<T>(tsk)) & KMASK);
        if (tid == 0) { s_count = 0; s_nwork = 0; }
        __syncthreads();
        for (int c = tid; c < sp.nvec; c += THREADS) {
          if (nsk(c) > tsk) {
            const int slot = atomicAdd(&s_nwork, 1);
            if (slot < WORK) work[slot] = c;
          }
        }
        auto above = [&](float f, int col) {
          const uint32_t key = key_of(f);
          if ((key & KMASK) > kth_c) {
            const int slot = atomicAdd(&s_count, 1);
            if (slot < CAP) ccomp[slot] = ((unsigned long long)key << 32) | (uint32_t)(~col);
          }
        };
        for (int e = tid; e < ne; e += THREADS) {
          const int col = edge_col(sp, e);
          above(Elem<T>::load1(rp + col), col);
        }
        __syncthreads();
        const int nwork = s_nwork;   // fewer than k, so it fits the list
        for (int w = tid; w < nwork && nwork <= WORK; w += THREADS) {
          const int c = work[w];
          float f[EPV];
          Elem<T>::unpack(load16(rp + sp.head + (int64_t)c * EPV), f);
#pragma unroll
          for (int e = 0; e < EPV; ++e) above(f[e], sp.head + c * EPV + e);
        }
        __syncthreads();
        const int got = s_count;
        __syncthreads();
        if (nwork <= WORK && got <= CAP) {
          if (got >= k) {   // the top k are among them
            rank_and_write(got);
            return;
          }
          // the k-th key is tau_v's: places [got, k) go to the first elements equal to it, in
          // column order (head edge, vectors, tail edge), found by a scan that stops when it has them
          const int need = k - got;
          int base = 0;
          auto place = [&](float f, int col, int pos) {
            ccomp[got + pos] = ((unsigned long long)key_of(f) << 32) | (uint32_t)(~col);
          };
          {
            float f0 = 0.f;
            int mine = 0;
            if (tid < sp.head) {
              f0 = Elem<T>::load1(rp + tid);
              mine = ((key_of(f0) & KMASK) == kth_c) ? 1 : 0;
            }
            int tot;
            const int ex = block_excl_scan(mine, s_int, NW, &tot);
            if (mine && base + ex < need) place(f0, tid, base + ex);
            base += tot;
          }
          const int niter = (sp.nvec + THREADS - 1) / THREADS;
          for (int i = 0; i < niter && base < need; ++i) {   // base is uniform
            const int c = i * THREADS + tid;
            float f[EPV];
            int mine = 0;
            if (c < sp.nvec) {
              Elem<T>::unpack(load16(rp + sp.head + (int64_t)c * EPV), f);
#pragma unroll
              for (int e = 0; e < EPV; ++e) mine += ((key_of(f[e]) & KMASK) == kth_c) ? 1 : 0;
            }
            int tot;
            int pos = base + block_excl_scan(mine, s_int, NW, &tot);
            if (mine && pos < need) {
#pragma unroll
              for (int e = 0; e < EPV; ++e) {
                if ((key_of(f[e]) & KMASK) == kth_c) {
                  if (pos < need) place(f[e], sp.head + c * EPV + e, pos);
                  ++pos;
                }
              }
            }
            base += tot;
          }
          const int ntail = v - sp.tail0;
          for (int t0 = 0; t0 < ntail && base < need; t0 += THREADS) {
            const int col = sp.tail0 + t0 + tid;
            float f0 = 0.f;
            int mine = 0;
            if (col < v) {
              f0 = Elem<T>::load1(rp + col);
              mine = ((key_of(f0) & KMASK) == kth_c) ? 1 : 0;
            }
            int tot;
            const int ex = block_excl_scan(mine, s_int, NW, &tot);
            if (mine && base + ex < need) place(f0, col, base + ex);
            base += tot;
          }
          __syncthreads();
          rank_and_write(k);
          return;
        }
      }
    }
    if (C > CAP) {
      // ---- exact path: k-th key by bitwise search over the whole row. Rows of up to RK vectors
      // per thread keep their (masked) keys in registers for the search; wider rows are
      // re-read once per key bit. Empty slots hold 0, which no predicate below accepts.
      constexpr int RK = 4;
      const bool cached = sp.nvec <= THREADS * RK && ne <= THREADS;
      uint32_t ck[RK][EPV];
      uint32_t ek = 0u;
      if (cached) {
#pragma unroll
        for (int i = 0; i < RK; ++i) {
          const int c = i * THREADS + tid;
          if (c < sp.nvec) {
            float f[EPV];
            Elem<T>::unpack(load16(rp + sp.head + (int64_t)c * EPV), f);
#pragma unroll
            for (int e = 0; e < EPV; ++e) ck[i][e] = key_of(f[e]) & KMASK;
          } else {
#pragma unroll
            for (int e = 0; e < EPV; ++e) ck[i][e] = 0u;
          }
        }
        if (tid < ne) ek = key_of(Elem<T>::load1(rp + edge_col(sp, tid))) & KMASK;
      }
      auto count_if = [&](auto pred) {
        int cnt = 0;
        if (cached) {
#pragma unroll
          for (int i = 0; i < RK; ++i) {
#pragma unroll
            for (int e = 0; e < EPV; ++e) cnt += pred(ck[i][e]) ? 1 : 0;
          }
          cnt += pred(ek) ? 1 : 0;
          return block_sum_int(cnt, s_int, NW);
        }
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
      int c_gt = 0;
      if (cached) {
        for (int bit = 31; bit >= KeyBits<T>::low; --bit) {
          const uint32_t trial = kth | (1u << bit);
          const int cnt = count_if([&](uint32_t key) { return key >= trial; });
          if (cnt >= k) kth = trial;
        }
        c_gt = count_if([&](uint32_t key) { return key > kth; });
      } else {
        // Rows that do not fit the registers: radix select, eight key bits per sweep of the row
        // (two sweeps for bf16, three for fp16, four for fp32) instead of one sweep per bit. A
        // sweep counts, in a 256-bin LDS histogram, the next key byte of the elements whose
        // higher bytes equal the prefix found so far. Rows come here because of runs of equal
        // values, so the lanes of a wave mostly hold the same bin: equal bins are found with a
        // ballot and added once by one lane (a plain LDS atomic per element would serialise the
        // whole wave on one address). The bin that holds the k-th largest follows from suffix sums.
        int* hist = crank;
        uint32_t prefix = 0u, pmask = 0u;
        int kk = k;   // rank still wanted inside the current prefix
        for (int shift = 24; shift + 8 > KeyBits<T>::low; shift -= 8) {
          for (int i = tid; i < 256; i += THREADS) hist[i] = 0;
          __syncthreads();
          auto tally = [&](uint32_t key, bool live) {   // called by whole waves
            const bool ok = live && (key & pmask) == prefix;
            const uint32_t bin = (key >> shift) & 255u;
            unsigned long long todo = __ballot(ok);
            while (todo != 0ull) {
              const int leader = __builtin_ctzll(todo);
              const uint32_t b = (uint32_t)__builtin_amdgcn_readlane((int)bin, leader);
              const unsigned long long same = __ballot(ok && bin == b);
              if (lane == leader) atomicAdd(&hist[b], (int)__builtin_popcountll(same));
              todo &= ~same;
            }
          };
          for (int c0 = 0; c0 < sp.nvec; c0 += THREADS * 4) {
            u32x4 raw[4];
#pragma unroll
            for (int u = 0; u < 4; ++u)
              raw[u] = load16(rp + sp.head + (int64_t)clamp_col(c0 + u * THREADS + tid, sp.nvec) * EPV);
#pragma unroll
            for (int u = 0; u < 4; ++u) {
              touch(raw[u]);
              const bool live = c0 + u * THREADS + tid < sp.nvec;
              float f[EPV];
              Elem<T>::unpack(raw[u], f);
#pragma unroll
              for (int e = 0; e < EPV; ++e) tally(key_of(f[e]) & KMASK, live);
            }
          }
          for (int e0 = 0; e0 < ne; e0 += THREADS) {
            const int e = e0 + tid;
            const bool live = e < ne;
            tally(key_of(Elem<T>::load1(rp + edge_col(sp, live ? e : ne - 1))) & KMASK, live);
          }
          __syncthreads();
          // bins from the top: thread t of a round owns bin 255 - (round + t); the exclusive scan
          // in thread order is the number of elements in higher bins
          int carry = 0;
          for (int round = 0; round < 256; round += THREADS) {
            const int bin = 255 - (round + tid);
            const int mine = bin >= 0 ? hist[bin] : 0;
            int tot;
            const int above = carry + block_excl_scan(mine, s_int, NW, &tot);
            if (bin >= 0 && above < kk && kk <= above + mine) { s_tau[0] = (uint32_t)bin; s_count = above; }
            carry += tot;
          }
          __syncthreads();
          const uint32_t sel = s_tau[0];
          const int above = s_count;
          __syncthreads();
          prefix |= sel << shift;
          pmask |= 255u << shift;
          kk -= above;
        }
        kth = prefix;
        c_gt = k - kk;
      }
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

  rank_and_write(C);
}

}  // namespace fm

namespace fm_host {
// Rows of more than 20480 vectors still fit the 160 KB of a compute unit, one 1024-thread
// workgroup at a time (rows of up to half a million bf16 / a quarter of a million fp32
// elements). Dynamic LDS beyond 64 KB has to be allowed per kernel and device before the first
// such launch; K is the kernel's address.
constexpr int kLdsWideMaxVec = 66560;
static_assert(sizeof(fm::TopkShared<1024, fm::kVecMaxLds, fm::kTopkBig>) + (size_t)(kLdsWideMaxVec + 8) * 2 <=
                  160 * 1024 - 256,
              "prefixes of the widest row plus the selection state must fit one compute unit's LDS");
template <auto K>
bool allow_wide_lds() {
  return grant_dynamic_lds<K>((kLdsWideMaxVec + 8) * 2);
}
}  // namespace fm_host
