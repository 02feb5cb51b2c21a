// MoE router: softmax + top-k + renormalised weights + per-expert counts + the stable
// (by expert) dispatch permutation, for gfx950.
//
// Reference semantics: forgemind/moe.py:86-91 (softmax -> topk -> renormalise),
// moe.py:52-60 (per-expert histogram), moe.py:232-236 (stable sort of the flat assignments).
// Ties are resolved in the canonical order of forgemind/kernels/topk.py:13-16: equal
// probabilities go to the lowest expert index.
//
// Launches, integer-only bookkeeping:
//   route_group_kernel  L lanes per row (8, 16, 32 or 64 for up to 64, 128, 256, 512 experts),
//                   eight neighbouring experts per lane, so a wave works on 64 / L rows at once
//                   and reads whole rows with 16-byte loads. Group max / sum give the softmax;
//                   the k picks come from order-preserving integer keys in one of three ways
//                   (kSelScan, kSelSorted, kSelCands below). Each 4-wave workgroup
//                   owns a contiguous tile of rows and leaves its expert histogram in
//                   `hist[tile][e]` (and, when asked, a partial row of the statistics).
//   route_stats_kernel  folds the statistics partials in a fixed order (only when asked for).
//   hist_scan_kernel    only for many tiles x many experts: exclusive scan of the histograms
//                   over the tiles, in place, and the expert totals. With statistics the two run
//                   as one launch (route_scan_stats_kernel), and the two auxiliary losses are then
//                   finished by one more workgroup of the permute_kernel launch.
//   permute_kernel  every workgroup takes (or, without the scan, sums) the histograms of the
//                   tiles before it and the expert totals, then walks its own tile in ascending
//                   flat position and gives each assignment the slot
//                     base[e] + (#assignments to e in earlier tiles) + (rank inside the tile),
//                   which is exactly the position a stable sort by expert would assign.
#include "fm_common.hip.h"

using namespace fm;

namespace {

constexpr int kMaxE = 512;
constexpr int kMaxK = 16;             // picks a row; the forms tuned for few picks are built for 8
constexpr int kMaxTiles = 1024;

constexpr int kGroupThreads = 256;    // 4 waves per tile
constexpr int kGE = 8;                // experts a lane holds

// How route_group_kernel selects a row's k experts.
constexpr int kSelScan = 0;     // every pick scans the lane's eight keys afresh (up to four picks)
constexpr int kSelSorted = 1;   // lanes sort their eight pairs first; a pick is the maximum over the lanes' heads
constexpr int kSelCands = 2;    // threshold, then a sort of the few candidates across the lanes

constexpr int kDppXor3 = 0x1B;      // quad_perm:[3,2,1,0]
constexpr int kDppRor8 = 0x128;     // row_ror:8 (lane ^ 8 inside a row of 16)
constexpr int kSwzXor4 = 0x101F;    // ds_swizzle, bit mode: lane ^ 4
constexpr int kSwzXor16 = 0x401F;   // lane ^ 16
constexpr int kSwzXor31 = 0x7C1F;   // lane ^ 31

template <int CTRL>
__device__ __forceinline__ unsigned long long dpp64(unsigned long long v) {
  // (every lane of these patterns has a source lane: no value for missing ones to set up)
  const uint32_t lo = (uint32_t)__builtin_amdgcn_mov_dpp((int)(uint32_t)v, CTRL, 0xf, 0xf, true);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_mov_dpp((int)(uint32_t)(v >> 32), CTRL, 0xf, 0xf, true);
  return ((unsigned long long)hi << 32) | lo;
}
template <int PATTERN>
__device__ __forceinline__ unsigned long long swz64(unsigned long long v) {
  const uint32_t lo = (uint32_t)__builtin_amdgcn_ds_swizzle((int)(uint32_t)v, PATTERN);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_ds_swizzle((int)(uint32_t)(v >> 32), PATTERN);
  return ((unsigned long long)hi << 32) | lo;
}
__device__ __forceinline__ unsigned long long xor64(unsigned long long v, int mask) {
  const uint32_t lo = (uint32_t)__shfl_xor((int)(uint32_t)v, mask, 64);
  const uint32_t hi = (uint32_t)__shfl_xor((int)(uint32_t)(v >> 32), mask, 64);
  return ((unsigned long long)hi << 32) | lo;
}
// one exchange of the network below: the lower lane of a pair keeps the larger value
__device__ __forceinline__ unsigned long long keep(unsigned long long mine, unsigned long long other, bool lower) {
  return ((other > mine) == lower) ? other : mine;
}
// Sorts one 64-bit value per lane over groups of L lanes, largest in the group's first lane: the
// bitonic network in its mirrored form (a merge of 2m lanes starts with lane ^ (2m - 1), then
// lane ^ m/2 ... lane ^ 1), whose exchanges all point the same way, so that every step is one of the
// lane patterns the hardware moves data by (quad permutes, row mirrors, a row rotation, swizzles).
template <int L>
__device__ __forceinline__ unsigned long long group_sort_desc(unsigned long long c, int l) {
  static_assert(L == 16 || L == 32 || L == 64, "groups of 16, 32 or 64 lanes");
  const bool u1 = (l & 1) == 0, u2 = (l & 2) == 0, u4 = (l & 4) == 0, u8 = (l & 8) == 0;
  c = keep(c, dpp64<kDppXor1>(c), u1);
  c = keep(c, dpp64<kDppXor3>(c), u2);
  c = keep(c, dpp64<kDppXor1>(c), u1);
  c = keep(c, dpp64<kDppHalfMirror>(c), u4);
  c = keep(c, dpp64<kDppXor2>(c), u2);
  c = keep(c, dpp64<kDppXor1>(c), u1);
  c = keep(c, dpp64<kDppMirror>(c), u8);
  c = keep(c, swz64<kSwzXor4>(c), u4);
  c = keep(c, dpp64<kDppXor2>(c), u2);
  c = keep(c, dpp64<kDppXor1>(c), u1);
  if constexpr (L >= 32) {
    const bool u16 = (l & 16) == 0;
    c = keep(c, swz64<kSwzXor31>(c), u16);
    c = keep(c, dpp64<kDppRor8>(c), u8);
    c = keep(c, swz64<kSwzXor4>(c), u4);
    c = keep(c, dpp64<kDppXor2>(c), u2);
    c = keep(c, dpp64<kDppXor1>(c), u1);
  }
  if constexpr (L == 64) {
    const bool u16 = (l & 16) == 0, u32 = (l & 32) == 0;
    c = keep(c, xor64(c, 63), u32);
    c = keep(c, swz64<kSwzXor16>(c), u16);
    c = keep(c, dpp64<kDppRor8>(c), u8);
    c = keep(c, swz64<kSwzXor4>(c), u4);
    c = keep(c, dpp64<kDppXor2>(c), u2);
    c = keep(c, dpp64<kDppXor1>(c), u1);
  }
  return c;
}

// Maximum of a float over a group of L lanes, through the integers: the bits of a float, with the
// magnitude of the negative ones inverted, order as signed integers the way the floats do, and an
// integer maximum takes its lane pattern in the same instruction, where the float maximum needs
// three more to fetch and quiet its operand. (A positive NaN wins, a negative one loses: the row
// is a NaN row either way, through its sum.)
template <int L>
__device__ __forceinline__ float group_max_f(float v) {
  auto flip = [](int i) { return i ^ ((i >> 31) & 0x7fffffff); };
  auto mx = [](int a, int b) { return a > b ? a : b; };
  int i = flip(__builtin_bit_cast(int, v));
  i = mx(i, FM_DPP_I(i, kDppXor1));
  i = mx(i, FM_DPP_I(i, kDppXor2));
  i = mx(i, FM_DPP_I(i, kDppHalfMirror));
  if constexpr (L >= 16) i = mx(i, FM_DPP_I(i, kDppMirror));
  if constexpr (L >= 32) i = mx(i, __builtin_amdgcn_ds_swizzle(i, kSwzXor16));
  if constexpr (L == 64) i = mx(i, __shfl_xor(i, 32, 64));
  return __builtin_bit_cast(float, flip(i));
}

// L lanes per row, eight neighbouring experts per lane: a wave works on 64 / L rows at once, reads
// whole rows with 16-byte loads (VEC: e a multiple of eight, aligned buffer) and reduces over L
// lanes only. Ties go to the lowest expert index: the lane keeps its first maximum, the group
// takes the smallest index among the lanes that hold the group's maximum.
// kSelSorted: every lane first sorts its eight (key, expert) pairs with a 19-exchange network, so
// that a pick is the group maximum over the lanes' heads, a ballot for the first lane that holds it
// and a shift in that lane, instead of a fresh scan of the lane's eight keys, a second reduction
// over the tied experts and three selects by position -- about 30 instead of 75 instructions a
// pick. kSelCands (129-256 experts, five picks or more): a cheap lower bound of the k-th key, the
// twenty or so experts at or above it compacted into LDS, one of them per lane, and ONE sort
// across the lanes in place of k rounds. The probability of a pick is read back from its key
// (they are the same bits above the sign), so all forms give identical results (a NaN row's
// weights are NaN either way, with whatever payload).
template <typename T, int L, bool VEC, int SEL, int KMAX = 8>
__global__ __launch_bounds__(kGroupThreads) void route_group_kernel(const T* __restrict__ logits,
                                                                     int32_t* __restrict__ idx,
                                                                     float* __restrict__ weights,
                                                                     int32_t* __restrict__ hist,
                                                                     float* __restrict__ fstat, int64_t n,
                                                                     int e, int k, int tile_rows) {
  static_assert(KMAX <= L && (KMAX == 8 || SEL == kSelSorted), "pick j is kept by lane j of the group; more than 8 picks come from the sorted heads");
  constexpr int NW = kGroupThreads / 64;
  constexpr int GPW = 64 / L;           // rows per wave and pass
  __shared__ int lh[L * kGE];
  __shared__ float wstat[NW][L * kGE];  // per-wave column sums of the probabilities
  __shared__ float wz[NW];              // per-wave sums of logsumexp^2
  constexpr int R = 2;                  // rows per lane group in flight
  // candidate lists (one per row in flight) and their lengths
  __shared__ unsigned long long cand[SEL == kSelCands ? NW * R : 1][SEL == kSelCands ? 64 * kGE : 1];
  __shared__ int ccount[SEL == kSelCands ? NW * R : 1][SEL == kSelCands ? GPW : 1];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane / L, l = lane % L;
  const int ex0 = l * kGE;              // this lane's first expert
  float psum[kGE];
  float zsum = 0.f;
#pragma unroll
  for (int q = 0; q < kGE; ++q) psum[q] = 0.f;
  for (int i = tid; i < L * kGE; i += kGroupThreads) lh[i] = 0;
  __syncthreads();
  const int64_t row0 = (int64_t)blockIdx.x * tile_rows;
  const int64_t row1 = row0 + tile_rows < n ? row0 + tile_rows : n;
  // R rows per lane group are in flight at once so that their dependent reduction chains overlap
  for (int64_t rb = row0 + wave * GPW; rb < row1; rb += (int64_t)NW * GPW * R) {
    int64_t row[R];
    bool live[R];
    float p[R][kGE];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      row[r] = rb + (int64_t)r * NW * GPW + g;
      live[r] = row[r] < row1;
      if constexpr (VEC) {
        constexpr int EPV = Elem<T>::kVec;
        if (live[r] && ex0 < e) {
#pragma unroll
          for (int h = 0; h < kGE / EPV; ++h) {
            float part[EPV];
            Elem<T>::unpack(load16(logits + row[r] * (int64_t)e + ex0 + h * EPV), part);
#pragma unroll
            for (int q = 0; q < EPV; ++q) p[r][h * EPV + q] = part[q];
          }
        } else {
#pragma unroll
          for (int q = 0; q < kGE; ++q) p[r][q] = -INFINITY;
        }
      } else {
#pragma unroll
        for (int q = 0; q < kGE; ++q)
          p[r][q] = (live[r] && ex0 + q < e) ? Elem<T>::load1(logits + row[r] * (int64_t)e + ex0 + q) : -INFINITY;
      }
    }
    float m[R], s[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      m[r] = p[r][0];
#pragma unroll
      for (int q = 1; q < kGE; ++q) m[r] = fmaxf(m[r], p[r][q]);
    }
#pragma unroll
    for (int r = 0; r < R; ++r) m[r] = group_max_f<L>(m[r]);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      s[r] = 0.f;
#pragma unroll
      for (int q = 0; q < kGE; ++q) {
        p[r][q] = fast_exp2((p[r][q] - m[r]) * kLog2e);
        s[r] += p[r][q];
      }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) s[r] = group_reduce<L, OpSum>(s[r]);
    uint32_t key[R][kGE];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      // one division per row: eight IEEE divisions a lane were a quarter of the kernel
      const float inv = 1.f / s[r];
      // A probability is +0 or positive, or the whole row is NaN (a NaN or +inf logit makes the
      // row's sum NaN): its key is its bit pattern with the top bit set, all ones for a NaN row.
      const uint32_t top = (s[r] != s[r]) ? 0xFFFFFFFFu : 0x80000000u;
#pragma unroll
      for (int q = 0; q < kGE; ++q) {
        p[r][q] = p[r][q] * inv;
        const bool real = VEC ? ex0 < e : (ex0 + q) < e;   // whole lanes when rows are vectors
        key[r][q] = real ? (__builtin_bit_cast(uint32_t, p[r][q]) | top) : 0u;   // 0 is below every real key
      }
      if (fstat != nullptr) {
#pragma unroll
        for (int q = 0; q < kGE; ++q) {
          const bool real = VEC ? ex0 < e : (ex0 + q) < e;
          if (live[r] && real) psum[q] += p[r][q];    // rows in ascending order
        }
        if (live[r] && l == 0) {
          const float lse = m[r] + fast_log2(s[r]) * kLn2;
          zsum += lse * lse;
        }
      }
    }
    int my_i[R];
    float my_p[R], wsum[R];
#pragma unroll
    for (int r = 0; r < R; ++r) { my_i[r] = 0; my_p[r] = 0.f; wsum[r] = 0.f; }
    if constexpr (SEL == kSelCands) {
      // Threshold: the lanes with equal l % 8 form eight disjoint sets of experts, none empty (the
      // launcher takes this form only when the row has more than 64 experts); the smallest of the
      // eight set maxima has eight different experts at or above it, so it is a lower bound of
      // the k-th largest key. On rows without long runs of equal keys some twenty experts reach it.
      uint32_t tau[R];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        uint32_t hm = key[r][0];
#pragma unroll
        for (int q = 1; q < kGE; ++q) hm = hm > key[r][q] ? hm : key[r][q];
        auto mx = [](uint32_t a, uint32_t b) { return a > b ? a : b; };
        auto mn = [](uint32_t a, uint32_t b) { return a < b ? a : b; };
        hm = mx(hm, (uint32_t)FM_DPP_I((int)hm, kDppRor8));
        if constexpr (L >= 32) hm = mx(hm, (uint32_t)__builtin_amdgcn_ds_swizzle((int)hm, kSwzXor16));
        if constexpr (L == 64) hm = mx(hm, (uint32_t)__shfl_xor((int)hm, 32, 64));
        hm = mn(hm, (uint32_t)FM_DPP_I((int)hm, kDppXor1));
        hm = mn(hm, (uint32_t)FM_DPP_I((int)hm, kDppXor2));
        hm = mn(hm, (uint32_t)FM_DPP_I((int)hm, kDppHalfMirror));
        tau[r] = hm;
      }
      // The experts at or above the threshold go to the group's list in LDS, in any order, as
      // (key, 65535 - expert): larger is better, equal keys keep the lower expert in front.
      const int gbase = lane & ~(L - 1);
      const int wr0 = wave * R;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        if (l == 0) ccount[wr0 + r][g] = 0;
      }
#pragma unroll
      for (int r = 0; r < R; ++r) {
        int at[kGE];
#pragma unroll
        for (int q = 0; q < kGE; ++q)
          at[q] = (live[r] && key[r][q] >= tau[r]) ? atomicAdd(&ccount[wr0 + r][g], 1) : -1;
#pragma unroll
        for (int q = 0; q < kGE; ++q) {
          if (at[q] >= 0)
            cand[wr0 + r][gbase * kGE + at[q]] =
                ((unsigned long long)key[r][q] << 32) | (uint32_t)(0xFFFF - (ex0 + q));
        }
      }
      // One candidate per lane, sorted across the group: its first k lanes then hold the picks in
      // order. A longer list is taken L - 8 at a time next to the best eight so far.
      int cn[R];
      unsigned long long c[R];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        cn[r] = ccount[wr0 + r][g];
        c[r] = l < cn[r] ? cand[wr0 + r][gbase * kGE + l] : 0ull;
      }
#pragma unroll
      for (int r = 0; r < R; ++r) c[r] = group_sort_desc<L>(c[r], l);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        for (int base = L; __builtin_amdgcn_ballot_w64(base < cn[r]) != 0ull; base += L - 8) {
          const int src = base + l - 8;
          const unsigned long long nx = (l >= 8 && src < cn[r]) ? cand[wr0 + r][gbase * kGE + src] : 0ull;
          c[r] = l < 8 ? c[r] : nx;
          c[r] = group_sort_desc<L>(c[r], l);
        }
      }
#pragma unroll
      for (int r = 0; r < R; ++r) {
        // a probability is never negative: its key is its bit pattern with the top bit set
        // (the all-ones NaN key reads back as a NaN)
        const float pv = __builtin_bit_cast(float, (uint32_t)(c[r] >> 32) & 0x7FFFFFFFu);
        my_p[r] = pv;
        my_i[r] = 0xFFFF - (int)((uint32_t)c[r] & 0xFFFFu);
#pragma unroll
        for (int j = 0; j < KMAX; ++j) {
          if (j < k) wsum[r] += __shfl(pv, gbase + j, 64);   // in pick order, as the other forms add them
        }
      }
    } else if constexpr (SEL == kSelSorted) {
      // (key, kGE - 1 - position) as one 64-bit value: larger is better, equal keys keep the
      // lower expert in front
      unsigned long long c[R][kGE];
#pragma unroll
      for (int r = 0; r < R; ++r) {
#pragma unroll
        for (int q = 0; q < kGE; ++q) c[r][q] = ((unsigned long long)key[r][q] << 32) | (uint32_t)(kGE - 1 - q);
        auto cx = [&](int a, int b) {
          const bool sw = c[r][b] > c[r][a];
          const unsigned long long hi = sw ? c[r][b] : c[r][a];
          c[r][b] = sw ? c[r][a] : c[r][b];
          c[r][a] = hi;
        };
        cx(0, 1); cx(2, 3); cx(4, 5); cx(6, 7);
        cx(0, 2); cx(1, 3); cx(4, 6); cx(5, 7);
        cx(1, 2); cx(5, 6);
        cx(0, 4); cx(1, 5); cx(2, 6); cx(3, 7);
        cx(2, 4); cx(3, 5);
        cx(1, 2); cx(3, 4); cx(5, 6);
      }
      // After the sort the keys stay in registers, head first; the positions are packed four bits
      // apiece into one register (head in the low bits), so that a winning lane moves its list up
      // with eight selects and one shift.
      uint32_t ck[R][kGE], ord[R];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        ord[r] = 0u;
#pragma unroll
        for (int q = 0; q < kGE; ++q) {
          ck[r][q] = (uint32_t)(c[r][q] >> 32);
          ord[r] |= ((uint32_t)c[r][q] & 7u) << (4 * q);
        }
      }
      const int gbase = lane & ~(L - 1);
#pragma unroll
      for (int j = 0; j < KMAX; ++j) {
        if (j < k) {
          uint32_t gk[R];
#pragma unroll
          for (int r = 0; r < R; ++r) gk[r] = group_max_u<L>(ck[r][0]);
#pragma unroll
          for (int r = 0; r < R; ++r) {
            // The lanes of a group hold ascending blocks of experts and a lane's equal keys are in
            // ascending order of expert, so the FIRST lane whose head is the group's maximum holds
            // the lowest expert among the tied ones: one ballot instead of a second reduction.
            const unsigned long long tied = __builtin_amdgcn_ballot_w64(ck[r][0] == gk[r]);
            int first;
            if constexpr (L == 64) {
              first = __builtin_ctzll(tied);
            } else {
              const uint32_t half = gbase >= 32 ? (uint32_t)(tied >> 32) : (uint32_t)tied;
              const uint32_t mine = L == 32 ? half : ((half >> (gbase & 31)) & ((1u << (L & 31)) - 1u));
              first = __builtin_ctz(mine);
            }
            const bool won = first == l;
            // a probability is never negative: its key is its bit pattern with the top bit set
            // (the all-ones NaN key reads back as a NaN)
            const float pv = __builtin_bit_cast(float, gk[r] & 0x7FFFFFFFu);
            wsum[r] += pv;
            if (l == j) my_p[r] = pv;
            if (won) {
              // the winner itself records the pick: no other lane needs to learn the expert
              const int ex = ex0 + (kGE - 1) - (int)(ord[r] & 7u);
              if (live[r]) {
                idx[row[r] * (int64_t)k + j] = ex;
                atomicAdd(&lh[ex], 1);
              }
            }
            if (j + 1 < k) {   // the winning lane moves its next pair to the front
#pragma unroll
              for (int q = 0; q + 1 < kGE; ++q) ck[r][q] = won ? ck[r][q + 1] : ck[r][q];
              ck[r][kGE - 1] = won ? 0u : ck[r][kGE - 1];
              ord[r] = won ? (ord[r] >> 4) : ord[r];
            }
          }
        }
      }
    } else {
#pragma unroll
    for (int j = 0; j < KMAX; ++j) {
      if (j < k) {
        uint32_t bk[R], gk[R];
        int bq[R], gi[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
          bk[r] = key[r][0];
          bq[r] = 0;
#pragma unroll
          for (int q = 1; q < kGE; ++q) {
            if (key[r][q] > bk[r]) { bk[r] = key[r][q]; bq[r] = q; }
          }
        }
#pragma unroll
        for (int r = 0; r < R; ++r) gk[r] = group_max_u<L>(bk[r]);
#pragma unroll
        for (int r = 0; r < R; ++r) gi[r] = group_min_i<L>((bk[r] == gk[r]) ? ex0 + bq[r] : 0x7fffffff);
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const int wl = gi[r] >> 3, wq = gi[r] & 7;
          float pv = p[r][0];
#pragma unroll
          for (int q = 1; q < kGE; ++q) pv = (q == wq) ? p[r][q] : pv;
          pv = __shfl(pv, (lane & ~(L - 1)) + wl, 64);
#pragma unroll
          for (int q = 0; q < kGE; ++q) {
            if (l == wl && q == wq) key[r][q] = 0u;
          }
          wsum[r] += pv;
          if (l == j) { my_i[r] = gi[r]; my_p[r] = pv; }
        }
      }
    }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      if (live[r] && l < k) {
        weights[row[r] * (int64_t)k + l] = my_p[r] / wsum[r];
        if constexpr (SEL != kSelSorted) {   // (the sorted form's winners have stored these themselves)
          idx[row[r] * (int64_t)k + l] = my_i[r];
          atomicAdd(&lh[my_i[r]], 1);
        }
      }
    }
  }
  if (fstat != nullptr) {
    // fold the wave's row groups (lanes l, l + L, ...) in group order, then the waves
#pragma unroll
    for (int q = 0; q < kGE; ++q) {
      float a = psum[q];
#pragma unroll
      for (int o = L; o < 64; o <<= 1) a += __shfl_xor(a, o, 64);
      psum[q] = a;
    }
    zsum = wave_sum(zsum);
    if (g == 0) {
#pragma unroll
      for (int q = 0; q < kGE; ++q) wstat[wave][ex0 + q] = psum[q];
    }
    if (lane == 0) wz[wave] = zsum;
  }
  __syncthreads();
  for (int i = tid; i < e; i += kGroupThreads) hist[(int64_t)blockIdx.x * e + i] = lh[i];
  if (fstat != nullptr) {   // fold the waves in wave order: one fp32 partial row per tile
    float* out = fstat + (int64_t)blockIdx.x * (e + 1);
    for (int i = tid; i < e; i += kGroupThreads) {
      float a = wstat[0][i];
#pragma unroll
      for (int w = 1; w < NW; ++w) a += wstat[w][i];
      out[i] = a;
    }
    if (tid == 0) {
      float a = wz[0];
#pragma unroll
      for (int w = 1; w < NW; ++w) a += wz[w];
      out[e] = a;
    }
  }
}

// Gradient of the routing outputs wrt the logits, one pass over [n, e] with the lane groups of
// route_group_kernel (one row per group): the softmax is recomputed, then
//   through the renormalised top-k weights  w_j = p[idx_j] / S,  S = sum_j p[idx_j]:
//     g_p[idx_j] = (gw_j - sum_i gw_i w_i) / S
//   through aux = E * sum_e frac_e * mean_rows(p)_e  (frac = counts / (n k), a constant):
//     g_p[e] += g_aux * E / n * frac_e
//   through the softmax:  g_x = (g_p - sum_e g_p p) p
//   through z = mean(lse^2):  g_x += g_z * 2 / n * lse * p.
template <typename T, int L, bool VEC>
__global__ __launch_bounds__(kGroupThreads) void route_bwd_kernel(const T* __restrict__ logits,
                                                                   const int32_t* __restrict__ idx,
                                                                   const float* __restrict__ gw,
                                                                   const int32_t* __restrict__ counts,
                                                                   const float* __restrict__ g_aux,
                                                                   const float* __restrict__ g_z,
                                                                   T* __restrict__ dlogits, int64_t n,
                                                                   int e, int k) {
  constexpr int GPW = 64 / L;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane / L, l = lane % L;
  const int ex0 = l * kGE;
  const float ca = (g_aux != nullptr && counts != nullptr) ? *g_aux * (float)e / (float)n : 0.f;
  const float cz = g_z != nullptr ? *g_z * 2.f / (float)n : 0.f;
  float fr[kGE];
#pragma unroll
  for (int q = 0; q < kGE; ++q)
    fr[q] = (ca != 0.f && ex0 + q < e) ? ca * ((float)counts[ex0 + q] / (float)(n * (int64_t)k)) : 0.f;
  const int64_t row = ((int64_t)blockIdx.x * (kGroupThreads / 64) + wave) * GPW + g;
  const bool live = row < n;
  float p[kGE];
  if constexpr (VEC) {
    constexpr int EPV = Elem<T>::kVec;
    if (live && ex0 < e) {
#pragma unroll
      for (int h = 0; h < kGE / EPV; ++h) {
        float part[EPV];
        Elem<T>::unpack(load16(logits + row * (int64_t)e + ex0 + h * EPV), part);
#pragma unroll
        for (int q = 0; q < EPV; ++q) p[h * EPV + q] = part[q];
      }
    } else {
#pragma unroll
      for (int q = 0; q < kGE; ++q) p[q] = -INFINITY;
    }
  } else {
#pragma unroll
    for (int q = 0; q < kGE; ++q)
      p[q] = (live && ex0 + q < e) ? Elem<T>::load1(logits + row * (int64_t)e + ex0 + q) : -INFINITY;
  }
  float m = p[0];
#pragma unroll
  for (int q = 1; q < kGE; ++q) m = fmaxf(m, p[q]);
  m = group_reduce<L, OpMax>(m);
  float s = 0.f;
#pragma unroll
  for (int q = 0; q < kGE; ++q) {
    p[q] = fast_exp2((p[q] - m) * kLog2e);
    s += p[q];
  }
  s = group_reduce<L, OpSum>(s);
  const float inv = 1.f / s;
  const float lse = m + fast_log2(s) * kLn2;
#pragma unroll
  for (int q = 0; q < kGE; ++q) p[q] *= inv;
  // the selected experts of this row and the gradients of their weights
  float gsel[kGE];
  bool sel[kGE];
#pragma unroll
  for (int q = 0; q < kGE; ++q) { gsel[q] = 0.f; sel[q] = false; }
  float s_loc = 0.f, d_loc = 0.f;
#pragma unroll
  for (int j = 0; j < kMaxK; ++j) {
    if (j >= k) break;
    if (live) {
      const int ij = idx[row * (int64_t)k + j];
      const float gj = gw != nullptr ? gw[row * (int64_t)k + j] : 0.f;
#pragma unroll
      for (int q = 0; q < kGE; ++q) {
        if (ij == ex0 + q) {
          sel[q] = true;
          gsel[q] = gj;
          s_loc += p[q];
          d_loc += gj * p[q];
        }
      }
    }
  }
  const float S = group_reduce<L, OpSum>(s_loc);
  const float D = group_reduce<L, OpSum>(d_loc);
  const float inv_s = 1.f / S;
  const float mean = D * inv_s;
  float gp[kGE];
  float dot = 0.f;
#pragma unroll
  for (int q = 0; q < kGE; ++q) {
    gp[q] = (sel[q] ? (gsel[q] - mean) * inv_s : 0.f) + fr[q];
    dot += gp[q] * p[q];
  }
  dot = group_reduce<L, OpSum>(dot);
  float o[kGE];
#pragma unroll
  for (int q = 0; q < kGE; ++q) o[q] = (gp[q] - dot) * p[q] + cz * lse * p[q];
  if (!live) return;
  T* op = dlogits + row * (int64_t)e + ex0;
  if constexpr (VEC) {
    constexpr int EPV = Elem<T>::kVec;
    if (ex0 < e) {
#pragma unroll
      for (int h = 0; h < kGE / EPV; ++h) {
        float part[EPV];
#pragma unroll
        for (int q = 0; q < EPV; ++q) part[q] = o[h * EPV + q];
        store16(op + h * EPV, Elem<T>::pack(part));
      }
    }
  } else {
#pragma unroll
    for (int q = 0; q < kGE; ++q)
      if (ex0 + q < e) Elem<T>::store1(op + q, o[q]);
  }
}

// Sums the per-tile partial rows [ntiles, e+1]: stats[0..e) = column sums of the probabilities,
// stats[e] = sum of logsumexp^2. A workgroup owns 64 columns; wave w adds tiles w, w + 16, ...
// of a column in that order, then the sixteen partial sums are added in wave order. The order
// depends on ntiles only, so equal inputs give equal bits.
__device__ __forceinline__ void stats_fold_block(const float* __restrict__ fstat, float* __restrict__ stats,
                                                 int e, int ntiles, int block, float (*part)[64]) {
  const int cols = e + 1;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = block * 64 + lane;
  float a = 0.f;
  if (c < cols) {
    // sixteen loads in flight; the additions stay in tile order
    int t = wave;
    for (; t + 15 * 16 < ntiles; t += 16 * 16) {
      float v[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) v[u] = fstat[(int64_t)(t + u * 16) * cols + c];
#pragma unroll
      for (int u = 0; u < 16; ++u) a += v[u];
    }
    for (; t < ntiles; t += 16) a += fstat[(int64_t)t * cols + c];
  }
  part[wave][lane] = a;
  __syncthreads();
  if (wave == 0 && c < cols) {
    float r = part[0][lane];
#pragma unroll
    for (int w = 1; w < 16; ++w) r += part[w][lane];
    stats[c] = r;
  }
}

__global__ __launch_bounds__(1024) void route_stats_kernel(const float* __restrict__ fstat,
                                                            float* __restrict__ stats, int e,
                                                            int ntiles) {
  __shared__ float part[16][64];
  stats_fold_block(fstat, stats, e, ntiles, (int)blockIdx.x, part);
}

// Exclusive scan of the tile histograms over the tiles, in place: hist[t][c] becomes the number
// of assignments to expert c in tiles before t, counts[c] their total. A workgroup owns 16
// experts; thread (s, c) walks tiles s * per, ..., (s + 1) * per - 1 of expert c.
__device__ __forceinline__ void hist_scan_block(int32_t* __restrict__ hist, int32_t* __restrict__ counts,
                                                int e, int ntiles, int block, int (*seg)[17]) {
  const int c = threadIdx.x & 15, sgm = threadIdx.x >> 4;
  const int col = block * 16 + c;
  constexpr int kPer = kMaxTiles / 64;   // tiles per segment at most
  const int per = (ntiles + 63) / 64;
  const int t0 = sgm * per;
  int v[kPer];
  int sum = 0;
#pragma unroll
  for (int u = 0; u < kPer; ++u) {
    const int t = t0 + u;
    v[u] = (col < e && u < per && t < ntiles) ? hist[(int64_t)t * e + col] : 0;
  }
#pragma unroll
  for (int u = 0; u < kPer; ++u) sum += v[u];
  seg[sgm][c] = sum;
  __syncthreads();
  if (threadIdx.x < 16) {       // one thread per expert: exclusive scan of its 64 segment sums
    int run = 0;
    for (int q = 0; q < 64; ++q) {
      const int w = seg[q][threadIdx.x];
      seg[q][threadIdx.x] = run;
      run += w;
    }
    if (block * 16 + (int)threadIdx.x < e) counts[block * 16 + threadIdx.x] = run;
  }
  __syncthreads();
  int run = seg[sgm][c];
#pragma unroll
  for (int u = 0; u < kPer; ++u) {
    const int t = t0 + u;
    if (col < e && u < per && t < ntiles) hist[(int64_t)t * e + col] = run;
    run += v[u];
  }
}

__global__ __launch_bounds__(1024) void hist_scan_kernel(int32_t* __restrict__ hist,
                                                          int32_t* __restrict__ counts, int e,
                                                          int ntiles) {
  __shared__ int seg[64][17];
  hist_scan_block(hist, counts, e, ntiles, (int)blockIdx.x, seg);
}

// The scan of the histograms and the fold of the statistics need nothing of each other: one
// launch, the first `scan_blocks` workgroups scan, the others fold.
__global__ __launch_bounds__(1024) void route_scan_stats_kernel(int32_t* __restrict__ hist,
                                                                 int32_t* __restrict__ counts,
                                                                 const float* __restrict__ fstat,
                                                                 float* __restrict__ stats, int e,
                                                                 int ntiles, int scan_blocks) {
  __shared__ int seg[64][17];
  __shared__ float part[16][64];
  if ((int)blockIdx.x < scan_blocks) hist_scan_block(hist, counts, e, ntiles, (int)blockIdx.x, seg);
  else stats_fold_block(fstat, stats, e, ntiles, (int)blockIdx.x - scan_blocks, part);
}

// The two auxiliary losses from the finished sums (forgemind/moe.py:92-95), one workgroup:
//   stats[e + 1] = aux = E * sum_c counts[c] / (n k) * stats[c] / n
//   stats[e + 2] = z   = stats[e] / n
__global__ __launch_bounds__(512) void route_aux_kernel(const int32_t* __restrict__ counts,
                                                         float* __restrict__ stats, int64_t n, int e,
                                                         int k) {
  __shared__ float part[8];
  const int c = threadIdx.x;
  const float rows = n > 0 ? (float)n : 1.f;
  const float slots = n > 0 ? (float)(n * (int64_t)k) : 1.f;
  float a = c < e ? ((float)counts[c] / slots) * (stats[c] / rows) : 0.f;
  a = wave_sum(a);
  if ((c & 63) == 0) part[c >> 6] = a;
  __syncthreads();
  if (c == 0) {
    float t = part[0];
#pragma unroll
    for (int w = 1; w < 8; ++w) t += part[w];
    stats[e + 1] = (float)e * t;
    stats[e + 2] = stats[e] / rows;
  }
}

// route_aux_kernel's arithmetic from a workgroup of 256 threads (the extra workgroup of a
// permute_kernel launch): every wave stands in for two of that kernel's eight, so the sums are
// formed from the same values in the same order.
__device__ __forceinline__ void aux_block_256(const int32_t* counts, float* __restrict__ stats, int64_t n,
                                              int e, int k) {
  __shared__ float part[8];
  const float rows = n > 0 ? (float)n : 1.f;
  const float slots = n > 0 ? (float)(n * (int64_t)k) : 1.f;
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    const int c = half * 256 + (int)threadIdx.x;
    float a = c < e ? ((float)counts[c] / slots) * (stats[c] / rows) : 0.f;
    a = wave_sum(a);
    if ((c & 63) == 0) part[c >> 6] = a;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    float t = part[0];
#pragma unroll
    for (int w = 1; w < 8; ++w) t += part[w];
    stats[e + 1] = (float)e * t;
    stats[e + 2] = stats[e] / rows;
  }
}

// route_stats_kernel and route_aux_kernel in one launch for small problems (at most two column
// blocks and 256 tiles): one workgroup folds the column blocks one after the other, in the same
// order and with the same additions as route_stats_kernel, keeps the sums in LDS and finishes
// with route_aux_kernel's arithmetic. Same bits as the two kernels, one launch fewer.
__global__ __launch_bounds__(1024) void route_stats_aux_kernel(const float* __restrict__ fstat,
                                                                const int32_t* __restrict__ counts,
                                                                float* __restrict__ stats, int64_t n,
                                                                int e, int k, int ntiles) {
  __shared__ float part[16][64];
  __shared__ float sums[2 * 64];
  __shared__ float apart[8];
  const int cols = e + 1;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int cb = 0; cb * 64 < cols; ++cb) {
    const int c = cb * 64 + lane;
    float a = 0.f;
    if (c < cols) {
      int t = wave;
      for (; t + 15 * 16 < ntiles; t += 16 * 16) {
        float v[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) v[u] = fstat[(int64_t)(t + u * 16) * cols + c];
#pragma unroll
        for (int u = 0; u < 16; ++u) a += v[u];
      }
      for (; t < ntiles; t += 16) a += fstat[(int64_t)t * cols + c];
    }
    part[wave][lane] = a;
    __syncthreads();
    if (wave == 0 && c < cols) {
      float r = part[0][lane];
#pragma unroll
      for (int w = 1; w < 16; ++w) r += part[w][lane];
      stats[c] = r;
      sums[c] = r;
    }
    __syncthreads();
  }
  const int c = threadIdx.x;
  const float rows = n > 0 ? (float)n : 1.f;
  const float slots = n > 0 ? (float)(n * (int64_t)k) : 1.f;
  if (c < 512) {
    float a = c < e ? ((float)counts[c] / slots) * (sums[c] / rows) : 0.f;
    a = wave_sum(a);
    if ((c & 63) == 0) apart[c >> 6] = a;
  }
  __syncthreads();
  if (c == 0) {
    float t = apart[0];
#pragma unroll
    for (int w = 1; w < 8; ++w) t += apart[w];
    stats[e + 1] = (float)e * t;
    stats[e + 2] = sums[e] / rows;
  }
}

typedef int i32x4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void permute_kernel(const int32_t* __restrict__ idx,
                                                       const int32_t* __restrict__ hist,
                                                       int32_t* counts,
                                                       int32_t* __restrict__ slot,
                                                       int32_t* __restrict__ order, int64_t n, int e,
                                                       int k, int tile_rows, int ntiles, int emit,
                                                       int scanned, float* aux_stats) {
  // partial sums of the tile histograms: [group][expert], "before my tile" and "all tiles"
  __shared__ int part_b[4 * kMaxE];   // flat [group][e]; groups * e <= 4 * kMaxE on every path
  __shared__ int part_t[4 * kMaxE];
  __shared__ int total[kMaxE];
  __shared__ int offs[kMaxE];      // next free slot of each expert for this tile
  __shared__ unsigned long long wmask[4][kMaxE];   // per wave and expert: the lanes assigned to it (current chunk)
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int me = blockIdx.x;
  if (aux_stats != nullptr && me == (int)gridDim.x - 1) {
    // one workgroup past the tiles finishes the two losses (the scanned totals and the folded
    // statistics are both complete before this launch starts)
    aux_block_256(counts, aux_stats, n, e, k);
    return;
  }

  // the first chunk of this tile's assignments is fetched now, under the histogram loads
  const int64_t p0 = (int64_t)me * tile_rows * k;
  int64_t p1 = p0 + (int64_t)tile_rows * k;
  const int64_t pend = n * (int64_t)k;
  if (p1 > pend) p1 = pend;
  int ex_next = (emit && p0 + tid < p1) ? idx[p0 + tid] : -1;

  const int e4 = e >> 2;
  int groups;
  if (scanned) {
    // hist already holds "before my tile" and counts the totals (hist_scan_kernel)
    groups = 1;
    for (int col = tid; col < e; col += 256) {
      part_b[col] = hist[(int64_t)me * e + col];
      part_t[col] = counts[col];
    }
  } else if ((e & 3) == 0 && e4 <= 256 && (e4 & (e4 - 1)) == 0) {
    // 16-byte loads: a thread keeps four neighbouring experts and walks tiles g, g+groups, ...
    groups = 256 / e4;
    if (groups > 16) groups = 16;
    const int col4 = tid % e4, g = tid / e4;
    i32x4 bef = {0, 0, 0, 0}, tot = {0, 0, 0, 0};
    if (g < groups) {
      const i32x4* h4 = reinterpret_cast<const i32x4*>(hist);
      int t = g;
      for (; t + 7 * groups < ntiles; t += 8 * groups) {
        i32x4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = h4[(int64_t)(t + u * groups) * e4 + col4];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          tot += v[u];
          if (t + u * groups < me) bef += v[u];
        }
      }
      for (; t < ntiles; t += groups) {
        const i32x4 v = h4[(int64_t)t * e4 + col4];
        tot += v;
        if (t < me) bef += v;
      }
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        part_b[g * e + col4 * 4 + c] = bef[c];
        part_t[g * e + col4 * 4 + c] = tot[c];
      }
    }
  } else {
    groups = 4;
    for (int c0 = 0; c0 < e; c0 += 64) {
      const int col = c0 + lane;
      int bef = 0, tot = 0;
      if (col < e) {
        for (int t = wave; t < ntiles; t += 4) {
          const int h = hist[(int64_t)t * e + col];
          tot += h;
          bef += t < me ? h : 0;
        }
        part_b[wave * e + col] = bef;
        part_t[wave * e + col] = tot;
      }
    }
  }
  for (int i = tid; i < 4 * kMaxE; i += 256) (&wmask[0][0])[i] = 0ull;
  __syncthreads();
  for (int col = tid; col < e; col += 256) {
    int tb = 0, tt = 0;
    for (int g = 0; g < groups; ++g) { tb += part_b[g * e + col]; tt += part_t[g * e + col]; }
    total[col] = tt;
    offs[col] = tb;
  }
  __syncthreads();
  // exclusive prefix of the expert totals: wave scan per 64 experts, chunks chained in order
  {
    int carry = 0;
    for (int c0 = 0; c0 < e; c0 += 64) {          // every wave walks all chunks (e <= 512)
      const int col = c0 + lane;
      const int v = col < e ? total[col] : 0;
      int inc = v;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const int up = __shfl_up(inc, o, 64);
        if (lane >= o) inc += up;
      }
      if (wave == 0 && col < e) {
        offs[col] += carry + inc - v;
        if (me == 0 && !scanned) counts[col] = v;
      }
      carry += __builtin_amdgcn_readlane(inc, 63);
    }
  }
  __syncthreads();
  if (!emit) return;

  for (int64_t c0 = p0; c0 < p1; c0 += 256) {
    const int64_t p = c0 + tid;
    const bool act = p < p1;
    const int ex = ex_next;
    ex_next = (p + 256 < p1) ? idx[p + 256] : -1;
    // rank among equal experts inside the wave, in lane (= flat position) order: the lanes of
    // an expert as a bit mask (the mask does not depend on the order the atomics land in)
    if (act) atomicOr(&wmask[wave][ex], 1ull << lane);
    __syncthreads();
    if (act) {
      const int rank = __builtin_popcountll(wmask[wave][ex] & ((1ull << lane) - 1ull));
      int prior = offs[ex];
      for (int w = 0; w < wave; ++w) prior += __builtin_popcountll(wmask[w][ex]);
      const int s = prior + rank;
      if (slot != nullptr) slot[p] = s;
      if (order != nullptr) order[s] = (int32_t)p;
    }
    __syncthreads();
    for (int col = tid; col < e; col += 256) {
      offs[col] += (__builtin_popcountll(wmask[0][col]) + __builtin_popcountll(wmask[1][col])) +
                   (__builtin_popcountll(wmask[2][col]) + __builtin_popcountll(wmask[3][col]));
      wmask[0][col] = 0ull; wmask[1][col] = 0ull; wmask[2][col] = 0ull; wmask[3][col] = 0ull;
    }
    __syncthreads();
  }
}

struct Tiling {
  int tile_rows;
  int ntiles;
};

Tiling make_tiling(int64_t n) {
  Tiling t;
  int64_t rows = 64;
  if ((n + rows - 1) / rows > kMaxTiles) rows = (n + kMaxTiles - 1) / kMaxTiles;
  rows = (rows + 15) / 16 * 16;
  t.tile_rows = (int)rows;
  t.ntiles = (int)((n + rows - 1) / rows);
  if (t.ntiles < 1) t.ntiles = 1;
  return t;
}

template <typename T>
int launch_route(const void* logits, int32_t* idx, float* weights, int32_t* hist, float* fstat,
                 int64_t n, int e, int k, const Tiling& tl, hipStream_t st) {
  const T* lp = static_cast<const T*>(logits);
  const dim3 grid((unsigned)tl.ntiles);
#define GOS(L_, VEC_, SEL_)                                                                           \
  FM_LAUNCH((route_group_kernel<T, L_, VEC_, SEL_>), grid, dim3(kGroupThreads), 0, st, lp, idx, weights, \
            hist, fstat, n, e, k, tl.tile_rows)
#define GOG(L_)                                                                                       \
  do {                                                                                                \
    if (vec && sel == kSelSorted) GOS(L_, true, kSelSorted);                                          \
    else if (vec) GOS(L_, true, kSelScan);                                                            \
    else if (sel == kSelSorted) GOS(L_, false, kSelSorted);                                           \
    else GOS(L_, false, kSelScan);                                                                    \
  } while (0)
  const bool vec = e % kGE == 0 && fm_host::aligned16(logits);
  // Kernel time at 65536 rows, fp32, by picks (1 / 2 / 4 / 8), in microseconds:
  //   128 experts: scan 15 / 17 / 21 / 27, sorted heads 17 / 18 / 20 / 22, candidates 24 at all four
  //   256 experts: scan 22 / 26 / 33 / 46, sorted heads 27 / 28 / 31 / 35, candidates 31 at all four
  //   512 experts (32768 rows): scan 25 / 29 / 38 / 56, sorted heads 30 / 32 / 35 / 43, candidates 42-44
  // Up to 64 experts the scan and the sorted heads tie at four picks.
  const int sel = k >= (e > 64 ? 4 : 5) ? kSelSorted : kSelScan;
  if (k > 8) {
    // more picks than the forms above are built for: sorted heads, 16 lanes a row at the least
    // (lane j of a group keeps pick j)
#define GOK(L_)                                                                                       \
  do {                                                                                                \
    if (vec)                                                                                          \
      FM_LAUNCH((route_group_kernel<T, L_, true, kSelSorted, 16>), grid, dim3(kGroupThreads), 0, st, lp, idx, \
                weights, hist, fstat, n, e, k, tl.tile_rows);                                         \
    else                                                                                              \
      FM_LAUNCH((route_group_kernel<T, L_, false, kSelSorted, 16>), grid, dim3(kGroupThreads), 0, st, lp, idx, \
                weights, hist, fstat, n, e, k, tl.tile_rows);                                         \
  } while (0)
    if (e <= 128) GOK(16);
    else if (e <= 256) GOK(32);
    else GOK(64);
#undef GOK
  } else if (e <= 64) GOG(8);
  else if (e <= 128) GOG(16);
  else if (e <= 256) {
    if (k >= 5 && vec) GOS(32, true, kSelCands);
    else if (k >= 5) GOS(32, false, kSelCands);
    else GOG(32);
  } else GOG(64);
#undef GOS
#undef GOG
  return FM_OK;
}

}  // namespace

extern "C" {

size_t fm_route_workspace(int64_t n, int e, int k) {
  (void)k;
  if (n < 0 || e <= 0) return 0;
  const Tiling tl = make_tiling(n);
  // [ntiles, e] int32 histograms, then [ntiles, e+1] fp32 statistics partials
  return (size_t)tl.ntiles * ((size_t)e * sizeof(int32_t) + (size_t)(e + 1) * sizeof(float));
}

int fm_route(const void* logits, int32_t* idx, float* weights, int32_t* counts, int32_t* slot,
             int32_t* order, float* stats, void* workspace, size_t workspace_bytes, int64_t n, int e,
             int k, int dtype, fm_stream_t stream) {
  FM_CHECK_ARG(n >= 0 && e > 0 && k >= 1, "fm_route: bad shape n=%lld e=%d k=%d", (long long)n, e, k);
  FM_CHECK_ARG(dtype == FM_F32 || dtype == FM_F16 || dtype == FM_BF16, "fm_route: bad dtype %d", dtype);
  FM_CHECK_ARG(k <= e, "fm_route: selected index k out of range (got %d vs %d)", k, e);
  if (e > kMaxE || k > kMaxK || n * (int64_t)k >= 0x7fffffffLL) {
    fm_host::set_error("fm_route: e <= %d, k <= %d and n*k < 2^31 required (e=%d k=%d n=%lld)", kMaxE,
                       kMaxK, e, k, (long long)n);
    return FM_ERR_UNSUPPORTED;
  }
  FM_CHECK_ARG(counts != nullptr, "fm_route: NULL counts");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const Tiling tl = make_tiling(n);
  const size_t hist_bytes = (size_t)tl.ntiles * (size_t)e * sizeof(int32_t);
  const size_t need = hist_bytes + (size_t)tl.ntiles * (size_t)(e + 1) * sizeof(float);
  if (workspace == nullptr || workspace_bytes < need) {
    fm_host::set_error("fm_route: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    return FM_ERR_WORKSPACE;
  }
  FM_CHECK_ARG(n == 0 || (logits && idx && weights), "fm_route: NULL pointer");
  int32_t* hist = static_cast<int32_t*>(workspace);
  float* fstat = stats != nullptr
                     ? reinterpret_cast<float*>(static_cast<char*>(workspace) + hist_bytes)
                     : nullptr;
  // with n == 0 the single tile has no rows and leaves all-zero partials
  if (dtype == FM_F32) launch_route<float>(logits, idx, weights, hist, fstat, n, e, k, tl, st);
  else if (dtype == FM_BF16) launch_route<bf16_t>(logits, idx, weights, hist, fstat, n, e, k, tl, st);
  else launch_route<f16_t>(logits, idx, weights, hist, fstat, n, e, k, tl, st);
  FM_CHECK_LAUNCH("fm_route");
  // few columns and tiles: the statistics are folded by the kernel that also finishes the losses
  const bool stats_late = stats != nullptr && e + 1 <= 128 && tl.ntiles <= 256;
  const int emit = (slot != nullptr || order != nullptr) && n > 0 ? 1 : 0;
  // Many tiles times many experts: every permutation workgroup summing all histograms before
  // its own would read ntiles^2 * e integers in total; scan them once instead.
  const int scanned = (int64_t)tl.ntiles * e > 32768 ? 1 : 0;
  const bool fold = stats != nullptr && !stats_late;
  const unsigned scan_blocks = (unsigned)((e + 15) / 16), fold_blocks = (unsigned)((e + 1 + 63) / 64);
  if (fold && scanned) {
    hipLaunchKernelGGL(route_scan_stats_kernel, dim3(scan_blocks + fold_blocks), dim3(1024), 0, st, hist, counts,
                       fstat, stats, e, tl.ntiles, (int)scan_blocks);
    FM_CHECK_LAUNCH("fm_route(scan + stats)");
  } else if (fold) {
    hipLaunchKernelGGL(route_stats_kernel, dim3(fold_blocks), dim3(1024), 0, st, fstat, stats, e, tl.ntiles);
    FM_CHECK_LAUNCH("fm_route(stats)");
  } else if (scanned) {
    hipLaunchKernelGGL(hist_scan_kernel, dim3(scan_blocks), dim3(1024), 0, st, hist, counts, e, tl.ntiles);
    FM_CHECK_LAUNCH("fm_route(scan)");
  }
  // after a scan the totals are final before the permutation starts: its launch takes one more
  // workgroup for the two losses
  const bool aux_inside = fold && scanned && emit;
  if (emit || !scanned) {
    hipLaunchKernelGGL(permute_kernel, dim3((emit ? (unsigned)tl.ntiles : 1u) + (aux_inside ? 1u : 0u)), dim3(256), 0,
                       st, idx, hist, counts, slot, order, n, e, k, tl.tile_rows, tl.ntiles, emit, scanned,
                       aux_inside ? stats : nullptr);
  }
  FM_CHECK_LAUNCH("fm_route(permute)");
  if (stats_late) {
    hipLaunchKernelGGL(route_stats_aux_kernel, dim3(1), dim3(1024), 0, st, fstat, counts, stats, n, e, k,
                       tl.ntiles);
    FM_CHECK_LAUNCH("fm_route(stats + aux)");
  } else if (stats != nullptr && !aux_inside) {
    hipLaunchKernelGGL(route_aux_kernel, dim3(1), dim3(512), 0, st, counts, stats, n, e, k);
    FM_CHECK_LAUNCH("fm_route(aux)");
  }
  return FM_OK;
}

int fm_route_bwd(const void* logits, const int32_t* idx, const float* gweights, const int32_t* counts,
                 const float* g_aux, const float* g_z, void* dlogits, int64_t n, int e, int k, int dtype,
                 fm_stream_t stream) {
  FM_CHECK_ARG(n >= 0 && e > 0 && k >= 1, "fm_route_bwd: bad shape n=%lld e=%d k=%d", (long long)n, e, k);
  FM_CHECK_ARG(dtype == FM_F32 || dtype == FM_F16 || dtype == FM_BF16, "fm_route_bwd: bad dtype %d", dtype);
  FM_CHECK_ARG(k <= e, "fm_route_bwd: selected index k out of range (got %d vs %d)", k, e);
  if (e > kMaxE || k > kMaxK || n * (int64_t)k >= 0x7fffffffLL) {
    fm_host::set_error("fm_route_bwd: e <= %d, k <= %d and n*k < 2^31 required (e=%d k=%d n=%lld)", kMaxE,
                       kMaxK, e, k, (long long)n);
    return FM_ERR_UNSUPPORTED;
  }
  FM_CHECK_ARG(g_aux == nullptr || counts != nullptr, "fm_route_bwd: g_aux needs counts");
  if (n == 0) return FM_OK;
  FM_CHECK_ARG(logits && idx && dlogits, "fm_route_bwd: NULL pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool vec = e % kGE == 0 && fm_host::aligned16(logits) && fm_host::aligned16(dlogits);
#define GOB(T, L_)                                                                                   \
  do {                                                                                               \
    constexpr int rows_per_block = (kGroupThreads / 64) * (64 / L_);                                 \
    const dim3 grid((unsigned)((n + rows_per_block - 1) / rows_per_block));                          \
    if (vec) FM_LAUNCH((route_bwd_kernel<T, L_, true>), grid, dim3(kGroupThreads), 0, st,   \
                                static_cast<const T*>(logits), idx, gweights, counts, g_aux, g_z,    \
                                static_cast<T*>(dlogits), n, e, k);                                  \
    else FM_LAUNCH((route_bwd_kernel<T, L_, false>), grid, dim3(kGroupThreads), 0, st,      \
                            static_cast<const T*>(logits), idx, gweights, counts, g_aux, g_z,        \
                            static_cast<T*>(dlogits), n, e, k);                                      \
  } while (0)
#define BY_L(T)                 \
  do {                          \
    if (e <= 64) GOB(T, 8);     \
    else if (e <= 128) GOB(T, 16); \
    else if (e <= 256) GOB(T, 32); \
    else GOB(T, 64);            \
  } while (0)
  if (dtype == FM_F32) BY_L(float);
  else if (dtype == FM_BF16) BY_L(bf16_t);
  else BY_L(f16_t);
#undef BY_L
#undef GOB
  FM_CHECK_LAUNCH("fm_route_bwd");
  return FM_OK;
}

}  // extern "C"
