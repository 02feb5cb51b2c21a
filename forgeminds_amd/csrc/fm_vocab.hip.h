// Helpers for kernels that give one workgroup a whole vocabulary-wide row
// (cross entropy, KL, softmax, top-k).
//
// A row of v elements starts at element offset row*v of a 16-byte aligned tensor, so the
// row itself is 16-byte aligned only when row*v is a multiple of the vector width. RowSplit
// peels the row into (unaligned head, whole 16-byte vectors, tail) so that vocabularies such
// as 50257 still stream through 16-byte accesses; because every tensor of one call shares
// the element offset, the same split is valid for all of them, whatever their dtypes.
#pragma once

#include "fm_common.hip.h"

namespace fm {

struct RowSplit {
  int head;   // scalar elements before the first aligned vector (always < EPV)
  int nvec;   // whole vectors of EPV elements (0 when vectors are off)
  int tail0;  // first element of the scalar tail, [tail0, v) (0 when vectors are off)
};

template <int EPV>
__device__ __forceinline__ RowSplit split_row(int64_t row, int v, bool vec_ok) {
  RowSplit s;
  if (!vec_ok) {  // every element is a scalar "tail" element
    s.head = 0; s.nvec = 0; s.tail0 = 0;
    return s;
  }
  int head = (int)((EPV - ((row * (int64_t)v) % EPV)) % EPV);
  if (head > v) head = v;
  s.head = head;
  s.nvec = (v - head) / EPV;
  s.tail0 = head + s.nvec * EPV;
  return s;
}

// Number of scalar "edge" elements (head + tail) and the column of the e-th one.
__device__ __forceinline__ int edge_count(const RowSplit& s, int v) { return s.head + (v - s.tail0); }
__device__ __forceinline__ int edge_col(const RowSplit& s, int e) {
  return e < s.head ? e : s.tail0 + (e - s.head);
}

// Column a lane fetches when its own column `c` may lie past the row's last vector: such lanes
// re-read the last vector and discard it. The load then needs no branch. A load behind a
// lane-dependent branch makes the compiler wait for every earlier load of the wave before it
// issues the next one (it cannot prove that the register's previous load was consumed), which
// leaves one 16-byte load per wave in flight however far the loop is unrolled.
__device__ __forceinline__ int clamp_col(int c, int nvec) { return c < nvec ? c : nvec - 1; }

// Online-softmax state in the base-2 domain: sum = sum_j exp2(z_j - m).
struct MaxSum {
  float m, s;
};

__device__ __forceinline__ MaxSum merge(const MaxSum& a, const MaxSum& b) {
  MaxSum r;
  r.m = fmaxf(a.m, b.m);
  r.s = a.s * fast_exp2(a.m - r.m) + b.s * fast_exp2(b.m - r.m);
  return r;
}

// Workgroup-wide merge of per-thread (m, s); every thread gets the result. `smem` holds
// 2 * NW floats. Lanes are merged max-first (exact), so the order of the float adds is fixed.
template <int NW>
__device__ __forceinline__ MaxSum block_merge(MaxSum v, float* smem) {
  const float wm = wave_max(v.m);
  const float ws = wave_sum(v.s * fast_exp2(v.m - wm));
  if constexpr (NW == 1) return MaxSum{wm, ws};
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) { smem[wave] = wm; smem[NW + wave] = ws; }
  __syncthreads();
  float M = smem[0];
#pragma unroll
  for (int i = 1; i < NW; ++i) M = fmaxf(M, smem[i]);
  float S = 0.f;
#pragma unroll
  for (int i = 0; i < NW; ++i) S += smem[NW + i] * fast_exp2(smem[i] - M);
  __syncthreads();
  return MaxSum{M, S};
}

template <int NW>
__device__ __forceinline__ float block_sum(float v, float* smem) {
  v = wave_sum(v);
  if constexpr (NW == 1) return v;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) smem[wave] = v;
  __syncthreads();
  float S = smem[0];
#pragma unroll
  for (int i = 1; i < NW; ++i) S += smem[i];
  __syncthreads();
  return S;
}

template <int NW>
__device__ __forceinline__ float block_max(float v, float* smem) {
  v = wave_max(v);
  if constexpr (NW == 1) return v;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) smem[wave] = v;
  __syncthreads();
  float S = smem[0];
#pragma unroll
  for (int i = 1; i < NW; ++i) S = fmaxf(S, smem[i]);
  __syncthreads();
  return S;
}

}  // namespace fm

namespace fm_host {
// Launch shape of the vocabulary kernels: threads per row and 16-byte vectors a thread has
// in flight. `pref_threads` is the per-kernel default (read-only kernels do best with 512
// threads on 64 KB rows, kernels that also write with 1024); both can be overridden for sweeps.
struct VocabShape { int threads, unroll; };
inline VocabShape vocab_shape(int64_t v, int esize, int pref_threads, int pref_unroll,
                              int64_t small_below = 16 * 1024) {
  VocabShape s{pref_threads, pref_unroll};
  const int64_t bytes = v * esize;
  if (bytes < small_below) s.threads = 256;
  else if (bytes < 48 * 1024 && s.threads > 512) s.threads = 512;
  const int t = get_param(P_VOCAB_THREADS);
  if (t == 256 || t == 512 || t == 1024) s.threads = t;
  const int u = get_param(P_VOCAB_UNROLL);
  if (u == 2 || u == 4 || u == 8) s.unroll = u;
  return s;
}
}  // namespace fm_host

// Dispatch a kernel template over (threads, unroll): FM_VOCAB_DISPATCH(shape, LAUNCH) expands
// LAUNCH(TH, UN) for the selected pair.
#define FM_VOCAB_DISPATCH(shape, LAUNCH)                              \
  do {                                                                \
    const int th__ = (shape).threads, un__ = (shape).unroll;          \
    if (th__ == 1024) {                                               \
      if (un__ == 2) { LAUNCH(1024, 2); } else if (un__ == 8) { LAUNCH(1024, 8); } else { LAUNCH(1024, 4); } \
    } else if (th__ == 512) {                                         \
      if (un__ == 2) { LAUNCH(512, 2); } else if (un__ == 8) { LAUNCH(512, 8); } else { LAUNCH(512, 4); }    \
    } else {                                                          \
      if (un__ == 2) { LAUNCH(256, 2); } else if (un__ == 8) { LAUNCH(256, 8); } else { LAUNCH(256, 4); }    \
    }                                                                 \
  } while (0)
