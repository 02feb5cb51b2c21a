// MoE router: softmax + top-k + renormalised weights + per-expert counts + the stable
// (by expert) dispatch permutation, for gfx950.
//
// Reference semantics: forgemind/moe.py:86-91 (softmax -> topk -> renormalise),
// moe.py:52-60 (per-expert histogram), moe.py:232-236 (stable sort of the flat assignments).
// Ties are resolved in the canonical order of forgemind/kernels/topk.py:13-16: equal
// probabilities go to the lowest expert index.
//
// Two launches, integer-only bookkeeping:
//   route_kernel    one wave per row, experts spread over the lanes (lane l owns experts
//                   l, l+64, ...). Wave max / sum give the softmax; each of the k picks is a
//                   wave max over order-preserving integer keys followed by a wave min over
//                   the tied expert indices. A wave keeps four rows in flight so that their
//                   dependent reduction chains overlap. Each 16-wave workgroup owns a
//                   contiguous tile of rows and leaves its expert histogram in `hist[tile][e]`.
//   permute_kernel  every workgroup sums the histograms of the tiles before it (and of all
//                   tiles, for the expert bases), then walks its own tile in ascending flat
//                   position and gives each assignment the slot
//                     base[e] + (#assignments to e in earlier tiles) + (rank inside the tile),
//                   which is exactly the position a stable sort by expert would assign.
#include "fm_common.cuh"

using namespace fm;

namespace {

constexpr int kMaxE = 512;
constexpr int kMaxK = 8;
constexpr int kMaxTiles = 1024;

__device__ __forceinline__ uint32_t key_of(float f) {
  if (f != f) return 0xFFFFFFFFu;
  f = f + 0.0f;
  const uint32_t b = __builtin_bit_cast(uint32_t, f);
  return b ^ ((uint32_t)((int32_t)b >> 31) | 0x80000000u);
}

constexpr int kRouteThreads = 1024;   // 16 waves per tile
constexpr int kRowsAtOnce = 4;        // rows a wave works on together (independent chains)

template <typename T, int EPL>
__global__ __launch_bounds__(kRouteThreads) void route_kernel(const T* __restrict__ logits,
                                                               int32_t* __restrict__ idx,
                                                               float* __restrict__ weights,
                                                               int32_t* __restrict__ hist,
                                                               float* __restrict__ fstat, int64_t n,
                                                               int e, int k, int tile_rows) {
  constexpr int R = kRowsAtOnce;
  constexpr int NW = kRouteThreads / 64;
  __shared__ int lh[kMaxE];
  __shared__ float wstat[NW][EPL * 64];   // per-wave column sums of the probabilities
  __shared__ float wz[NW];                // per-wave sums of logsumexp^2
  float psum[EPL];
  float zsum = 0.f;
#pragma unroll
  for (int q = 0; q < EPL; ++q) psum[q] = 0.f;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int i = tid; i < e; i += kRouteThreads) lh[i] = 0;
  __syncthreads();
  const int64_t row0 = (int64_t)blockIdx.x * tile_rows;
  const int64_t row1 = row0 + tile_rows < n ? row0 + tile_rows : n;
  // wave w owns rows row0 + w, + NW, ...; R of them are in flight at once so that the
  // dependent DPP / readlane chains of different rows overlap
  for (int64_t rb = row0 + wave; rb < row1; rb += (int64_t)NW * R) {
    float p[R][EPL];
    uint32_t key[R][EPL];
    bool live[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int64_t row = rb + (int64_t)r * NW;
      live[r] = row < row1;
#pragma unroll
      for (int q = 0; q < EPL; ++q) {
        const int ex = lane + 64 * q;
        p[r][q] = (live[r] && ex < e) ? Elem<T>::load1(logits + row * (int64_t)e + ex) : -INFINITY;
      }
    }
    float m[R], s[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      m[r] = p[r][0];
#pragma unroll
      for (int q = 1; q < EPL; ++q) m[r] = fmaxf(m[r], p[r][q]);
    }
#pragma unroll
    for (int r = 0; r < R; ++r) m[r] = wave_max(m[r]);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      s[r] = 0.f;
#pragma unroll
      for (int q = 0; q < EPL; ++q) {
        p[r][q] = fast_exp2((p[r][q] - m[r]) * kLog2e);
        s[r] += p[r][q];
      }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) s[r] = wave_sum(s[r]);
#pragma unroll
    for (int r = 0; r < R; ++r) {
#pragma unroll
      for (int q = 0; q < EPL; ++q) {
        p[r][q] = p[r][q] / s[r];
        key[r][q] = (lane + 64 * q) < e ? key_of(p[r][q]) : 0u;   // 0 is below every real key
        if (live[r] && (lane + 64 * q) < e) psum[q] += p[r][q];    // rows in ascending order
      }
      if (live[r]) {
        const float lse = m[r] + fast_log2(s[r]) * kLn2;
        zsum += lse * lse;
      }
    }
    int my_i[R];
    float my_p[R], wsum[R];
#pragma unroll
    for (int r = 0; r < R; ++r) { my_i[r] = 0; my_p[r] = 0.f; wsum[r] = 0.f; }
#pragma unroll
    for (int j = 0; j < kMaxK; ++j) {
      if (j < k) {
        uint32_t bk[R];
        int bq[R], wi[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
          bk[r] = key[r][0];
          bq[r] = 0;
#pragma unroll
          for (int q = 1; q < EPL; ++q) {
            if (key[r][q] > bk[r]) { bk[r] = key[r][q]; bq[r] = q; }
          }
        }
        uint32_t wk[R];
#pragma unroll
        for (int r = 0; r < R; ++r) wk[r] = wave_max_u(bk[r]);
#pragma unroll
        for (int r = 0; r < R; ++r) wi[r] = wave_min_i((bk[r] == wk[r]) ? lane + 64 * bq[r] : 0x7fffffff);
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const int wq = wi[r] >> 6, wl = wi[r] & 63;
          float pv = p[r][0];
#pragma unroll
          for (int q = 1; q < EPL; ++q) pv = (q == wq) ? p[r][q] : pv;
          pv = __shfl(pv, wl, 64);
#pragma unroll
          for (int q = 0; q < EPL; ++q) {
            if (lane == wl && q == wq) key[r][q] = 0u;
          }
          wsum[r] += pv;
          if (lane == j) { my_i[r] = wi[r]; my_p[r] = pv; }
        }
      }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int64_t row = rb + (int64_t)r * NW;
      if (live[r] && lane < k) {
        idx[row * (int64_t)k + lane] = my_i[r];
        weights[row * (int64_t)k + lane] = my_p[r] / wsum[r];
        atomicAdd(&lh[my_i[r]], 1);
      }
    }
  }
  if (fstat != nullptr) {
#pragma unroll
    for (int q = 0; q < EPL; ++q) wstat[wave][lane + 64 * q] = psum[q];
    if (lane == 0) wz[wave] = zsum;
  }
  __syncthreads();
  for (int i = tid; i < e; i += kRouteThreads) hist[(int64_t)blockIdx.x * e + i] = lh[i];
  if (fstat != nullptr) {   // fold the waves in wave order: one fp32 partial row per tile
    float* out = fstat + (int64_t)blockIdx.x * (e + 1);
    for (int i = tid; i < e; i += kRouteThreads) {
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

// Sums the per-tile partial rows [ntiles, e+1] in tile order: stats[0..e) = column sums of the
// probabilities, stats[e] = sum of logsumexp^2. One workgroup; thread c owns column c.
__global__ __launch_bounds__(1024) void route_stats_kernel(const float* __restrict__ fstat,
                                                            float* __restrict__ stats, int e,
                                                            int ntiles) {
  const int c = threadIdx.x;
  if (c > e) return;
  float a = 0.f;
  int t = 0;
  for (; t + 7 < ntiles; t += 8) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = fstat[(int64_t)(t + u) * (e + 1) + c];
#pragma unroll
    for (int u = 0; u < 8; ++u) a += v[u];
  }
  for (; t < ntiles; ++t) a += fstat[(int64_t)t * (e + 1) + c];
  stats[c] = a;
}

typedef int i32x4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void permute_kernel(const int32_t* __restrict__ idx,
                                                       const int32_t* __restrict__ hist,
                                                       int32_t* __restrict__ counts,
                                                       int32_t* __restrict__ slot,
                                                       int32_t* __restrict__ order, int64_t n, int e,
                                                       int k, int tile_rows, int ntiles, int emit) {
  // partial sums of the tile histograms: [group][expert], "before my tile" and "all tiles"
  __shared__ int part_b[4 * kMaxE];   // flat [group][e]; groups * e <= 4 * kMaxE on every path
  __shared__ int part_t[4 * kMaxE];
  __shared__ int total[kMaxE];
  __shared__ int offs[kMaxE];      // next free slot of each expert for this tile
  __shared__ int wcnt[4][kMaxE];   // per-wave assignment counts of the current chunk
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int me = blockIdx.x;

  // the first chunk of this tile's assignments is fetched now, under the histogram loads
  const int64_t p0 = (int64_t)me * tile_rows * k;
  int64_t p1 = p0 + (int64_t)tile_rows * k;
  const int64_t pend = n * (int64_t)k;
  if (p1 > pend) p1 = pend;
  int ex_next = (emit && p0 + tid < p1) ? idx[p0 + tid] : -1;

  const int e4 = e >> 2;
  int groups;
  if ((e & 3) == 0 && e4 <= 256 && (e4 & (e4 - 1)) == 0) {
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
  for (int i = tid; i < 4 * kMaxE; i += 256) (&wcnt[0][0])[i] = 0;
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
        if (me == 0) counts[col] = v;
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
    // rank among equal experts inside the wave, in lane (= flat position) order
    int rank = 0;
    unsigned long long todo = __ballot(act);
    while (todo != 0ull) {
      const int leader = __builtin_ctzll(todo);
      const int e0 = __builtin_amdgcn_readlane(ex, leader);
      const unsigned long long same = __ballot(act && ex == e0);
      if (act && ex == e0) {
        rank = __builtin_popcountll(same & ((1ull << lane) - 1ull));
        if (lane == leader) wcnt[wave][e0] = __builtin_popcountll(same);
      }
      todo &= ~same;
    }
    __syncthreads();
    if (act) {
      int prior = offs[ex];
      for (int w = 0; w < wave; ++w) prior += wcnt[w][ex];
      const int s = prior + rank;
      if (slot != nullptr) slot[p] = s;
      if (order != nullptr) order[s] = (int32_t)p;
    }
    __syncthreads();
    for (int col = tid; col < e; col += 256) {
      offs[col] += (wcnt[0][col] + wcnt[1][col]) + (wcnt[2][col] + wcnt[3][col]);
      wcnt[0][col] = 0; wcnt[1][col] = 0; wcnt[2][col] = 0; wcnt[3][col] = 0;
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
  const dim3 grid((unsigned)tl.ntiles), block(kRouteThreads);
#define GO(EPL) \
  hipLaunchKernelGGL((route_kernel<T, EPL>), grid, block, 0, st, lp, idx, weights, hist, fstat, n, e, k, tl.tile_rows)
  if (e <= 64) GO(1);
  else if (e <= 128) GO(2);
  else if (e <= 256) GO(4);
  else GO(8);
#undef GO
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
  if (stats != nullptr) {
    hipLaunchKernelGGL(route_stats_kernel, dim3(1), dim3(1024), 0, st, fstat, stats, e, tl.ntiles);
    FM_CHECK_LAUNCH("fm_route(stats)");
  }
  const int emit = (slot != nullptr || order != nullptr) && n > 0 ? 1 : 0;
  hipLaunchKernelGGL(permute_kernel, dim3(emit ? (unsigned)tl.ntiles : 1u), dim3(256), 0, st, idx, hist,
                     counts, slot, order, n, e, k, tl.tile_rows, tl.ntiles, emit);
  FM_CHECK_LAUNCH("fm_route(permute)");
  return FM_OK;
}

}  // extern "C"
