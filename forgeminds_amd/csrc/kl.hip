// Forward KL(teacher || student) over vocabulary-wide rows, forward and backward, gfx950.
//
// Reference semantics: forgemind/kernels/_fallback.py:52-69 and forgemind/kernels/kl.py:73-135
// (per row: KL = sum_j p_t (log p_t - log p_s); gradient wrt the student only).
//
// The reference kernel walks each row twice (log-sum-exps, then KL + gradient). Rows of
// 128k logits do not fit LDS, so the forward here is a true single pass: with
//   KL = (sum_j e^{t_j - m_t} (t_j - s_j)) / d_t - lse_t + lse_s
// a thread carries (m_s, d_s, m_t, d_t, A) and rescales d_t and A whenever its teacher
// maximum moves. The backward recomputes both softmaxes from the saved lse values.
// Two more forms: kl_loss_grad_kernel writes the gradient in the forward from one read of rows
// that fit the register file, and kl_fwd_topk_kernel also selects the teacher's top-k.
// All exponentials run in the base-2 domain; the temperature is folded into the scale.
#include "fm_topk.hip.h"

using namespace fm;

namespace {

// widest row (in 16-byte vectors) the fused KL + top-k kernel keeps key prefixes for
constexpr int kFusedMaxVec = 20480;

// widest row (in 16-byte vectors) that the one-pass loss + gradient kernel keeps in registers
constexpr int kOnePassMaxVec = 4096;

struct KLState {
  float ms, ds, mt, dt, a;
};

// Folds UNROLL vectors of student / teacher logits (vector u is column c_first + u * stride,
// live when that is below nvec, or always with ALL) into the running state.
template <typename T, int UNROLL, bool ALL = false>
__device__ __forceinline__ void kl_update(KLState& k, const u32x4 (&rs)[UNROLL],
                                          const u32x4 (&rt)[UNROLL], int c_first, int stride,
                                          int nvec, float c1) {
  constexpr int EPV = Elem<T>::kVec;
  // maxima are taken on the raw logits and scaled once per batch; the temperature scale rides
  // in the fma that feeds exp2, and the (t - s) factor of A is scaled once per batch too
  float zs[UNROLL][EPV], zt[UNROLL][EPV];
  float raw_ms = -INFINITY, raw_mt = -INFINITY;
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    const int c = c_first + u * stride;
    if (ALL || c < nvec) {
      Elem<T>::unpack(rs[u], zs[u]);
      Elem<T>::unpack(rt[u], zt[u]);
#pragma unroll
      for (int e = 0; e < EPV; ++e) {
        raw_ms = fmaxf(raw_ms, zs[u][e]);
        raw_mt = fmaxf(raw_mt, zt[u][e]);
      }
    }
  }
  const float cms = fmaxf(k.ms, raw_ms * c1), cmt = fmaxf(k.mt, raw_mt * c1);   // finite: k.ms, k.mt are
  float ds = k.ds * fast_exp2(k.ms - cms);
  const float ft = fast_exp2(k.mt - cmt);
  float dt = k.dt * ft;
  float a_raw = 0.f;
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    const int c = c_first + u * stride;
    if (ALL || c < nvec) {   // uniform per vector; keeps (-inf) - (-inf) out of the A term
#pragma unroll
      for (int e = 0; e < EPV; ++e) {
        ds += fast_exp2(__builtin_fmaf(zs[u][e], c1, -cms));
        const float et = fast_exp2(__builtin_fmaf(zt[u][e], c1, -cmt));
        dt += et;
        a_raw += et * (zt[u][e] - zs[u][e]);
      }
    }
  }
  k.ms = cms; k.ds = ds; k.mt = cmt; k.dt = dt; k.a = k.a * ft + a_raw * c1;
}

// One scalar column.
__device__ __forceinline__ void kl_update1(KLState& k, float zs, float zt) {
  const float cms = fmaxf(k.ms, zs), cmt = fmaxf(k.mt, zt);
  k.ds = k.ds * fast_exp2(k.ms - cms) + fast_exp2(zs - cms);
  const float ft = fast_exp2(k.mt - cmt);
  const float et = fast_exp2(zt - cmt);
  k.dt = k.dt * ft + et;
  k.a = k.a * ft + et * (zt - zs);
  k.ms = cms; k.mt = cmt;
}

// Workgroup merge: maxima first (exact), then rescaled sums in lane / wave order. Every thread
// returns the row's base-2 log-sum-exps and KL (in bits); smem holds 5 * NW floats.
template <int NW>
__device__ __forceinline__ void kl_merge(const KLState& k, float* smem, float* l2s, float* l2t,
                                         float* kl2) {
  const int tid = threadIdx.x;
  const float wms = wave_max(k.ms), wmt = wave_max(k.mt);
  const float fs = fast_exp2(k.ms - wms), ft = fast_exp2(k.mt - wmt);
  float wds = wave_sum(k.ds * fs), wdt = wave_sum(k.dt * ft), wa = wave_sum(k.a * ft);
  float Ms = wms, Mt = wmt, Ds = wds, Dt = wdt, A = wa;
  if constexpr (NW > 1) {
    const int lane = tid & 63, wave = tid >> 6;
    if (lane == 0) {
      smem[wave] = wms; smem[NW + wave] = wmt; smem[2 * NW + wave] = wds;
      smem[3 * NW + wave] = wdt; smem[4 * NW + wave] = wa;
    }
    __syncthreads();
    Ms = smem[0]; Mt = smem[NW];
#pragma unroll
    for (int i = 1; i < NW; ++i) { Ms = fmaxf(Ms, smem[i]); Mt = fmaxf(Mt, smem[NW + i]); }
    Ds = 0.f; Dt = 0.f; A = 0.f;
#pragma unroll
    for (int i = 0; i < NW; ++i) {
      const float gs = fast_exp2(smem[i] - Ms), gt = fast_exp2(smem[NW + i] - Mt);
      Ds += smem[2 * NW + i] * gs;
      Dt += smem[3 * NW + i] * gt;
      A += smem[4 * NW + i] * gt;
    }
  }
  *l2s = Ms + fast_log2(Ds);
  *l2t = Mt + fast_log2(Dt);
  *kl2 = A / Dt - *l2t + *l2s;
}

// (softmax(s) - softmax(t)) * mul of one 16-byte vector of each, from the row's base-2 log-sum-exps.
template <typename T, typename GT>
__device__ __forceinline__ void kl_grad_vec(const u32x4& rs, const u32x4& rt, GT* dst, float c1, float l2s,
                                            float l2t, float mul) {
  constexpr int EPV = Elem<T>::kVec;
  float zs[EPV], zt[EPV], o[EPV];
  Elem<T>::unpack(rs, zs);
  Elem<T>::unpack(rt, zt);
#pragma unroll
  for (int e = 0; e < EPV; ++e)
    o[e] = (fast_exp2(zs[e] * c1 - l2s) - fast_exp2(zt[e] * c1 - l2t)) * mul;
  if constexpr (sizeof(GT) == sizeof(T)) {
    store16_stream(dst, Elem<GT>::pack(o));
  } else {  // fp32 gradient next to 16-bit logits: two 16-byte stores
    static_assert(sizeof(GT) == 4 && EPV == 8, "gradient is the logits' dtype or fp32");
    float lo[4] = {o[0], o[1], o[2], o[3]}, hi[4] = {o[4], o[5], o[6], o[7]};
    store16_stream(dst, Elem<float>::pack(lo));
    store16_stream(dst + 4, Elem<float>::pack(hi));
  }
}

// One sweep over a row (from vector c_begin on) that writes (softmax(s) - softmax(t)) * mul from the
// row's base-2 log-sum-exps: the body of the backward, shared by the kernels that append it to a
// forward.
template <typename T, typename GT, int THREADS, int UNROLL>
__device__ __forceinline__ void kl_grad_sweep(const T* sp_, const T* tp_, GT* gp, const RowSplit& sp,
                                              int v, float c1, float l2s, float l2t, float mul,
                                              int c_begin = 0) {
  constexpr int EPV = Elem<T>::kVec;
  const int tid = threadIdx.x;
  for (int c0 = c_begin; c0 < sp.nvec; c0 += THREADS * UNROLL) {
    u32x4 rs[UNROLL], rt[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int c = clamp_col(c0 + u * THREADS + tid, sp.nvec);
      rs[u] = load16_stream(sp_ + sp.head + (int64_t)c * EPV);
      rt[u] = load16_stream(tp_ + sp.head + (int64_t)c * EPV);
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int c = c0 + u * THREADS + tid;
      if (c < sp.nvec) {
        float zs[EPV], zt[EPV], o[EPV];
        Elem<T>::unpack(rs[u], zs);
        Elem<T>::unpack(rt[u], zt);
#pragma unroll
        for (int e = 0; e < EPV; ++e)
          o[e] = (fast_exp2(zs[e] * c1 - l2s) - fast_exp2(zt[e] * c1 - l2t)) * mul;
        GT* dst = gp + sp.head + (int64_t)c * EPV;
        if constexpr (sizeof(GT) == sizeof(T)) {
          store16_stream(dst, Elem<GT>::pack(o));
        } else {  // fp32 gradient next to 16-bit logits: two 16-byte stores
          static_assert(sizeof(GT) == 4 && EPV == 8, "gradient is the logits' dtype or fp32");
          float lo[4] = {o[0], o[1], o[2], o[3]}, hi[4] = {o[4], o[5], o[6], o[7]};
          store16_stream(dst, Elem<float>::pack(lo));
          store16_stream(dst + 4, Elem<float>::pack(hi));
        }
      }
    }
  }
  const int ne = edge_count(sp, v);
  for (int e = tid; e < ne; e += THREADS) {
    const int col = edge_col(sp, e);
    const float ps = fast_exp2(Elem<T>::load1(sp_ + col) * c1 - l2s);
    const float pt = fast_exp2(Elem<T>::load1(tp_ + col) * c1 - l2t);
    Elem<GT>::store1(gp + col, (ps - pt) * mul);
  }
}

template <typename T, int THREADS, int UNROLL>
__global__ __launch_bounds__(THREADS) void kl_fwd_kernel(const T* __restrict__ student,
                                                          const T* __restrict__ teacher,
                                                          float* __restrict__ lse_s,
                                                          float* __restrict__ lse_t,
                                                          float* __restrict__ row_kl, int v,
                                                          float inv_temp, bool vec_ok) {
  constexpr int EPV = Elem<T>::kVec;
  constexpr int NW = THREADS / 64;
  __shared__ float smem[5 * NW];
  const int64_t row = blockIdx.x;
  const T* sp_ = student + row * (int64_t)v;
  const T* tp_ = teacher + row * (int64_t)v;
  const RowSplit sp = split_row<EPV>(row, v, vec_ok);
  const int tid = threadIdx.x;
  const float c1 = kLog2e * inv_temp;

  KLState k{kNegBig, 0.f, kNegBig, 0.f, 0.f};
  for (int c0 = 0; c0 < sp.nvec; c0 += THREADS * UNROLL) {
    u32x4 rs[UNROLL], rt[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int c = clamp_col(c0 + u * THREADS + tid, sp.nvec);
      rs[u] = load16_stream(sp_ + sp.head + (int64_t)c * EPV);
      rt[u] = load16_stream(tp_ + sp.head + (int64_t)c * EPV);
    }
    kl_update<T, UNROLL>(k, rs, rt, c0 + tid, THREADS, sp.nvec, c1);
  }
  const int ne = edge_count(sp, v);
  for (int e = tid; e < ne; e += THREADS) {
    const int col = edge_col(sp, e);
    kl_update1(k, Elem<T>::load1(sp_ + col) * c1, Elem<T>::load1(tp_ + col) * c1);
  }

  float l2s, l2t, kl2;
  kl_merge<NW>(k, smem, &l2s, &l2t, &kl2);
  if (tid == 0) {
    lse_s[row] = l2s * kLn2;
    lse_t[row] = l2t * kLn2;
    row_kl[row] = kl2 * kLn2;
  }
}

// The same forward, also returning the exact top-k of the teacher row (raw logits; softmax and
// the temperature are monotone, so the order is that of the probabilities). The streaming pass
// leaves a 16-bit key prefix of every teacher vector's maximum in LDS (2 bytes per 16 bytes of
// row), so the selection revisits only the few vectors that can hold a winner.
template <typename T, int THREADS, int UNROLL, bool GRAD>
__global__ __launch_bounds__(THREADS) void kl_fwd_topk_kernel(
    const T* __restrict__ student, const T* __restrict__ teacher, float* __restrict__ lse_s,
    float* __restrict__ lse_t, float* __restrict__ row_kl, T* __restrict__ tk_values,
    int32_t* __restrict__ tk_idx32, int64_t* __restrict__ tk_idx64, float* __restrict__ tk_probs,
    T* __restrict__ dstudent, float mul, int v, int k, float inv_temp, bool vec_ok) {
  constexpr int EPV = Elem<T>::kVec;
  constexpr int NW = THREADS / 64;
  __shared__ float smem[5 * NW];
  __shared__ TopkShared<THREADS, kVecMaxLds> sh;
  extern __shared__ __align__(16) uint16_t vhi[];
  const int64_t row = blockIdx.x;
  const T* sp_ = student + row * (int64_t)v;
  const T* tp_ = teacher + row * (int64_t)v;
  const RowSplit sp = split_row<EPV>(row, v, vec_ok);
  const int tid = threadIdx.x;
  const float c1 = kLog2e * inv_temp;

  KLState st{kNegBig, 0.f, kNegBig, 0.f, 0.f};
  float fm = -INFINITY;
  bool has_nan = false;
  // (with the gradient sweep behind it the float form schedules better: 780 against 795 us at
  // 4096 x 128256, so only the forward-only kernel takes the packed keys)
  constexpr bool SK = SKey<T>::ok && !GRAD;
  uint32_t sm = 0u;   // largest 16-bit stream key of this thread's vectors (0 is -inf)
  {  // zero the padding of the last quad of prefixes
    const int p = ((sp.nvec + 3) & ~3) - 1 - tid;
    if (tid < 3 && p >= sp.nvec) vhi[p] = 0;
  }
  __syncthreads();
  for (int c0 = 0; c0 < sp.nvec; c0 += THREADS * UNROLL) {
    u32x4 rs[UNROLL], rt[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int c = clamp_col(c0 + u * THREADS + tid, sp.nvec);
      if constexpr (GRAD) {   // a gradient sweep follows: leave the row to the caches
        rs[u] = load16(sp_ + sp.head + (int64_t)c * EPV);
        rt[u] = load16(tp_ + sp.head + (int64_t)c * EPV);
      } else {
        rs[u] = load16_stream(sp_ + sp.head + (int64_t)c * EPV);
        rt[u] = load16_stream(tp_ + sp.head + (int64_t)c * EPV);
      }
    }
    kl_update<T, UNROLL>(st, rs, rt, c0 + tid, THREADS, sp.nvec, c1);
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int c = c0 + u * THREADS + tid;
      if (c < sp.nvec) {
        if constexpr (SK) {   // half types: 16-bit keys straight from the packed words
          const uint32_t m = skey_vector_max<T>(rt[u]);
          vhi[c] = (uint16_t)m;
          sm = m > sm ? m : sm;
        } else {
          const float m = fold_vector_max<T>(rt[u]);
          const bool bad = m != m;
          vhi[c] = (uint16_t)(bad ? 0xFFFFu : key_prefix(key_of(m)));
          fm = fmaxf(fm, m);
          has_nan |= bad;
        }
      }
    }
  }
  if constexpr (SK) {
    if (sm > SKeyC<T>::kNanAbove) has_nan = true;
    else fm = float_of_skey<T>(sm);
  }
  const int ne = edge_count(sp, v);
  for (int e = tid; e < ne; e += THREADS) {
    const int col = edge_col(sp, e);
    const float t = Elem<T>::load1(tp_ + col);
    kl_update1(st, Elem<T>::load1(sp_ + col) * c1, t * c1);
    fm = fmaxf(fm, t);
    has_nan |= (t != t);
  }
  float l2s, l2t, kl2;
  kl_merge<NW>(st, smem, &l2s, &l2t, &kl2);
  if (tid == 0) {
    lse_s[row] = l2s * kLn2;
    lse_t[row] = l2t * kLn2;
    row_kl[row] = kl2 * kLn2;
  }
  const float none[1] = {0.f};
  topk_finish<T, THREADS, 1, kVecMaxLds, kTopkNormal, SK ? kVhiStream16 : kVhiPrefix>(tp_, sp, v, k, none, vhi, fm, has_nan, sh, row,
                                                          tk_values, tk_idx32, tk_idx64, tk_probs, c1, l2t);
  if constexpr (GRAD)
    kl_grad_sweep<T, T, THREADS, UNROLL>(sp_, tp_, dstudent + row * (int64_t)v, sp, v, c1, l2s, l2t, mul);
}

// loss = sum(row_kl) * scale in a fixed order (thread i adds rows i, i+1024, ...).
__global__ __launch_bounds__(1024) void kl_finalize_kernel(const float* __restrict__ row_kl,
                                                           int64_t n, float scale,
                                                           float* __restrict__ loss) {
  __shared__ float sf[16];
  float a = 0.f;
  int64_t i = threadIdx.x;
  for (; i + 7 * 1024 < n; i += 8 * 1024) {   // eight loads in flight; additions in the same order
    float r[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) r[u] = row_kl[i + u * 1024];
#pragma unroll
    for (int u = 0; u < 8; ++u) a += r[u];
  }
  for (; i < n; i += 1024) a += row_kl[i];
  a = wave_sum(a);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) sf[wave] = a;
  __syncthreads();
  if (threadIdx.x == 0) {
    float t = sf[0];
    for (int i = 1; i < 16; ++i) t += sf[i];
    *loss = t * scale;
  }
}

template <typename T, typename GT, int THREADS, int UNROLL>
__global__ __launch_bounds__(THREADS) void kl_bwd_kernel(const T* __restrict__ student,
                                                          const T* __restrict__ teacher,
                                                          const float* __restrict__ lse_s,
                                                          const float* __restrict__ lse_t,
                                                          const float* __restrict__ grad_out,
                                                          int grad_per_row, GT* __restrict__ dstudent,
                                                          int v, float inv_temp, float scale,
                                                          bool vec_ok, int chunks) {
  constexpr int EPV = Elem<T>::kVec;
  // chunks > 1: a workgroup takes one tile of THREADS * UNROLL vectors of a row, not the whole row
  const int64_t row = chunks > 1 ? (int64_t)(blockIdx.x / (unsigned)chunks) : (int64_t)blockIdx.x;
  const int chunk = chunks > 1 ? (int)(blockIdx.x % (unsigned)chunks) : 0;
  const T* sp_ = student + row * (int64_t)v;
  const T* tp_ = teacher + row * (int64_t)v;
  GT* gp = dstudent + row * (int64_t)v;
  const RowSplit sp = split_row<EPV>(row, v, vec_ok);
  const int tid = threadIdx.x;
  const float c1 = kLog2e * inv_temp;
  const float l2s = lse_s[row] * kLog2e, l2t = lse_t[row] * kLog2e;
  float g = 1.f;
  if (grad_out != nullptr) g = grad_per_row ? grad_out[row] : grad_out[0];
  const float mul = inv_temp * scale * g;
  const int c_begin = chunks > 1 ? chunk * THREADS * UNROLL : 0;
  const int c_end = chunks > 1 ? (c_begin + THREADS * UNROLL < sp.nvec ? c_begin + THREADS * UNROLL : sp.nvec) : sp.nvec;

  for (int c0 = c_begin; c0 < c_end; c0 += THREADS * UNROLL) {
    u32x4 rs[UNROLL], rt[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int c = clamp_col(c0 + u * THREADS + tid, sp.nvec);
      rs[u] = load16_stream(sp_ + sp.head + (int64_t)c * EPV);
      rt[u] = load16_stream(tp_ + sp.head + (int64_t)c * EPV);
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int c = c0 + u * THREADS + tid;
      touch(rs[u]);
      touch(rt[u]);
      if (c < sp.nvec) {
        float zs[EPV], zt[EPV], o[EPV];
        Elem<T>::unpack(rs[u], zs);
        Elem<T>::unpack(rt[u], zt);
#pragma unroll
        for (int e = 0; e < EPV; ++e)
          o[e] = (fast_exp2(zs[e] * c1 - l2s) - fast_exp2(zt[e] * c1 - l2t)) * mul;
        GT* dst = gp + sp.head + (int64_t)c * EPV;
        if constexpr (sizeof(GT) == sizeof(T)) {
          store16_stream(dst, Elem<GT>::pack(o));
        } else {  // fp32 gradient next to 16-bit logits: two 16-byte stores
          static_assert(sizeof(GT) == 4 && EPV == 8, "gradient is the logits' dtype or fp32");
          float lo[4] = {o[0], o[1], o[2], o[3]}, hi[4] = {o[4], o[5], o[6], o[7]};
          store16_stream(dst, Elem<float>::pack(lo));
          store16_stream(dst + 4, Elem<float>::pack(hi));
        }
      }
    }
  }
  if (chunk != 0) return;
  const int ne = edge_count(sp, v);
  for (int e = tid; e < ne; e += THREADS) {
    const int col = edge_col(sp, e);
    const float ps = fast_exp2(Elem<T>::load1(sp_ + col) * c1 - l2s);
    const float pt = fast_exp2(Elem<T>::load1(tp_ + col) * c1 - l2t);
    Elem<GT>::store1(gp + col, (ps - pt) * mul);
  }
}

// KL and its gradient from ONE read of both rows: student and teacher stay in registers
// (ITERS 16-byte vectors each per thread) between the log-sum-exps and the gradient store,
// the dataflow of the reference's kernel (kl.py:73-135) without its second read. The gradient
// is for an upstream gradient of 1: (p_s - p_t) * mul, mul = inv_temp * (1/n for the mean).
// dstudent may be the student buffer itself when both have the same dtype: every element
// is read by the thread that later writes it.
template <typename T, typename GT, int THREADS, int ITERS>
__global__ __launch_bounds__(THREADS) void kl_loss_grad_kernel(const T* student,
                                                                const T* __restrict__ teacher,
                                                                float* __restrict__ lse_s,
                                                                float* __restrict__ lse_t,
                                                                float* __restrict__ row_kl,
                                                                GT* dstudent, int v, float inv_temp,
                                                                float mul) {
  constexpr int EPV = Elem<T>::kVec;
  constexpr int NW = THREADS / 64;
  __shared__ float smem[5 * NW];
  const int64_t row = blockIdx.x;
  const T* sp_ = student + row * (int64_t)v;
  const T* tp_ = teacher + row * (int64_t)v;
  GT* gp = dstudent + row * (int64_t)v;
  const RowSplit sp = split_row<EPV>(row, v, true);
  const int tid = threadIdx.x;
  const int ne = edge_count(sp, v);
  const float c1 = kLog2e * inv_temp;

  u32x4 rs[ITERS], rt[ITERS];
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
    const int c = i * THREADS + tid;
    if (c < sp.nvec) {
      rs[i] = load16_stream(sp_ + sp.head + (int64_t)c * EPV);
      rt[i] = load16_stream(tp_ + sp.head + (int64_t)c * EPV);
    }
  }
  // the unaligned ends of the row (at most EPV - 1 elements each): thread e keeps edge e
  int edge_at = -1;
  float es = -INFINITY, et = -INFINITY;
  if (tid < ne) {
    edge_at = edge_col(sp, tid);
    es = Elem<T>::load1(sp_ + edge_at) * c1;
    et = Elem<T>::load1(tp_ + edge_at) * c1;
  }
  KLState k{fmaxf(es, kNegBig), 0.f, fmaxf(et, kNegBig), 0.f, 0.f};
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
    const int c = i * THREADS + tid;
    if (c < sp.nvec) {
      float zs[EPV], zt[EPV];
      Elem<T>::unpack(rs[i], zs);
      Elem<T>::unpack(rt[i], zt);
#pragma unroll
      for (int e = 0; e < EPV; ++e) {
        k.ms = fmaxf(k.ms, zs[e] * c1);
        k.mt = fmaxf(k.mt, zt[e] * c1);
      }
    }
  }
  if (edge_at >= 0) {
    const float w = fast_exp2(et - k.mt);
    k.ds = fast_exp2(es - k.ms);
    k.dt = w;
    k.a = w * (et - es);
  }
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
    const int c = i * THREADS + tid;
    if (c < sp.nvec) {
      float zs[EPV], zt[EPV];
      Elem<T>::unpack(rs[i], zs);
      Elem<T>::unpack(rt[i], zt);
#pragma unroll
      for (int e = 0; e < EPV; ++e) {
        const float a = zs[e] * c1, b = zt[e] * c1;
        k.ds += fast_exp2(a - k.ms);
        const float w = fast_exp2(b - k.mt);
        k.dt += w;
        k.a += w * (b - a);
      }
    }
  }
  float l2s, l2t, kl2;
  kl_merge<NW>(k, smem, &l2s, &l2t, &kl2);
  if (tid == 0) {
    if (lse_s != nullptr) lse_s[row] = l2s * kLn2;
    if (lse_t != nullptr) lse_t[row] = l2t * kLn2;
    row_kl[row] = kl2 * kLn2;
  }
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
    const int c = i * THREADS + tid;
    if (c < sp.nvec) {
      float zs[EPV], zt[EPV], o[EPV];
      Elem<T>::unpack(rs[i], zs);
      Elem<T>::unpack(rt[i], zt);
#pragma unroll
      for (int e = 0; e < EPV; ++e)
        o[e] = (fast_exp2(zs[e] * c1 - l2s) - fast_exp2(zt[e] * c1 - l2t)) * mul;
      GT* dst = gp + sp.head + (int64_t)c * EPV;
      if constexpr (sizeof(GT) == sizeof(T)) {
        store16_stream(dst, Elem<GT>::pack(o));
      } else {  // fp32 gradient next to 16-bit logits: two 16-byte stores
        static_assert(sizeof(GT) == 4 && EPV == 8, "gradient is the logits' dtype or fp32");
        float lo[4] = {o[0], o[1], o[2], o[3]}, hi[4] = {o[4], o[5], o[6], o[7]};
        store16_stream(dst, Elem<float>::pack(lo));
        store16_stream(dst + 4, Elem<float>::pack(hi));
      }
    }
  }
  if (edge_at >= 0) Elem<GT>::store1(gp + edge_at, (fast_exp2(es - l2s) - fast_exp2(et - l2t)) * mul);
}

template <typename T>
void launch_fwd(const void* s, const void* t, float* lse_s, float* lse_t, float* row_kl, int64_t n,
                int v, float inv_temp, bool vec_ok, hipStream_t st) {
  const T* sp = static_cast<const T*>(s);
  const T* tp = static_cast<const T*>(t);
  const fm_host::VocabShape sh = fm_host::vocab_shape(v, sizeof(T), 512, 4);
  const dim3 grid((unsigned)n);
#define LAUNCH(TH, UN)                                                                            \
  FM_LAUNCH((kl_fwd_kernel<T, TH, UN>), grid, dim3(TH), 0, st, sp, tp, lse_s, lse_t, row_kl, \
                     v, inv_temp, vec_ok)
  FM_VOCAB_DISPATCH(sh, LAUNCH);
#undef LAUNCH
}

template <typename T, typename GT>
void launch_bwd(const void* s, const void* t, const float* lse_s, const float* lse_t,
                const float* grad_out, int grad_per_row, void* ds, int64_t n, int v, float inv_temp,
                float scale, bool vec_ok, hipStream_t st) {
  const T* sp = static_cast<const T*>(s);
  const T* tp = static_cast<const T*>(t);
  GT* gp = static_cast<GT*>(ds);
  const fm_host::VocabShape sh = fm_host::vocab_shape(v, sizeof(T), 1024, 8);
  // The backward needs nothing from the rest of its row but the two saved log-sum-exps, so a row
  // longer than one tile (threads x unroll vectors) is cut into tiles with a workgroup each: no
  // workgroup waits on its own stores before its next loads, and the last, shorter tile of a row
  // is another workgroup's work (4096 x 128256 bf16: 556 -> 524 us).
  const int64_t tile = (int64_t)sh.threads * sh.unroll;
  int64_t chunks = (v / Elem<T>::kVec + 1 + tile - 1) / tile;
  if (chunks < 1 || n * chunks > 0x7fffffffLL) chunks = 1;
  const dim3 grid((unsigned)(n * chunks));
#define LAUNCH(TH, UN)                                                                           \
  FM_LAUNCH((kl_bwd_kernel<T, GT, TH, UN>), grid, dim3(TH), 0, st, sp, tp, lse_s, lse_t, \
                     grad_out, grad_per_row, gp, v, inv_temp, scale, vec_ok, (int)chunks)
  FM_VOCAB_DISPATCH(sh, LAUNCH);
#undef LAUNCH
}

// Rows too wide for registers, loss and gradient in ONE launch: the streaming forward, the
// workgroup merge, then a second sweep over the same row that writes the gradient. The second
// sweep follows the first at once, so a cache that still holds the row serves it (the first
// sweep uses ordinary loads for that reason; the rows in flight, one or two per compute unit,
// are no larger than the memory-side cache). Measured 15-20 % faster than two launches. The
// gradient is for an upstream gradient of 1 and may overwrite the student (each element is
// re-read by the thread that writes it).
template <typename T, typename GT, int THREADS, int UNROLL>
__global__ __launch_bounds__(THREADS) void kl_loss_grad_wide_kernel(const T* student,
                                                                     const T* __restrict__ teacher,
                                                                     float* __restrict__ lse_s,
                                                                     float* __restrict__ lse_t,
                                                                     float* __restrict__ row_kl,
                                                                     GT* dstudent, int v, float inv_temp,
                                                                     float mul, bool vec_ok) {
  constexpr int EPV = Elem<T>::kVec;
  constexpr int NW = THREADS / 64;
  __shared__ float smem[5 * NW];
  const int64_t row = blockIdx.x;
  const T* sp_ = student + row * (int64_t)v;
  const T* tp_ = teacher + row * (int64_t)v;
  GT* gp = dstudent + row * (int64_t)v;
  const RowSplit sp = split_row<EPV>(row, v, vec_ok);
  const int tid = threadIdx.x;
  const int ne = edge_count(sp, v);
  const float c1 = kLog2e * inv_temp;

  KLState k{kNegBig, 0.f, kNegBig, 0.f, 0.f};
  for (int c0 = 0; c0 < sp.nvec; c0 += THREADS * UNROLL) {
    u32x4 rs[UNROLL], rt[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int c = clamp_col(c0 + u * THREADS + tid, sp.nvec);
      rs[u] = load16(sp_ + sp.head + (int64_t)c * EPV);
      rt[u] = load16(tp_ + sp.head + (int64_t)c * EPV);
    }
    kl_update<T, UNROLL>(k, rs, rt, c0 + tid, THREADS, sp.nvec, c1);
  }
  for (int e = tid; e < ne; e += THREADS) {
    const int col = edge_col(sp, e);
    kl_update1(k, Elem<T>::load1(sp_ + col) * c1, Elem<T>::load1(tp_ + col) * c1);
  }
  float l2s, l2t, kl2;
  kl_merge<NW>(k, smem, &l2s, &l2t, &kl2);
  if (tid == 0) {
    if (lse_s != nullptr) lse_s[row] = l2s * kLn2;
    if (lse_t != nullptr) lse_t[row] = l2t * kLn2;
    row_kl[row] = kl2 * kLn2;
  }
  kl_grad_sweep<T, GT, THREADS, UNROLL>(sp_, tp_, gp, sp, v, c1, l2s, l2t, mul);
}

// The same for rows that fit the CHIP: one 512-thread workgroup per compute unit has 256 registers a
// thread and 144 KB of LDS to itself, which hold 22 + 9 vectors of each row per thread, 15872 vector
// pairs (a 126976-column bf16 pair of rows, 496 KB) in all. The row is then read from memory once:
// 6 bytes per logit pair cross the L2 boundary instead of the 10 of the two sweeps above (which run
// at the bandwidth of that boundary). Vectors past those, if any, are streamed and re-read
// as above. Every thread fetches only its own LDS slots: no barrier between the passes.
//
// The grid is persistent (a workgroup per compute unit walks rows blockIdx.x, + gridDim.x, ...), and
// the one workgroup a compute unit holds would otherwise load, then compute, then store in turn,
// so the NEXT row's loads are issued from inside the gradient pass: as soon as a held vector pair has
// given its gradient, its registers (or its LDS slots, filled straight from memory without a register
// in between) take the same columns of the next row, and the loads run under the
// exponentials of the rest of the pass. (A spilled register in that pass undoes this: its reload is
// a vector-memory operation too, and waiting for it means waiting for every load issued before it.)
constexpr int kHeldThreads = 512;
constexpr int kHeldRegs = 22;    // vector pairs a thread keeps in registers
constexpr int kHeldLds = 9;      // and in LDS
template <typename T, typename GT, int THREADS = kHeldThreads, int RI = kHeldRegs, int LI = kHeldLds>
__global__ __launch_bounds__(THREADS) void kl_loss_grad_held_kernel(const T* student,
                                                                          const T* __restrict__ teacher,
                                                                          float* __restrict__ lse_s,
                                                                          float* __restrict__ lse_t,
                                                                          float* __restrict__ row_kl,
                                                                          GT* dstudent, int64_t n, int v,
                                                                          float inv_temp, float mul,
                                                                          bool vec_ok) {
  constexpr int EPV = Elem<T>::kVec;
  constexpr int NW = THREADS / 64;
  extern __shared__ u32x4 parked[];          // [LI][2][THREADS]
  __shared__ float smem[2][5 * NW];          // by row parity: a wave may reach the next row's merge
                                             // while another still reads this row's
  const int tid = threadIdx.x;
  const int wave_first = __builtin_amdgcn_readfirstlane(tid & ~63);   // (a scalar, and known to be one)
  const uint32_t lane_el = (uint32_t)tid * EPV;   // this thread's first element inside a slot
  const float c1 = kLog2e * inv_temp;
  // slot i of a row: THREADS vectors from vector i * THREADS on, one per thread. The row's base is
  // the same for the whole workgroup; a thread adds its own 32-bit offset.
  auto slot = [&](auto* row_base, int i) { return row_base + (int64_t)i * (THREADS * EPV) + lane_el; };
  auto park = [&](int j, int which) { return parked + (j * 2 + which) * THREADS; };

  u32x4 hs[RI], ht[RI];
  int64_t row = blockIdx.x;
  if (row >= n) return;
  // A slot is held only when every thread has a column in it (`full` of them, the same for the
  // whole workgroup); the ragged end of the row is streamed with the remainder.
  auto full_slots = [](const RowSplit& sp) {
    const int f = sp.nvec / THREADS;
    return f < RI + LI ? f : RI + LI;
  };
  {
    const RowSplit sp = split_row<EPV>(row, v, vec_ok);
    const T* sb = student + row * (int64_t)v + sp.head;
    const T* tb = teacher + row * (int64_t)v + sp.head;
    const int full = full_slots(sp);
#pragma unroll
    for (int i = 0; i < RI; ++i) {
      if (i < full) {
        hs[i] = load16_stream(slot(sb, i));
        ht[i] = load16_stream(slot(tb, i));
      }
    }
#pragma unroll
    for (int j = 0; j < LI; ++j) {
      if (RI + j < full) {
        load16_stream_to_lds(slot(sb, RI + j), park(j, 0) + wave_first);
        load16_stream_to_lds(slot(tb, RI + j), park(j, 1) + wave_first);
      }
    }
  }
  for (int flip = 0; row < n; row += gridDim.x, flip ^= 1) {
    const T* sp_ = student + row * (int64_t)v;
    const T* tp_ = teacher + row * (int64_t)v;
    GT* gp = dstudent + row * (int64_t)v;
    const RowSplit sp = split_row<EPV>(row, v, vec_ok);
    const int ne = edge_count(sp, v);
    const int full = full_slots(sp);

    // (one vector pair at a time: two at a time need 16 more registers, and then one held pair
    // is spilled)
    KLState k{kNegBig, 0.f, kNegBig, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < RI; ++i) {
      if (i < full) {
        const u32x4 rs[1] = {hs[i]}, rt[1] = {ht[i]};
        kl_update<T, 1, true>(k, rs, rt, 0, 0, 0, c1);
      }
    }
    wait_vmem_all();   // the LDS slots were filled by loads that name no register
#pragma unroll
    for (int j = 0; j < LI; ++j) {
      if (RI + j < full) {
        const u32x4 rs[1] = {park(j, 0)[tid]}, rt[1] = {park(j, 1)[tid]};
        kl_update<T, 1, true>(k, rs, rt, 0, 0, 0, c1);
      }
    }
    const int held = full * THREADS;
    for (int c0 = held; c0 < sp.nvec; c0 += THREADS * 2) {
      u32x4 rs[2], rt[2];
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int c = clamp_col(c0 + u * THREADS + tid, sp.nvec);
        rs[u] = load16(sp_ + sp.head + (int64_t)c * EPV);
        rt[u] = load16(tp_ + sp.head + (int64_t)c * EPV);
      }
      kl_update<T, 2>(k, rs, rt, c0 + tid, THREADS, sp.nvec, c1);
    }
    for (int e = tid; e < ne; e += THREADS) {
      const int col = edge_col(sp, e);
      kl_update1(k, Elem<T>::load1(sp_ + col) * c1, Elem<T>::load1(tp_ + col) * c1);
    }
    float l2s, l2t, kl2;
    kl_merge<NW>(k, smem[flip], &l2s, &l2t, &kl2);
    if (tid == 0) {
      if (lse_s != nullptr) lse_s[row] = l2s * kLn2;
      if (lse_t != nullptr) lse_t[row] = l2t * kLn2;
      row_kl[row] = kl2 * kLn2;
    }

    // the gradient of every held pair, and in its place the same columns of the next row
    const int64_t next = row + gridDim.x;
    const bool more = next < n;   // the same for the whole workgroup
    const RowSplit nsp = split_row<EPV>(more ? next : row, v, vec_ok);
    const int nfull = more ? full_slots(nsp) : 0;
    const T* nsb = student + (more ? next : row) * (int64_t)v + nsp.head;
    const T* ntb = teacher + (more ? next : row) * (int64_t)v + nsp.head;
    GT* gb = gp + sp.head;
#pragma unroll
    for (int i = 0; i < RI; ++i) {
      if (i < full) {
        // (behind an empty asm, so that the compiler unpacks the vector again here instead of
        // keeping the floats of the first pass alive for all the pairs)
        touch(hs[i]);
        touch(ht[i]);
        kl_grad_vec<T, GT>(hs[i], ht[i], slot(gb, i), c1, l2s, l2t, mul);
      }
      if (i < nfull) {
        hs[i] = load16_stream(slot(nsb, i));
        ht[i] = load16_stream(slot(ntb, i));
      }
    }
#pragma unroll
    for (int j = 0; j < LI; ++j) {
      u32x4 rs, rt;
      if (RI + j < full) {
        rs = park(j, 0)[tid];
        rt = park(j, 1)[tid];
        touch(rs);   // in registers before the slots are given away
        touch(rt);
      }
      if (RI + j < nfull) {
        load16_stream_to_lds(slot(nsb, RI + j), park(j, 0) + wave_first);
        load16_stream_to_lds(slot(ntb, RI + j), park(j, 1) + wave_first);
      }
      if (RI + j < full) kl_grad_vec<T, GT>(rs, rt, slot(gb, RI + j), c1, l2s, l2t, mul);
    }
    // what was not held, and the row's unaligned edges
    kl_grad_sweep<T, GT, THREADS, 2>(sp_, tp_, gp, sp, v, c1, l2s, l2t, mul, held);
  }
}

// One launch shape of the kernel above; false when the device does not grant the LDS it needs.
template <typename T, typename GT, int TH, int RI, int LI>
bool launch_held_shape(const T* student, const T* teacher, float* lse_s, float* lse_t, float* row_kl,
                       GT* dstudent, int64_t n, int v, float inv_temp, float mul, bool vec_ok,
                       hipStream_t st) {
  constexpr int lds = LI * 2 * TH * 16;
  if (lds > 65536 && !fm_host::grant_dynamic_lds<&kl_loss_grad_held_kernel<T, GT, TH, RI, LI>>(lds)) return false;
  const int64_t fit = (int64_t)fm_host::num_cus() *
                      fm_host::resident_per_cu<&kl_loss_grad_held_kernel<T, GT, TH, RI, LI>>(TH, lds);
  FM_LAUNCH((kl_loss_grad_held_kernel<T, GT, TH, RI, LI>), dim3((unsigned)(n < fit ? n : fit)), dim3(TH),
            (size_t)lds, st, student, teacher, lse_s, lse_t, row_kl, dstudent, n, v, inv_temp, mul, vec_ok);
  return true;
}

// The shape by row width. 16-bit rows are bound by arithmetic, and a compute unit that holds
// SEVERAL workgroups, each on a row of its own, keeps its vector ALUs busy while one of them waits
// for memory or at its barrier: three 256-thread workgroups (13 + 3 slots, which hold 4096 vectors:
// at most 168 registers and 24 KB of LDS each) for rows of up to 4608 vectors, two (22 + 9 slots,
// 7936 vectors) up to 8192, one 512-thread workgroup beyond; what a row has past the slots is
// streamed. us for bf16 rows, three / two / one workgroup a unit: [8192,20000] 204 / 226 /
// 264, [16384,24576] 446 / 463 / 504, [16384,32000] 598 / 638 / 769, [8192,50304] 510 / 494 / 511,
// [4096,65536] 344 / 325 / 325. fp32 rows are bound by bytes and run the same in every shape
// ([8192,32000]: 588 / 576 / 568), so they take the one.
template <typename T, typename GT>
bool launch_held(const T* student, const T* teacher, float* lse_s, float* lse_t, float* row_kl,
                 GT* dstudent, int64_t n, int v, int64_t nvec, float inv_temp, float mul, bool vec_ok,
                 hipStream_t st) {
  if constexpr (sizeof(T) == 2) {
    if (nvec <= 4608)
      return launch_held_shape<T, GT, 256, 13, 3>(student, teacher, lse_s, lse_t, row_kl, dstudent, n, v,
                                                  inv_temp, mul, vec_ok, st);
    if (nvec <= 8192 &&
        launch_held_shape<T, GT, 256, 22, 9>(student, teacher, lse_s, lse_t, row_kl, dstudent, n, v, inv_temp,
                                             mul, vec_ok, st))
      return true;
  }
  return launch_held_shape<T, GT, kHeldThreads, kHeldRegs, kHeldLds>(student, teacher, lse_s, lse_t, row_kl,
                                                                     dstudent, n, v, inv_temp, mul, vec_ok, st);
}

// Narrow rows (at most 1024 classes: classifier distillation, not vocabularies): TPR lanes per
// row, several rows per 256-thread workgroup, both rows in registers (ITERS scalar loads each
// per lane), any alignment. LOSS writes the log-sum-exps and the row's KL; GRAD writes the
// gradient, from the sums just computed (LOSS) or from saved log-sum-exps. dstudent may be
// the student buffer when the dtypes agree: each element is read by the lane that writes it.
template <typename T, typename GT, int TPR, int ITERS, bool LOSS, bool GRAD>
__global__ __launch_bounds__(256) void kl_rows_kernel(const T* student, const T* __restrict__ teacher,
                                                      float* lse_s, float* lse_t,
                                                      float* __restrict__ row_kl,
                                                      const float* __restrict__ grad_out,
                                                      int grad_per_row, GT* dstudent, int64_t n, int v,
                                                      float inv_temp, float mul) {
  constexpr int RPB = 256 / TPR;
  const int tid = threadIdx.x;
  const int rib = tid / TPR;
  const int t = tid % TPR;
  const int64_t row = (int64_t)blockIdx.x * RPB + rib;
  const bool valid = row < n;
  const int64_t base = row * (int64_t)v;
  const float c1 = kLog2e * inv_temp;
  float zs[ITERS], zt[ITERS];
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
    const int c = i * TPR + t;
    const bool in = valid && c < v;
    zs[i] = in ? Elem<T>::load1(student + base + c) * c1 : -INFINITY;
    zt[i] = in ? Elem<T>::load1(teacher + base + c) * c1 : -INFINITY;
  }
  float l2s, l2t;
  if constexpr (LOSS) {
    float ms = kNegBig, mt = kNegBig;
#pragma unroll
    for (int i = 0; i < ITERS; ++i) { ms = fmaxf(ms, zs[i]); mt = fmaxf(mt, zt[i]); }
    ms = group_reduce<TPR, OpMax>(ms);
    mt = group_reduce<TPR, OpMax>(mt);
    float ds = 0.f, dt = 0.f, a = 0.f;
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      const int c = i * TPR + t;
      if (valid && c < v) {            // keeps (-inf) - (-inf) of the padding out of the A term
        ds += fast_exp2(zs[i] - ms);
        const float et = fast_exp2(zt[i] - mt);
        dt += et;
        a += et * (zt[i] - zs[i]);
      }
    }
    ds = group_reduce<TPR, OpSum>(ds);
    dt = group_reduce<TPR, OpSum>(dt);
    a = group_reduce<TPR, OpSum>(a);
    l2s = ms + fast_log2(ds);
    l2t = mt + fast_log2(dt);
    if (valid && t == 0) {
      if (lse_s != nullptr) lse_s[row] = l2s * kLn2;
      if (lse_t != nullptr) lse_t[row] = l2t * kLn2;
      row_kl[row] = (a / dt - l2t + l2s) * kLn2;
    }
  } else {
    l2s = valid ? lse_s[row] * kLog2e : 0.f;
    l2t = valid ? lse_t[row] * kLog2e : 0.f;
  }
  if constexpr (GRAD) {
    float g = mul;
    if (grad_out != nullptr && valid) g *= grad_per_row ? grad_out[row] : grad_out[0];
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      const int c = i * TPR + t;
      if (valid && c < v)
        Elem<GT>::store1(dstudent + base + c, (fast_exp2(zs[i] - l2s) - fast_exp2(zt[i] - l2t)) * g);
    }
  }
}

// The same lane groups with 16-byte accesses, for rows that are a whole number of aligned
// vectors: lane t of a row's TPR lanes keeps vectors t, t + TPR, ... of both rows packed and
// unpacks them once per pass. The gradient may overwrite the student (a lane stores only what it
// loaded).
template <typename T, typename GT, int TPR, int ITERS, bool LOSS, bool GRAD>
__global__ __launch_bounds__(256) void kl_vrows_kernel(const T* student, const T* __restrict__ teacher,
                                                       float* lse_s, float* lse_t,
                                                       float* __restrict__ row_kl,
                                                       const float* __restrict__ grad_out,
                                                       int grad_per_row, GT* dstudent, int64_t n, int v,
                                                       float inv_temp, float mul) {
  constexpr int EPV = Elem<T>::kVec;
  constexpr int RPB = 256 / TPR;
  const int tid = threadIdx.x;
  const int rib = tid / TPR;
  const int t = tid % TPR;
  const int64_t row = (int64_t)blockIdx.x * RPB + rib;
  const bool valid = row < n;
  const int64_t base = row * (int64_t)v;
  const int nvec = v / EPV;
  const float c1 = kLog2e * inv_temp;
  u32x4 rs[ITERS], rt[ITERS];
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
    const int c = i * TPR + t;
    if (valid && c < nvec) {
      rs[i] = load16_stream(student + base + (int64_t)c * EPV);
      rt[i] = load16_stream(teacher + base + (int64_t)c * EPV);
    }
  }
  float l2s, l2t;
  if constexpr (LOSS) {
    float ms = kNegBig, mt = kNegBig;
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      if (valid && i * TPR + t < nvec) {
        float zs[EPV], zt[EPV];
        Elem<T>::unpack(rs[i], zs);
        Elem<T>::unpack(rt[i], zt);
#pragma unroll
        for (int e = 0; e < EPV; ++e) { ms = fmaxf(ms, zs[e] * c1); mt = fmaxf(mt, zt[e] * c1); }
      }
    }
    ms = group_reduce<TPR, OpMax>(ms);
    mt = group_reduce<TPR, OpMax>(mt);
    float ds = 0.f, dt = 0.f, a = 0.f;
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      if (valid && i * TPR + t < nvec) {
        float zs[EPV], zt[EPV];
        Elem<T>::unpack(rs[i], zs);
        Elem<T>::unpack(rt[i], zt);
#pragma unroll
        for (int e = 0; e < EPV; ++e) {
          const float x = zs[e] * c1, y = zt[e] * c1;
          ds += fast_exp2(x - ms);
          const float et = fast_exp2(y - mt);
          dt += et;
          a += et * (y - x);
        }
      }
    }
    ds = group_reduce<TPR, OpSum>(ds);
    dt = group_reduce<TPR, OpSum>(dt);
    a = group_reduce<TPR, OpSum>(a);
    l2s = ms + fast_log2(ds);
    l2t = mt + fast_log2(dt);
    if (valid && t == 0) {
      if (lse_s != nullptr) lse_s[row] = l2s * kLn2;
      if (lse_t != nullptr) lse_t[row] = l2t * kLn2;
      row_kl[row] = (a / dt - l2t + l2s) * kLn2;
    }
  } else {
    l2s = valid ? lse_s[row] * kLog2e : 0.f;
    l2t = valid ? lse_t[row] * kLog2e : 0.f;
  }
  if constexpr (GRAD) {
    float g = mul;
    if (grad_out != nullptr && valid) g *= grad_per_row ? grad_out[row] : grad_out[0];
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      const int c = i * TPR + t;
      if (valid && c < nvec) {
        float zs[EPV], zt[EPV], o[EPV];
        Elem<T>::unpack(rs[i], zs);
        Elem<T>::unpack(rt[i], zt);
#pragma unroll
        for (int e = 0; e < EPV; ++e) o[e] = (fast_exp2(zs[e] * c1 - l2s) - fast_exp2(zt[e] * c1 - l2t)) * g;
        GT* dst = dstudent + base + (int64_t)c * EPV;
        if constexpr (sizeof(GT) == sizeof(T)) {
          store16_stream(dst, Elem<GT>::pack(o));
        } else {  // fp32 gradient next to 16-bit logits: two 16-byte stores
          static_assert(sizeof(GT) == 4 && EPV == 8, "gradient is the logits' dtype or fp32");
          float lo[4] = {o[0], o[1], o[2], o[3]}, hi[4] = {o[4], o[5], o[6], o[7]};
          store16_stream(dst, Elem<float>::pack(lo));
          store16_stream(dst + 4, Elem<float>::pack(hi));
        }
      }
    }
  }
}

// Widest row, in 16-byte vectors, of the vector lane-group kernel (tunable downwards with
// "rows_vec_max").
constexpr int kVRowsMaxVec = 256;

template <typename T, typename GT, bool LOSS, bool GRAD>
bool launch_vrows(const void* student, const void* teacher, float* lse_s, float* lse_t, float* row_kl,
                  const float* grad_out, int grad_per_row, void* dstudent, int64_t n, int v, float inv_temp,
                  float mul, hipStream_t st) {
  constexpr int EPV = Elem<T>::kVec;
  if (v % EPV != 0 || v / EPV > kVRowsMaxVec || !fm_host::aligned16(student) || !fm_host::aligned16(teacher) ||
      (GRAD && !fm_host::aligned16(dstudent)))
    return false;
  // two vectors of each row a lane where the rows have them: a wave then keeps 4 KiB in
  // flight, and narrow rows share it
  const int nvec = v / EPV;
  int tpr = 4;
  while (tpr < 64 && tpr * 2 < nvec) tpr *= 2;
  int iters = 1;
  while (tpr * iters < nvec) iters *= 2;
  const dim3 grid((unsigned)((n + 256 / tpr - 1) / (256 / tpr)));
#define GOV(TPR_, IT_)                                                                             \
  if (tpr == TPR_ && iters == IT_) {                                                               \
    FM_LAUNCH((kl_vrows_kernel<T, GT, TPR_, IT_, LOSS, GRAD>), grid, dim3(256), 0, st,    \
                       static_cast<const T*>(student), static_cast<const T*>(teacher), lse_s, lse_t, \
                       row_kl, grad_out, grad_per_row, static_cast<GT*>(dstudent), n, v, inv_temp, mul); \
    return true;                                                                                   \
  }
  GOV(4, 1) GOV(4, 2) GOV(8, 2) GOV(16, 2) GOV(32, 2) GOV(64, 2) GOV(64, 4)
#undef GOV
  return false;
}

constexpr int kRowsMaxV = 1024;
// widest row either lane-group kernel can take (the vector form, fp16 / bf16)
constexpr int kRowsReach = kVRowsMaxVec * 8 > kRowsMaxV ? kVRowsMaxVec * 8 : kRowsMaxV;

template <typename T, typename GT, bool LOSS, bool GRAD>
bool launch_rows(const void* student, const void* teacher, float* lse_s, float* lse_t, float* row_kl,
                 const float* grad_out, int grad_per_row, void* dstudent, int64_t n, int v, float inv_temp,
                 float mul, hipStream_t st) {
  if (launch_vrows<T, GT, LOSS, GRAD>(student, teacher, lse_s, lse_t, row_kl, grad_out, grad_per_row, dstudent,
                                      n, v, inv_temp, mul, st))
    return true;
  if (v > kRowsMaxV) return false;
  const int tpr = v <= 16 * 16 ? 16 : 64;
  int iters = 1;
  while (tpr * iters < v) iters *= 2;
  const dim3 grid((unsigned)((n + 256 / tpr - 1) / (256 / tpr)));
#define GOR(TPR_, IT_)                                                                             \
  if (tpr == TPR_ && iters == IT_) {                                                               \
    FM_LAUNCH((kl_rows_kernel<T, GT, TPR_, IT_, LOSS, GRAD>), grid, dim3(256), 0, st,     \
                       static_cast<const T*>(student), static_cast<const T*>(teacher), lse_s, lse_t, \
                       row_kl, grad_out, grad_per_row, static_cast<GT*>(dstudent), n, v, inv_temp, mul); \
    return true;                                                                                   \
  }
  GOR(16, 1) GOR(16, 2) GOR(16, 4) GOR(16, 8) GOR(16, 16) GOR(64, 8) GOR(64, 16)
#undef GOR
  return false;
}

#define FM_KL_BY_DTYPES(dtype, grad_dtype, CALL)                        \
  do {                                                                  \
    if ((dtype) == FM_F32) { CALL(float, float); }                      \
    else if ((dtype) == FM_BF16 && (grad_dtype) == FM_BF16) { CALL(bf16_t, bf16_t); } \
    else if ((dtype) == FM_BF16) { CALL(bf16_t, float); }               \
    else if ((grad_dtype) == FM_F16) { CALL(f16_t, f16_t); }            \
    else { CALL(f16_t, float); }                                        \
  } while (0)

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

int fm_kl_fwd(const void* student, const void* teacher, float* lse_s, float* lse_t, float* row_kl,
              float* loss, int64_t n, int64_t v, int dtype, float inv_temperature, int reduction,
              fm_stream_t stream) {
  int rc = check_shape("fm_kl_fwd", n, v, dtype);
  if (rc != FM_OK) return rc;
  FM_CHECK_ARG(reduction == FM_REDUCE_NONE || reduction == FM_REDUCE_SUM || reduction == FM_REDUCE_MEAN,
               "fm_kl_fwd: bad reduction %d", reduction);
  FM_CHECK_ARG(n == 0 || (student && teacher && lse_s && lse_t && row_kl), "fm_kl_fwd: NULL pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  bool narrow = false;
  if (n > 0 && v <= kRowsReach) {
#define CALL(T, GT) \
  narrow = launch_rows<T, GT, true, false>(student, teacher, lse_s, lse_t, row_kl, nullptr, 0, nullptr, n, \
                                           (int)v, inv_temperature, 0.f, st)
    FM_KL_BY_DTYPES(dtype, dtype, CALL);
#undef CALL
    if (narrow) FM_CHECK_LAUNCH("fm_kl_fwd");
  }
  if (n > 0 && !narrow) {
    const bool vec_ok = fm_host::aligned16(student) && fm_host::aligned16(teacher);
    if (dtype == FM_F32) launch_fwd<float>(student, teacher, lse_s, lse_t, row_kl, n, (int)v, inv_temperature, vec_ok, st);
    else if (dtype == FM_BF16) launch_fwd<bf16_t>(student, teacher, lse_s, lse_t, row_kl, n, (int)v, inv_temperature, vec_ok, st);
    else launch_fwd<f16_t>(student, teacher, lse_s, lse_t, row_kl, n, (int)v, inv_temperature, vec_ok, st);
    FM_CHECK_LAUNCH("fm_kl_fwd");
  }
  if (reduction != FM_REDUCE_NONE && loss != nullptr) {
    const float scale = (reduction == FM_REDUCE_MEAN && n > 0) ? 1.f / (float)n : 1.f;
    hipLaunchKernelGGL(kl_finalize_kernel, dim3(1), dim3(1024), 0, st, row_kl, n, scale, loss);
    FM_CHECK_LAUNCH("fm_kl_fwd(finalize)");
  }
  return FM_OK;
}

static int kl_topk_entry(const char* what, const void* student, const void* teacher, float* lse_s,
                         float* lse_t, float* row_kl, float* loss, void* dstudent, void* topk_values,
                         void* topk_indices, float* topk_probs, int64_t n, int64_t v, int k, int dtype,
                         int index_bits, float inv_temperature, int reduction, fm_stream_t stream) {
  int rc = check_shape(what, n, v, dtype);
  if (rc != FM_OK) return rc;
  FM_CHECK_ARG(reduction == FM_REDUCE_NONE || reduction == FM_REDUCE_SUM || reduction == FM_REDUCE_MEAN,
               "%s: bad reduction %d", what, reduction);
  FM_CHECK_ARG(index_bits == 32 || index_bits == 64, "%s: index_bits must be 32 or 64", what);
  FM_CHECK_ARG(k >= 1 && k <= v, "%s: selected index k out of range (k=%d, v=%lld)", what, k,
               (long long)v);
  FM_CHECK_ARG(inv_temperature > 0.f, "%s: the temperature must be positive", what);
  const int esize = dtype == FM_F32 ? 4 : 2;
  const int64_t nvec_max = v / (16 / esize);
  // rows past kFusedMaxVec vectors: one 1024-thread workgroup per compute unit, more than 64 KB of LDS
  const bool wide = nvec_max > kFusedMaxVec;
  bool wide_ok = !wide;
  if (wide && k <= kMaxK && nvec_max <= fm_host::kLdsWideMaxVec) {
#define ALLOW(T)                                                                                   \
  (dstudent != nullptr ? fm_host::allow_wide_lds<&kl_fwd_topk_kernel<T, 1024, 2, true>>()          \
                       : fm_host::allow_wide_lds<&kl_fwd_topk_kernel<T, 1024, 2, false>>())
    wide_ok = dtype == FM_F32 ? ALLOW(float) : (dtype == FM_BF16 ? ALLOW(bf16_t) : ALLOW(f16_t));
#undef ALLOW
  }
  if (k > kMaxK || !wide_ok) {
    fm_host::set_error("%s: k <= %d and rows of at most %d bytes are fused (k=%d, v=%lld); "
                       "call fm_kl_fwd and fm_topk instead", what, kMaxK, fm_host::kLdsWideMaxVec * 16, k,
                       (long long)v);
    return FM_ERR_UNSUPPORTED;
  }
  FM_CHECK_ARG(n == 0 || (student && teacher && lse_s && lse_t && row_kl && topk_indices),
               "%s: NULL pointer", what);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (n > 0) {
    const bool vec_ok = fm_host::aligned16(student) && fm_host::aligned16(teacher);
    int32_t* i32 = index_bits == 32 ? static_cast<int32_t*>(topk_indices) : nullptr;
    int64_t* i64 = index_bits == 64 ? static_cast<int64_t*>(topk_indices) : nullptr;
    int threads = fm_host::get_param(fm_host::P_VOCAB_THREADS);
    if (threads != 256 && threads != 1024) threads = 512;
    if (wide) threads = 1024;
    const size_t lds = (size_t)((nvec_max + 3) / 4 * 4 + 4) * sizeof(uint16_t);
    const dim3 grid((unsigned)n);
    // gradient (when asked for) is for an upstream gradient of 1
    const float mul = inv_temperature * ((reduction == FM_REDUCE_MEAN) ? 1.f / (float)n : 1.f);
#define LAUNCH_AS(T, TH, GRAD_)                                                                     \
  FM_LAUNCH((kl_fwd_topk_kernel<T, TH, 2, GRAD_>), grid, dim3(TH), lds, st,               \
                     static_cast<const T*>(student), static_cast<const T*>(teacher), lse_s, lse_t, \
                     row_kl, static_cast<T*>(topk_values), i32, i64, topk_probs,                   \
                     static_cast<T*>(dstudent), mul, (int)v, k, inv_temperature, vec_ok)
#define LAUNCH(T, TH)                         \
  do {                                        \
    if (dstudent != nullptr) LAUNCH_AS(T, TH, true); \
    else LAUNCH_AS(T, TH, false);             \
  } while (0)
#define BY_THREADS(T)                      \
  do {                                     \
    if (threads == 256) LAUNCH(T, 256);    \
    else if (threads == 512) LAUNCH(T, 512); \
    else LAUNCH(T, 1024);                  \
  } while (0)
    if (dtype == FM_F32) BY_THREADS(float);
    else if (dtype == FM_BF16) BY_THREADS(bf16_t);
    else BY_THREADS(f16_t);
#undef BY_THREADS
#undef LAUNCH
#undef LAUNCH_AS
    FM_CHECK_LAUNCH(what);
  }
  if (reduction != FM_REDUCE_NONE && loss != nullptr) {
    const float scale = (reduction == FM_REDUCE_MEAN && n > 0) ? 1.f / (float)n : 1.f;
    hipLaunchKernelGGL(kl_finalize_kernel, dim3(1), dim3(1024), 0, st, row_kl, n, scale, loss);
    FM_CHECK_LAUNCH(what);
  }
  return FM_OK;
}

int fm_kl_fwd_topk(const void* student, const void* teacher, float* lse_s, float* lse_t,
                   float* row_kl, float* loss, void* topk_values, void* topk_indices,
                   float* topk_probs, int64_t n, int64_t v, int k, int dtype, int index_bits,
                   float inv_temperature, int reduction, fm_stream_t stream) {
  return kl_topk_entry("fm_kl_fwd_topk", student, teacher, lse_s, lse_t, row_kl, loss, nullptr, topk_values,
                       topk_indices, topk_probs, n, v, k, dtype, index_bits, inv_temperature, reduction,
                       stream);
}

int fm_kl_loss_grad_topk(const void* student, const void* teacher, float* lse_s, float* lse_t,
                         float* row_kl, float* loss, void* dstudent, void* topk_values,
                         void* topk_indices, float* topk_probs, int64_t n, int64_t v, int k, int dtype,
                         int index_bits, float inv_temperature, int reduction, fm_stream_t stream) {
  FM_CHECK_ARG(reduction == FM_REDUCE_SUM || reduction == FM_REDUCE_MEAN,
               "fm_kl_loss_grad_topk: reduction must be sum or mean (got %d)", reduction);
  FM_CHECK_ARG(n == 0 || (dstudent != nullptr && dstudent != student),
               "fm_kl_loss_grad_topk: dstudent must be a buffer of its own");
  return kl_topk_entry("fm_kl_loss_grad_topk", student, teacher, lse_s, lse_t, row_kl, loss, dstudent,
                       topk_values, topk_indices, topk_probs, n, v, k, dtype, index_bits, inv_temperature,
                       reduction, stream);
}

int fm_kl_bwd(const void* student, const void* teacher, const float* lse_s, const float* lse_t,
              const float* grad_out, int grad_per_row, void* dstudent, int64_t n, int64_t v, int dtype,
              int grad_dtype, float inv_temperature, float scale, fm_stream_t stream) {
  int rc = check_shape("fm_kl_bwd", n, v, dtype);
  if (rc != FM_OK) return rc;
  FM_CHECK_ARG(grad_dtype == dtype || grad_dtype == FM_F32,
               "fm_kl_bwd: grad_dtype must equal dtype or be fp32 (dtype=%d grad_dtype=%d)", dtype,
               grad_dtype);
  if (n == 0) return FM_OK;
  FM_CHECK_ARG(student && teacher && lse_s && lse_t && dstudent, "fm_kl_bwd: NULL pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (v <= kRowsReach) {
    bool narrow = false;
#define CALL(T, GT)                                                                                 \
  narrow = launch_rows<T, GT, false, true>(student, teacher, const_cast<float*>(lse_s),             \
                                           const_cast<float*>(lse_t), nullptr, grad_out, grad_per_row, \
                                           dstudent, n, (int)v, inv_temperature, inv_temperature * scale, st)
    FM_KL_BY_DTYPES(dtype, grad_dtype, CALL);
#undef CALL
    if (narrow) {
      FM_CHECK_LAUNCH("fm_kl_bwd");
      return FM_OK;
    }
  }
  const bool vec_ok = fm_host::aligned16(student) && fm_host::aligned16(teacher) &&
                      fm_host::aligned16(dstudent);
#define CALL(T, GT) \
  launch_bwd<T, GT>(student, teacher, lse_s, lse_t, grad_out, grad_per_row, dstudent, n, (int)v, \
                    inv_temperature, scale, vec_ok, st)
  if (dtype == FM_F32) CALL(float, float);
  else if (dtype == FM_BF16 && grad_dtype == FM_BF16) CALL(bf16_t, bf16_t);
  else if (dtype == FM_BF16) CALL(bf16_t, float);
  else if (grad_dtype == FM_F16) CALL(f16_t, f16_t);
  else CALL(f16_t, float);
#undef CALL
  FM_CHECK_LAUNCH("fm_kl_bwd");
  return FM_OK;
}

int fm_kl_loss_grad(const void* student, const void* teacher, float* lse_s, float* lse_t,
                    float* row_kl, float* loss, void* dstudent, int64_t n, int64_t v, int dtype,
                    int grad_dtype, float inv_temperature, int reduction, fm_stream_t stream) {
  int rc = check_shape("fm_kl_loss_grad", n, v, dtype);
  if (rc != FM_OK) return rc;
  FM_CHECK_ARG(reduction == FM_REDUCE_SUM || reduction == FM_REDUCE_MEAN,
               "fm_kl_loss_grad: reduction must be sum or mean (got %d)", reduction);
  FM_CHECK_ARG(grad_dtype == dtype || grad_dtype == FM_F32,
               "fm_kl_loss_grad: grad_dtype must equal dtype or be fp32 (dtype=%d grad_dtype=%d)", dtype,
               grad_dtype);
  FM_CHECK_ARG(n == 0 || (student && teacher && row_kl && dstudent), "fm_kl_loss_grad: NULL pointer");
  FM_CHECK_ARG(dstudent != student || grad_dtype == dtype,
               "fm_kl_loss_grad: the gradient can overwrite the student only in the student's dtype");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const float scale = (reduction == FM_REDUCE_MEAN && n > 0) ? 1.f / (float)n : 1.f;
  const int esize = dtype == FM_F32 ? 4 : 2;
  const int64_t nvec = v / (16 / esize);
  if (n > 0 && v <= kRowsReach) {   // narrow rows: lane groups, in place allowed
    bool narrow = false;
#define CALL(T, GT)                                                                                  \
  narrow = launch_rows<T, GT, true, true>(student, teacher, lse_s, lse_t, row_kl, nullptr, 0, dstudent, n, \
                                          (int)v, inv_temperature, inv_temperature * scale, st)
    FM_KL_BY_DTYPES(dtype, grad_dtype, CALL);
#undef CALL
    if (narrow) {
      FM_CHECK_LAUNCH("fm_kl_loss_grad");
      if (loss != nullptr) {
        hipLaunchKernelGGL(kl_finalize_kernel, dim3(1), dim3(1024), 0, st, row_kl, n, scale, loss);
        FM_CHECK_LAUNCH("fm_kl_loss_grad(finalize)");
      }
      return FM_OK;
    }
  }
  // Aligned rows of more than 2048 vectors: the form that keeps the row pair on the chip (registers
  // and LDS of one to three workgroups per compute unit; more than 64 KB of LDS has to be granted
  // by the device once per kernel), the next row's loads under this row's gradient. It reads the row
  // once where the two sweeps of the wide form read it twice, and below 4096 vectors it beats the
  // register form wherever that one's power-of-two vectors per thread leave lanes idle. Measured
  // against what it replaced (us, 2^28 bf16 or 2^27 fp32 logits per tensor; r = the register form,
  // w = the two sweeps):
  //   bf16 columns 16384: 289 / 270 r (stays)   18432: 291 / 442 r   24576: 286 / 374 r
  //                32000: 292 / 364 r   40000: 321 / 351 w   50304: 310 / 347 w   65536: 315 / 372 w
  //                80000: 335 / 368 w  128256: 335 / 372 w  151936: 317 / 338 w  262144: 407 / 416 w
  //   fp32 columns  8192: 318 / 261 r (stays)    9216: 320 / 364 r   16384: 292 / 333 r
  //                32000: 294 / 358 w   65536: 306 / 379 w  128256: 336 / 409 w  262144: 393 / 440 w
  const bool aligned = fm_host::aligned16(student) && fm_host::aligned16(teacher) &&
                       fm_host::aligned16(dstudent);
  const bool held = n > 0 && aligned && nvec > 2048 && nvec <= 32768;
  const bool one_pass = n > 0 && aligned && nvec <= kOnePassMaxVec && !held;
  if (!one_pass) {
    if (n == 0) {
      return fm_kl_fwd(student, teacher, lse_s, lse_t, row_kl, loss, n, v, dtype, inv_temperature, reduction,
                       stream);
    }
    // wide (or unaligned) rows: two sweeps in one launch. With a
    // gradient in another dtype than the student the buffers must differ, which the argument
    // check above already ensures.
    const bool vec_ok = fm_host::aligned16(student) && fm_host::aligned16(teacher) &&
                        fm_host::aligned16(dstudent);
    const float mul_w = inv_temperature * scale;
    const dim3 wgrid((unsigned)n);
#define WIDE(T, GT)                                                                                \
  if (!(held && launch_held<T, GT>(static_cast<const T*>(student), static_cast<const T*>(teacher), \
                                   lse_s, lse_t, row_kl, static_cast<GT*>(dstudent), n, (int)v,   \
                                   nvec, inv_temperature, mul_w, vec_ok, st)))                     \
    FM_LAUNCH((kl_loss_grad_wide_kernel<T, GT, 1024, 2>), wgrid, dim3(1024), 0, st,                \
              static_cast<const T*>(student), static_cast<const T*>(teacher), lse_s, lse_t,        \
              row_kl, static_cast<GT*>(dstudent), (int)v, inv_temperature, mul_w, vec_ok)
    FM_KL_BY_DTYPES(dtype, grad_dtype, WIDE);
#undef WIDE
    FM_CHECK_LAUNCH("fm_kl_loss_grad");
    if (loss != nullptr) {
      hipLaunchKernelGGL(kl_finalize_kernel, dim3(1), dim3(1024), 0, st, row_kl, n, scale, loss);
      FM_CHECK_LAUNCH("fm_kl_loss_grad(finalize)");
    }
    return FM_OK;
  }
  // the fewest threads that hold both rows in at most 4 vectors each per thread
  int threads = 256;
  while (threads < 1024 && nvec > (int64_t)threads * 4) threads *= 2;
  int iters = 1;
  while ((int64_t)threads * iters < nvec) iters *= 2;
  const float mul = inv_temperature * scale;
  const dim3 grid((unsigned)n);
#define LAUNCH(T, GT, TH, IT)                                                                      \
  FM_LAUNCH((kl_loss_grad_kernel<T, GT, TH, IT>), grid, dim3(TH), 0, st,                  \
                     static_cast<const T*>(student), static_cast<const T*>(teacher), lse_s, lse_t, \
                     row_kl, static_cast<GT*>(dstudent), (int)v, inv_temperature, mul)
#define BY_ITERS(T, GT, TH)                       \
  do {                                            \
    if (iters == 1) LAUNCH(T, GT, TH, 1);         \
    else if (iters == 2) LAUNCH(T, GT, TH, 2);    \
    else LAUNCH(T, GT, TH, 4);                    \
  } while (0)
#define BY_SHAPE(T, GT)                               \
  do {                                                \
    if (threads == 256) BY_ITERS(T, GT, 256);         \
    else if (threads == 512) BY_ITERS(T, GT, 512);    \
    else BY_ITERS(T, GT, 1024);                       \
  } while (0)
  if (dtype == FM_F32) BY_SHAPE(float, float);
  else if (dtype == FM_BF16 && grad_dtype == FM_BF16) BY_SHAPE(bf16_t, bf16_t);
  else if (dtype == FM_BF16) BY_SHAPE(bf16_t, float);
  else if (grad_dtype == FM_F16) BY_SHAPE(f16_t, f16_t);
  else BY_SHAPE(f16_t, float);
#undef BY_SHAPE
#undef BY_ITERS
#undef LAUNCH
  FM_CHECK_LAUNCH("fm_kl_loss_grad");
  if (loss != nullptr) {
    hipLaunchKernelGGL(kl_finalize_kernel, dim3(1), dim3(1024), 0, st, row_kl, n, scale, loss);
    FM_CHECK_LAUNCH("fm_kl_loss_grad(finalize)");
  }
  return FM_OK;
}

}  // extern "C"
