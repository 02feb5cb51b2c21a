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
// All exponentials run in the base-2 domain; the temperature is folded into the scale.
#include "fm_vocab.cuh"

using namespace fm;

namespace {

struct KLState {
  float ms, ds, mt, dt, a;
};

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
      const int c = c0 + u * THREADS + tid;
      if (c < sp.nvec) {
        rs[u] = load16_stream(sp_ + sp.head + (int64_t)c * EPV);
        rt[u] = load16_stream(tp_ + sp.head + (int64_t)c * EPV);
      }
    }
    float zs[UNROLL][EPV], zt[UNROLL][EPV];
    float cms = k.ms, cmt = k.mt;
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int c = c0 + u * THREADS + tid;
      if (c < sp.nvec) {
        Elem<T>::unpack(rs[u], zs[u]);
        Elem<T>::unpack(rt[u], zt[u]);
#pragma unroll
        for (int e = 0; e < EPV; ++e) {
          zs[u][e] *= c1;
          zt[u][e] *= c1;
          cms = fmaxf(cms, zs[u][e]);
          cmt = fmaxf(cmt, zt[u][e]);
        }
      } else {
#pragma unroll
        for (int e = 0; e < EPV; ++e) { zs[u][e] = -INFINITY; zt[u][e] = -INFINITY; }
      }
    }
    float ds = k.ds * fast_exp2(k.ms - cms);
    const float ft = fast_exp2(k.mt - cmt);
    float dt = k.dt * ft;
    float a = k.a * ft;
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int c = c0 + u * THREADS + tid;
      if (c < sp.nvec) {   // uniform per vector; keeps (-inf) - (-inf) out of the A term
#pragma unroll
        for (int e = 0; e < EPV; ++e) {
          ds += fast_exp2(zs[u][e] - cms);
          const float et = fast_exp2(zt[u][e] - cmt);
          dt += et;
          a += et * (zt[u][e] - zs[u][e]);
        }
      }
    }
    k.ms = cms; k.ds = ds; k.mt = cmt; k.dt = dt; k.a = a;
  }
  const int ne = edge_count(sp, v);
  for (int e = tid; e < ne; e += THREADS) {
    const int col = edge_col(sp, e);
    const float zs = Elem<T>::load1(sp_ + col) * c1;
    const float zt = Elem<T>::load1(tp_ + col) * c1;
    const float cms = fmaxf(k.ms, zs), cmt = fmaxf(k.mt, zt);
    k.ds = k.ds * fast_exp2(k.ms - cms) + fast_exp2(zs - cms);
    const float ft = fast_exp2(k.mt - cmt);
    const float et = fast_exp2(zt - cmt);
    k.dt = k.dt * ft + et;
    k.a = k.a * ft + et * (zt - zs);
    k.ms = cms; k.mt = cmt;
  }

  // workgroup merge: maxima first (exact), then rescaled sums in lane / wave order
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
  if (tid == 0) {
    const float l2s = Ms + fast_log2(Ds), l2t = Mt + fast_log2(Dt);
    lse_s[row] = l2s * kLn2;
    lse_t[row] = l2t * kLn2;
    row_kl[row] = (A / Dt - l2t + l2s) * kLn2;
  }
}

// loss = sum(row_kl) * scale in a fixed order (thread i adds rows i, i+1024, ...).
__global__ __launch_bounds__(1024) void kl_finalize_kernel(const float* __restrict__ row_kl,
                                                           int64_t n, float scale,
                                                           float* __restrict__ loss) {
  __shared__ float sf[16];
  float a = 0.f;
  for (int64_t i = threadIdx.x; i < n; i += 1024) a += row_kl[i];
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
                                                          bool vec_ok) {
  constexpr int EPV = Elem<T>::kVec;
  const int64_t row = blockIdx.x;
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

  for (int c0 = 0; c0 < sp.nvec; c0 += THREADS * UNROLL) {
    u32x4 rs[UNROLL], rt[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int c = c0 + u * THREADS + tid;
      if (c < sp.nvec) {
        rs[u] = load16_stream(sp_ + sp.head + (int64_t)c * EPV);
        rt[u] = load16_stream(tp_ + sp.head + (int64_t)c * EPV);
      }
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

template <typename T>
void launch_fwd(const void* s, const void* t, float* lse_s, float* lse_t, float* row_kl, int64_t n,
                int v, float inv_temp, bool vec_ok, hipStream_t st) {
  const T* sp = static_cast<const T*>(s);
  const T* tp = static_cast<const T*>(t);
  const fm_host::VocabShape sh = fm_host::vocab_shape(v, sizeof(T), 512, 2);
  const dim3 grid((unsigned)n);
#define LAUNCH(TH, UN)                                                                            \
  hipLaunchKernelGGL((kl_fwd_kernel<T, TH, UN>), grid, dim3(TH), 0, st, sp, tp, lse_s, lse_t, row_kl, \
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
  const dim3 grid((unsigned)n);
#define LAUNCH(TH, UN)                                                                           \
  hipLaunchKernelGGL((kl_bwd_kernel<T, GT, TH, UN>), grid, dim3(TH), 0, st, sp, tp, lse_s, lse_t, \
                     grad_out, grad_per_row, gp, v, inv_temp, scale, vec_ok)
  FM_VOCAB_DISPATCH(sh, LAUNCH);
#undef LAUNCH
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

int fm_kl_fwd(const void* student, const void* teacher, float* lse_s, float* lse_t, float* row_kl,
              float* loss, int64_t n, int64_t v, int dtype, float inv_temperature, int reduction,
              fm_stream_t stream) {
  int rc = check_shape("fm_kl_fwd", n, v, dtype);
  if (rc != FM_OK) return rc;
  FM_CHECK_ARG(reduction == FM_REDUCE_NONE || reduction == FM_REDUCE_SUM || reduction == FM_REDUCE_MEAN,
               "fm_kl_fwd: bad reduction %d", reduction);
  FM_CHECK_ARG(n == 0 || (student && teacher && lse_s && lse_t && row_kl), "fm_kl_fwd: NULL pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (n > 0) {
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

}  // extern "C"
