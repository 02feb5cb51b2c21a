// Shared device helpers for the gfx950 (CDNA4, wave64) row kernels.
//
// Everything in this library is a memory-bound row reduction, so the helpers are about
// three things only: 16-byte global accesses, fp32 math on packed 16-bit storage, and
// fixed-order reductions (DPP inside a wave, LDS across waves; never a float atomic, so
// every result is run-to-run deterministic).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/fm_hip.h"

namespace fm {

constexpr int kWave = 64;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
// Finite stand-in for -inf as the running maximum of an online softmax: exp2(x - kNegBig)
// never produces inf - inf = NaN, and a row of true -inf still ends with a sum of zero.
constexpr float kNegBig = -3.0e38f;

struct bf16_t { uint16_t bits; };
struct f16_t { uint16_t bits; };

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2_hw __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_hw __attribute__((ext_vector_type(2)));

// ---------------------------------------------------------------- scalar conversions
// Bit casts always go through by-value scalars: __builtin_bit_cast applied directly to an
// element of an ext_vector (`v[i]`) reads element 0 with this compiler.
__device__ __forceinline__ float u2f(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t f2u(float f) { return __builtin_bit_cast(uint32_t, f); }
__device__ __forceinline__ float bf16_bits_to_float(uint32_t b) {
  return __builtin_bit_cast(float, b << 16);
}
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  f32x2 f = {lo, hi};
  bf16x2_hw h = __builtin_convertvector(f, bf16x2_hw);   // v_cvt_pk_bf16_f32, RNE
  return __builtin_bit_cast(uint32_t, h);
}
__device__ __forceinline__ uint32_t pack_f16(float lo, float hi) {
  f32x2 f = {lo, hi};
  f16x2_hw h = __builtin_convertvector(f, f16x2_hw);     // v_cvt_pk_f16_f32 (RNE)
  return __builtin_bit_cast(uint32_t, h);
}

template <typename T> struct Elem;

template <> struct Elem<float> {
  static constexpr int kVec = 4;          // elements per 16-byte access
  static constexpr int kDtype = FM_F32;
  __device__ static __forceinline__ float load1(const float* p) { return *p; }
  __device__ static __forceinline__ void store1(float* p, float v) { *p = v; }
  __device__ static __forceinline__ void unpack(const u32x4& r, float (&o)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t u = r[i];
      o[i] = u2f(u);
    }
  }
  __device__ static __forceinline__ u32x4 pack(const float (&v)[4]) {
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float f = v[i];
      r[i] = f2u(f);
    }
    return r;
  }
  __device__ static __forceinline__ float round(float v) { return v; }
};

template <> struct Elem<bf16_t> {
  static constexpr int kVec = 8;
  static constexpr int kDtype = FM_BF16;
  __device__ static __forceinline__ float load1(const bf16_t* p) {
    return bf16_bits_to_float(p->bits);
  }
  __device__ static __forceinline__ void store1(bf16_t* p, float v) {
    p->bits = (uint16_t)(pack_bf16(v, 0.f) & 0xffffu);
  }
  __device__ static __forceinline__ void unpack(const u32x4& r, float (&o)[8]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t u = r[i];
      o[2 * i] = u2f(u << 16);
      o[2 * i + 1] = u2f(u & 0xffff0000u);
    }
  }
  __device__ static __forceinline__ u32x4 pack(const float (&v)[8]) {
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = pack_bf16(v[2 * i], v[2 * i + 1]);
    return r;
  }
  // value after one rounding to the storage type (what a bf16 tensor op would have stored)
  __device__ static __forceinline__ float round(float v) {
    return __builtin_bit_cast(float, (pack_bf16(v, 0.f) & 0xffffu) << 16);
  }
};

template <> struct Elem<f16_t> {
  static constexpr int kVec = 8;
  static constexpr int kDtype = FM_F16;
  __device__ static __forceinline__ float load1(const f16_t* p) {
    const uint16_t b = p->bits;
    return (float)__builtin_bit_cast(_Float16, b);
  }
  __device__ static __forceinline__ void store1(f16_t* p, float v) {
    const _Float16 hv = (_Float16)v;
    p->bits = __builtin_bit_cast(uint16_t, hv);
  }
  __device__ static __forceinline__ void unpack(const u32x4& r, float (&o)[8]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t u = r[i];
      const uint16_t lo = (uint16_t)(u & 0xffffu), hi = (uint16_t)(u >> 16);
      o[2 * i] = (float)__builtin_bit_cast(_Float16, lo);
      o[2 * i + 1] = (float)__builtin_bit_cast(_Float16, hi);
    }
  }
  __device__ static __forceinline__ u32x4 pack(const float (&v)[8]) {
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = pack_f16(v[2 * i], v[2 * i + 1]);
    return r;
  }
  __device__ static __forceinline__ float round(float v) { return (float)(_Float16)v; }
};

// ---------------------------------------------------------------- 16-byte global access
template <typename T>
__device__ __forceinline__ u32x4 load16(const T* p) {
  return *reinterpret_cast<const u32x4*>(p);
}
// Streaming variants: data that is touched once should not evict what is re-read.
template <typename T>
__device__ __forceinline__ u32x4 load16_stream(const T* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
}
template <typename T>
__device__ __forceinline__ void store16(T* p, const u32x4& v) {
  *reinterpret_cast<u32x4*>(p) = v;
}
template <typename T>
__device__ __forceinline__ void store16_stream(T* p, const u32x4& v) {
  __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p));
}

// 16 bytes per lane from global memory straight into LDS, no register in between
// (global_load_lds_dwordx4): lane i of the wave writes wave_base[i]. `wave_base` is the same for
// every lane of the wave; `src` is the lane's own address. Non-temporal like load16_stream.
// The data is in LDS once the wave's outstanding vector-memory count says so (wait_vmem_all).
template <typename T>
__device__ __forceinline__ void load16_stream_to_lds(const T* src, u32x4* wave_base) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                   (__attribute__((address_space(3))) void*)wave_base, 16, 0, /*nt*/ 2);
}
// every vector-memory operation of this wave issued so far has completed
__device__ __forceinline__ void wait_vmem_all() { __builtin_amdgcn_s_waitcnt(0x0F70); }

// Unpack a vector that is used by several passes without letting the compiler keep the
// converted floats of the first pass alive for the later ones (fp16 conversions are otherwise
// hoisted, and eight vectors per lane then take 230 registers instead of 60). FRESH = false is
// the plain unpack.
template <typename T, bool FRESH, int N>
__device__ __forceinline__ void unpack_again(u32x4 raw, float (&f)[N]) {
  if constexpr (FRESH) asm volatile("" : "+v"(raw.x), "+v"(raw.y), "+v"(raw.z), "+v"(raw.w));
  Elem<T>::unpack(raw, f);
}

// Marks the point where a loaded vector is taken into use, unconditionally. Without it the
// compiler sinks a load whose only use sits behind a lane-dependent branch into that branch, and
// then has to wait for every outstanding load before the next one may reuse the register; with it
// the wait for vector u sits in straight-line code and counts exactly the loads issued after it.
__device__ __forceinline__ void touch(u32x4& raw) {
  asm volatile("" : "+v"(raw.x), "+v"(raw.y), "+v"(raw.z), "+v"(raw.w));
}
// The same with the vector as ONE operand: its four registers stay a tuple. (With four operands
// they become four values of their own, which the register allocator may keep apart; where it
// does, the halves are copied out of the load's destination right behind the load, behind a wait
// for it.) For kernels that keep many loaded vectors alive across several passes.
__device__ __forceinline__ void touch_whole(u32x4& raw) { asm("" : "+v"(raw)); }

// ---------------------------------------------------------------- wave reductions (DPP)
__device__ __forceinline__ int lane_id() {
  return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}

#define FM_DPP_F(v, ctrl) \
  __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, (v)), (ctrl), 0xf, 0xf, false))
#define FM_DPP_I(v, ctrl) __builtin_amdgcn_update_dpp(0, (v), (ctrl), 0xf, 0xf, false)

constexpr int kDppXor1 = 0xB1;        // quad_perm:[1,0,3,2]
constexpr int kDppXor2 = 0x4E;        // quad_perm:[2,3,0,1]
constexpr int kDppHalfMirror = 0x141; // row_half_mirror (lane i <-> 7-i inside 8)
constexpr int kDppMirror = 0x140;     // row_mirror      (lane i <-> 15-i inside 16)

__device__ __forceinline__ float readlane_f(float v, int l) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), l));
}

struct OpSum { __device__ static __forceinline__ float f(float a, float b) { return a + b; } };
struct OpMax { __device__ static __forceinline__ float f(float a, float b) { return fmaxf(a, b); } };

// Reduce over aligned groups of G consecutive lanes (G a power of two <= 64); every lane of
// a group ends with the group's result. The combination order is fixed by the lane layout.
template <int G, typename Op>
__device__ __forceinline__ float group_reduce(float v) {
  if constexpr (G >= 2) v = Op::f(v, FM_DPP_F(v, kDppXor1));
  if constexpr (G >= 4) v = Op::f(v, FM_DPP_F(v, kDppXor2));
  if constexpr (G >= 8) v = Op::f(v, FM_DPP_F(v, kDppHalfMirror));
  if constexpr (G >= 16) v = Op::f(v, FM_DPP_F(v, kDppMirror));
  if constexpr (G == 32) {
    v = Op::f(v, __shfl_xor(v, 16, 64));
  }
  if constexpr (G == 64) {
    float a = readlane_f(v, 0), b = readlane_f(v, 16), c = readlane_f(v, 32), d = readlane_f(v, 48);
    v = Op::f(Op::f(a, b), Op::f(c, d));
  }
  return v;
}

__device__ __forceinline__ float wave_sum(float v) { return group_reduce<64, OpSum>(v); }
__device__ __forceinline__ float wave_max(float v) { return group_reduce<64, OpMax>(v); }

__device__ __forceinline__ int wave_sum_i(int v) {
  v += FM_DPP_I(v, kDppXor1);
  v += FM_DPP_I(v, kDppXor2);
  v += FM_DPP_I(v, kDppHalfMirror);
  v += FM_DPP_I(v, kDppMirror);
  return __builtin_amdgcn_readlane(v, 0) + __builtin_amdgcn_readlane(v, 16) +
         __builtin_amdgcn_readlane(v, 32) + __builtin_amdgcn_readlane(v, 48);
}

__device__ __forceinline__ uint32_t wave_max_u(uint32_t v) {
  auto mx = [](uint32_t a, uint32_t b) { return a > b ? a : b; };
  v = mx(v, (uint32_t)FM_DPP_I((int)v, kDppXor1));
  v = mx(v, (uint32_t)FM_DPP_I((int)v, kDppXor2));
  v = mx(v, (uint32_t)FM_DPP_I((int)v, kDppHalfMirror));
  v = mx(v, (uint32_t)FM_DPP_I((int)v, kDppMirror));
  const uint32_t a = (uint32_t)__builtin_amdgcn_readlane((int)v, 0), b = (uint32_t)__builtin_amdgcn_readlane((int)v, 16);
  const uint32_t c = (uint32_t)__builtin_amdgcn_readlane((int)v, 32), d = (uint32_t)__builtin_amdgcn_readlane((int)v, 48);
  return mx(mx(a, b), mx(c, d));
}

__device__ __forceinline__ int wave_min_i(int v) {
  auto mn = [](int a, int b) { return a < b ? a : b; };
  v = mn(v, FM_DPP_I(v, kDppXor1));
  v = mn(v, FM_DPP_I(v, kDppXor2));
  v = mn(v, FM_DPP_I(v, kDppHalfMirror));
  v = mn(v, FM_DPP_I(v, kDppMirror));
  return mn(mn(__builtin_amdgcn_readlane(v, 0), __builtin_amdgcn_readlane(v, 16)),
            mn(__builtin_amdgcn_readlane(v, 32), __builtin_amdgcn_readlane(v, 48)));
}

// The same two over aligned groups of L consecutive lanes (L = 8, 16, 32 or 64); every lane of a
// group ends with the group's result.
template <int L>
__device__ __forceinline__ uint32_t group_max_u(uint32_t v) {
  static_assert(L == 8 || L == 16 || L == 32 || L == 64, "group of 8, 16, 32 or 64 lanes");
  if constexpr (L == 64) return wave_max_u(v);
  auto mx = [](uint32_t a, uint32_t b) { return a > b ? a : b; };
  v = mx(v, (uint32_t)FM_DPP_I((int)v, kDppXor1));
  v = mx(v, (uint32_t)FM_DPP_I((int)v, kDppXor2));
  v = mx(v, (uint32_t)FM_DPP_I((int)v, kDppHalfMirror));
  if constexpr (L >= 16) v = mx(v, (uint32_t)FM_DPP_I((int)v, kDppMirror));
  if constexpr (L >= 32) v = mx(v, (uint32_t)__shfl_xor((int)v, 16, 64));
  return v;
}

template <int L>
__device__ __forceinline__ int group_min_i(int v) {
  static_assert(L == 8 || L == 16 || L == 32 || L == 64, "group of 8, 16, 32 or 64 lanes");
  if constexpr (L == 64) return wave_min_i(v);
  auto mn = [](int a, int b) { return a < b ? a : b; };
  v = mn(v, FM_DPP_I(v, kDppXor1));
  v = mn(v, FM_DPP_I(v, kDppXor2));
  v = mn(v, FM_DPP_I(v, kDppHalfMirror));
  if constexpr (L >= 16) v = mn(v, FM_DPP_I(v, kDppMirror));
  if constexpr (L >= 32) v = mn(v, __shfl_xor(v, 16, 64));
  return v;
}

// Reduce across the T threads that share one row. T <= 64: a lane group inside one wave.
// T > 64: T/64 whole waves of one workgroup; partials go through LDS and are combined in
// wave order. `smem` must hold (rows per block) * (T/64) floats; `row_in_block` selects the
// slice. Contains __syncthreads() when T > 64, so every thread of the block must call it.
template <int T, typename Op>
__device__ __forceinline__ float row_reduce(float v, float* smem, int row_in_block, int tid_in_row) {
  if constexpr (T <= 64) {
    return group_reduce<T, Op>(v);
  } else {
    constexpr int W = T / 64;
    v = group_reduce<64, Op>(v);
    if ((tid_in_row & 63) == 0) smem[row_in_block * W + (tid_in_row >> 6)] = v;
    __syncthreads();
    float r = smem[row_in_block * W];
#pragma unroll
    for (int i = 1; i < W; ++i) r = Op::f(r, smem[row_in_block * W + i]);
    __syncthreads();
    return r;
  }
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

}  // namespace fm

// ---------------------------------------------------------------- host-side plumbing
namespace fm_host {

void set_error(const char* fmt, ...);
int get_param(int which);

// Launch-shape parameters a caller may move for another part or shape (fm_set_param); none of
// them selects between code paths, the results do not depend on them.
enum Param { P_NORM_BWD_BLOCKS_PER_CU = 0, P_NORM_FWD_BLOCKS_PER_CU, P_VOCAB_THREADS, P_VOCAB_UNROLL, P_COUNT };

int num_cus();  // compute units of the current device (cached per device)

// Which kernel did the work: every launch of a main kernel (not the small finishing kernels)
// leaves the kernel's host-side handle for fm_last_kernel(), which asks the runtime for the
// device function's name and demangles it, so the name (template arguments resolved) cannot
// drift from what was launched.
void note_kernel(const void* host_function);

#define FM_LAUNCH(K, grid, block, shmem, st, ...)                    \
  do {                                                               \
    fm_host::note_kernel(reinterpret_cast<const void*>(&K));         \
    hipLaunchKernelGGL(K, grid, block, shmem, st, __VA_ARGS__);      \
  } while (0)

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Dynamic LDS beyond 64 KB has to be allowed per kernel and device before the first such launch;
// K is the kernel's address, `bytes` the most it will ever ask for. False when the device says no
// (the caller then takes a form that needs less).
template <auto K>
bool grant_dynamic_lds(int bytes) {
  static std::atomic<uint64_t> allowed{0};   // one bit per device
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return false;
  if ((allowed.load(std::memory_order_acquire) >> dev) & 1u) return true;
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(K), hipFuncAttributeMaxDynamicSharedMemorySize,
                          bytes) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  allowed.fetch_or(1ull << dev, std::memory_order_release);
  return true;
}

// Workgroups of kernel K (`threads` threads, `dynamic_lds` bytes) one compute unit holds at once,
// asked of the runtime once per kernel: the grid of a persistent kernel is this many per compute
// unit and no more (a workgroup beyond them would start when the others have done their whole share).
template <auto K>
int resident_per_cu(int threads, size_t dynamic_lds) {
  static std::atomic<int> cached{0};
  int o = cached.load(std::memory_order_relaxed);
  if (o == 0) {
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&o, K, threads, dynamic_lds) != hipSuccess || o < 1) {
      (void)hipGetLastError();
      o = 1;
    }
    cached.store(o, std::memory_order_relaxed);
  }
  return o;
}

#define FM_CHECK_ARG(cond, ...)                 \
  do {                                          \
    if (!(cond)) {                              \
      fm_host::set_error(__VA_ARGS__);          \
      return FM_ERR_INVALID;                    \
    }                                           \
  } while (0)

#define FM_CHECK_LAUNCH(what)                                                   \
  do {                                                                          \
    hipError_t e__ = hipGetLastError();                                         \
    if (e__ != hipSuccess) {                                                    \
      fm_host::set_error("%s: launch failed: %s", what, hipGetErrorString(e__)); \
      return FM_ERR_LAUNCH;                                                     \
    }                                                                           \
  } while (0)

}  // namespace fm_host
