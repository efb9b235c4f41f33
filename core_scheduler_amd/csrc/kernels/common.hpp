// Shared device helpers for the gfx950 kernels: storage <-> fp32 conversion,
// 128-bit vector access, wavefront-64 and workgroup reductions, launch checks.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "cs_hip_kernels.h"

namespace cs_hip {

constexpr int kWave = 64;  // CDNA wavefront width

// ---------------------------------------------------------------- storage
struct bf16_t {
  uint16_t bits;
};
struct f16_t {
  _Float16 v;
};

template <typename T>
struct Acc {
  using type = float;
};
template <>
struct Acc<double> {
  using type = double;
};

__device__ __forceinline__ float to_acc(float x) { return x; }
__device__ __forceinline__ double to_acc(double x) { return x; }
__device__ __forceinline__ float to_acc(f16_t x) { return (float)x.v; }
__device__ __forceinline__ float to_acc(bf16_t x) {
  return __uint_as_float((uint32_t)x.bits << 16);
}

// fp32 -> bf16, round to nearest even, NaN stays NaN (quiet).
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  __bf16 h = (__bf16)f;  // v_cvt_pk_bf16_f32 on gfx950
  return __builtin_bit_cast(uint16_t, h);
}

template <typename T>
__device__ __forceinline__ T from_acc(typename Acc<T>::type x);
template <>
__device__ __forceinline__ float from_acc<float>(float x) {
  return x;
}
template <>
__device__ __forceinline__ double from_acc<double>(double x) {
  return x;
}
template <>
__device__ __forceinline__ f16_t from_acc<f16_t>(float x) {
  // The float result is rounded to half here and nowhere else: without the empty asm the
  // compiler may merge this conversion into the multiply or add that produced x (one rounding
  // of the exact result instead of two), which changes ties and makes variants of a kernel
  // disagree in the last bit.
  asm volatile("" : "+v"(x));
  f16_t r;
  r.v = (_Float16)x;
  return r;
}
template <>
__device__ __forceinline__ bf16_t from_acc<bf16_t>(float x) {
  bf16_t r;
  r.bits = f32_to_bf16_bits(x);
  return r;
}

// x rounded to T's precision and widened again, for arithmetic that must see what a store to
// T followed by a load would give.
template <typename T>
__device__ __forceinline__ typename Acc<T>::type round_through(typename Acc<T>::type x) {
  return to_acc(from_acc<T>(x));
}
template <>
__device__ __forceinline__ float round_through<f16_t>(float x) {
  return (float)from_acc<f16_t>(x).v;  // from_acc keeps the conversion a separate rounding
}

// ------------------------------------------------------- 128-bit vectors
// VecN<T>::n elements of T in one 16-byte access.
template <typename T>
struct alignas(16) Vec16 {
  static constexpr int n = 16 / sizeof(T);
  T e[n];
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename T>
__device__ __forceinline__ Vec16<T> load16(const T *p) {
  // one global_load_dwordx4
  const u32x4 raw = *reinterpret_cast<const u32x4 *>(p);
  return __builtin_bit_cast(Vec16<T>, raw);
}
template <typename T>
__device__ __forceinline__ void store16(T *p, const Vec16<T> &v) {
  *reinterpret_cast<u32x4 *>(p) = __builtin_bit_cast(u32x4, v);
}
// Streaming variants: the data is touched once, so mark the access
// nontemporal and keep it from displacing lines that are reused.
template <typename T>
__device__ __forceinline__ Vec16<T> load16_stream(const T *p) {
  const u32x4 raw = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
  return __builtin_bit_cast(Vec16<T>, raw);
}
// Every streaming store of the library goes through here.  Stores with the agent-scope
// write-through bit (sc1, alone or with nt) were measured instead: a flat copy gains 2-6% at
// 100-400 MB, but the kernels of this library ran up to 8% slower with them, so it stays nt.
__device__ __forceinline__ void store_stream(u32x4 *p, const u32x4 v) { __builtin_nontemporal_store(v, p); }
template <typename T>
__device__ __forceinline__ void store16_stream(T *p, const Vec16<T> &v) {
  store_stream(reinterpret_cast<u32x4 *>(p), __builtin_bit_cast(u32x4, v));
}

__host__ __device__ __forceinline__ bool is_aligned16(const void *p) {
  return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

// ------------------------------------------------------------ reductions
struct SumOp {
  template <typename A>
  __device__ __forceinline__ A operator()(A a, A b) const {
    return a + b;
  }
};
struct MaxOp {
  template <typename A>
  __device__ __forceinline__ A operator()(A a, A b) const {
    return a > b ? a : b;
  }
};

// Butterfly over the 64 lanes of a wavefront through the LDS crossbar
// (ds_bpermute); every lane ends with the full result and the combination
// order is fixed, so results are reproducible.  Works for any 4/8-byte type.
template <typename A, typename Op>
__device__ __forceinline__ A wave_reduce_generic(A v, Op op) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) {
    v = op(v, __shfl_xor(v, off, kWave));
  }
  return v;
}

// DPP lane exchanges inside a row of 16 lanes: no LDS traffic, a few cycles.
// All 64 lanes must be active.
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
  const int r = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false);
  return __builtin_bit_cast(float, r);
}
template <int CTRL>
__device__ __forceinline__ int dpp_i32(int v) {
  return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, false);
}
constexpr int kDppQuadXor1 = 0xB1;     // quad_perm [1,0,3,2]
constexpr int kDppQuadXor2 = 0x4E;     // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141;  // lane i <-> 7-i inside each 8
constexpr int kDppRowMirror = 0x140;   // lane i <-> 15-i inside each 16

// fp32 wavefront all-reduce: four DPP steps give every lane its row's
// result, four v_readlane + three ops fold the four rows.  Fixed order.
template <typename Op>
__device__ __forceinline__ float wave_reduce(float v, Op op) {
  v = op(v, dpp_f32<kDppQuadXor1>(v));
  v = op(v, dpp_f32<kDppQuadXor2>(v));
  v = op(v, dpp_f32<kDppHalfMirror>(v));
  v = op(v, dpp_f32<kDppRowMirror>(v));
  const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
  const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 16));
  const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
  const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 48));
  return op(op(r0, r1), op(r2, r3));
}
template <typename Op>
__device__ __forceinline__ int wave_reduce(int v, Op op) {
  v = op(v, dpp_i32<kDppQuadXor1>(v));
  v = op(v, dpp_i32<kDppQuadXor2>(v));
  v = op(v, dpp_i32<kDppHalfMirror>(v));
  v = op(v, dpp_i32<kDppRowMirror>(v));
  const int r0 = __builtin_amdgcn_readlane(v, 0), r1 = __builtin_amdgcn_readlane(v, 16);
  const int r2 = __builtin_amdgcn_readlane(v, 32), r3 = __builtin_amdgcn_readlane(v, 48);
  return op(op(r0, r1), op(r2, r3));
}
template <typename Op>
__device__ __forceinline__ double wave_reduce(double v, Op op) {
  return wave_reduce_generic(v, op);
}

// Workgroup reduction through LDS.  `scratch` holds one A per wavefront.
// All threads of the workgroup must call it; all get the result.  The caller
// must not reuse `scratch` for something else without a barrier in between.
template <typename A, typename Op>
__device__ __forceinline__ A block_reduce(A v, Op op, A identity, A *scratch) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  const int n_waves = (blockDim.x + kWave - 1) >> 6;
  v = wave_reduce(v, op);
  if (n_waves == 1) return v;
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  A r = lane < n_waves ? scratch[lane] : identity;
  r = wave_reduce(r, op);
  __syncthreads();
  return r;
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() carries a workgroup-scope fence,
// for which the compiler waits until every global store the wave has issued is acknowledged
// (s_waitcnt vmcnt(0)): behind a row's worth of streaming stores that is one to two microseconds.
// Here a wave only waits for its own LDS accesses before it joins the barrier.  Use it where the
// data exchanged between the waves lives in the LDS and nowhere else.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// ------------------------------------------------------------ host side
inline int launch_status() {
  const hipError_t e = hipGetLastError();
  return e == hipSuccess ? CS_OK : (int)e;
}

inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

inline bool aligned_to(const void *p, size_t a) {
  return (reinterpret_cast<uintptr_t>(p) % a) == 0;
}

inline size_t dtype_size(int dtype) {
  switch (dtype) {
    case CS_F32: return 4;
    case CS_F64: return 8;
    case CS_F16: return 2;
    case CS_BF16: return 2;
    default: return 0;
  }
}

template <typename A, typename B>
constexpr inline A ceil_div(A a, B b) {
  return (a + b - 1) / b;
}

}  // namespace cs_hip
