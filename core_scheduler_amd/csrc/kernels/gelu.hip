// GeLU forward / backward for gfx950, exact (erf) and tanh-approximated.
//
// The reference op is at::gelu / at::gelu_backward (src/compute/gelu.cpp:39,
// :61-62); its formulas and constants are ATen's (native/cpu/Gelu.h:
// kGeluBeta = sqrt(2) * 2/sqrt(pi) * 0.5, kGeluKappa = 0.044715, reduced
// precision inputs widened to float first).
//
// Elementwise and HBM bound: 2 accesses per element forward, 3 backward, each
// lane moving 16 bytes per access.  At bf16 the budget is about 19 VALU lane
// cycles per element forward, which libm's tanhf would exceed, so 16-bit
// storage uses the identity 0.5*(1+tanh(u)) = 1/(1+exp(-2u)) with the hardware
// exp2 and reciprocal (1 ulp each, far inside the 8-bit mantissa of the
// result); the exact form uses an erfc polynomial for 16-bit storage (see below);
// fp32/fp64 storage uses libm and ATen's expression as written.
#include "common.hpp"

#include <math.h>

namespace cs_hip {
namespace {

constexpr double kBeta = 1.41421356237309504880 * 1.12837916709551257390 * 0.5;  // sqrt(2/pi)
constexpr double kKappa = 0.044715;
constexpr double kAlpha = 0.70710678118654752440;     // 1/sqrt(2)
constexpr double kPdfScale = 0.39894228040143267794;  // 1/sqrt(2 pi)
constexpr double kLog2e = 1.44269504088896340736;

// ---------------------------------------------------------------- accurate
template <typename U>
__device__ __forceinline__ U gelu_erf_fwd(U x) {
  return x * (U)0.5 * ((U)1 + erf(x * (U)kAlpha));
}
template <>
__device__ __forceinline__ float gelu_erf_fwd<float>(float x) {
  return x * 0.5f * (1.0f + erff(x * (float)kAlpha));
}
template <typename U>
__device__ __forceinline__ U gelu_erf_bwd(U dy, U x) {
  const U cdf = (U)0.5 * ((U)1 + erf(x * (U)kAlpha));
  const U pdf = exp((U)-0.5 * x * x) * (U)kPdfScale;
  return dy * (cdf + x * pdf);
}
template <>
__device__ __forceinline__ float gelu_erf_bwd<float>(float dy, float x) {
  const float cdf = 0.5f * (1.0f + erff(x * (float)kAlpha));
  const float pdf = expf(-0.5f * x * x) * (float)kPdfScale;
  return dy * (cdf + x * pdf);
}
template <typename U>
__device__ __forceinline__ U gelu_tanh_fwd(U x) {
  const U inner = (U)kBeta * (x + (U)kKappa * (x * x * x));
  return (U)0.5 * x * ((U)1 + tanh(inner));
}
template <>
__device__ __forceinline__ float gelu_tanh_fwd<float>(float x) {
  const float inner = (float)kBeta * (x + (float)kKappa * (x * x * x));
  return 0.5f * x * (1.0f + tanhf(inner));
}
template <typename U>
__device__ __forceinline__ U gelu_tanh_bwd(U dy, U x) {
  const U x_sq = x * x;
  const U inner = (U)kBeta * (x + (U)kKappa * (x_sq * x));
  const U t = tanh(inner);
  const U left = (U)0.5 * x;
  const U right = (U)1 + t;
  const U left_d = (U)0.5 * right;
  const U tanh_d = (U)1 - t * t;
  const U inner_d = (U)kBeta * ((U)1 + (U)3 * (U)kKappa * x_sq);
  return dy * (left_d + left * tanh_d * inner_d);
}
template <>
__device__ __forceinline__ float gelu_tanh_bwd<float>(float dy, float x) {
  const float x_sq = x * x;
  const float inner = (float)kBeta * (x + (float)kKappa * (x_sq * x));
  const float t = tanhf(inner);
  const float left = 0.5f * x;
  const float right = 1.0f + t;
  const float left_d = 0.5f * right;
  const float tanh_d = 1.0f - t * t;
  const float inner_d = (float)kBeta * (1.0f + 3.0f * (float)kKappa * x_sq);
  return dy * (left_d + left * tanh_d * inner_d);
}

// ------------------------------------------------- fast forms (16-bit data)
// s = 0.5 * (1 + tanh(u)) = 1 / (1 + 2^(x * (A + B x^2))),
// A = -2 kBeta log2(e), B = A kKappa.
__device__ __forceinline__ float tanh_gate(float x, float x_sq) {
  constexpr float A = (float)(-2.0 * kBeta * kLog2e);
  constexpr float B = (float)(-2.0 * kBeta * kLog2e * kKappa);
  const float e = __builtin_amdgcn_exp2f(x * (A + B * x_sq));
  return __builtin_amdgcn_rcpf(1.0f + e);
}
__device__ __forceinline__ float gelu_tanh_fwd_fast(float x) {
  return x * tanh_gate(x, x * x);
}
__device__ __forceinline__ float gelu_tanh_bwd_fast(float dy, float x) {
  // with s as above: 1 + t = 2s, 1 - t^2 = 4 s (1 - s), so
  // d/dx = s * (1 + 2 x (1 - s) kBeta (1 + 3 kKappa x^2))
  constexpr float C0 = (float)(2.0 * kBeta);
  constexpr float C1 = (float)(6.0 * kBeta * kKappa);
  // beyond |x| = 12 the derivative is 1 or 0 to the last bit already; evaluating it at the
  // clamped point keeps x^3 from overflowing into 0 * inf for |x| > 7e12.  A NaN input stays NaN.
  const float xc = __builtin_fminf(__builtin_fmaxf(x, -12.0f), 12.0f);
  const float x_sq = xc * xc;
  const float s = tanh_gate(xc, x_sq);
  const float inner_d2 = C0 + C1 * x_sq;
  const float d = s * (1.0f + xc * (1.0f - s) * inner_d2);
  return dy * (x != x ? x : d);
}

// Exact (erf) form for 16-bit data.  libm's erff costs more VALU time than the memory
// traffic of a 16-bit element, so the normal CDF is formed from the complementary error
// function in the Abramowitz-Stegun 7.1.26 shape
//   erfc(z) = t (a1 + t (a2 + t (a3 + t (a4 + t a5)))) exp(-z^2),  t = 1 / (1 + p z),  z >= 0,
// whose error is itself proportional to exp(-z^2): the relative error of erfc stays near
// 1e-6 over the whole range, so Phi(x) = erfc(-x / sqrt 2) / 2 keeps full relative accuracy in
// the left tail, where 1 + erf(.) cancels.  Far inside the 2^-9 / 2^-11 of a bf16 / f16 result.
struct ErfcParts {
  float half_erfc;  // erfc(|x| / sqrt 2) / 2
  float gauss;      // exp(-x^2 / 2)
};
__device__ __forceinline__ ErfcParts half_erfc_abs(float x) {
  constexpr float P = 0.3275911f * (float)kAlpha;  // p z = p |x| / sqrt 2
  constexpr float A1 = 0.5f * 0.254829592f, A2 = 0.5f * -0.284496736f, A3 = 0.5f * 1.421413741f,
                  A4 = 0.5f * -1.453152027f, A5 = 0.5f * 1.061405429f;
  const float ax = fabsf(x);
  const float t = __builtin_amdgcn_rcpf(1.0f + P * ax);
  const float poly = t * (A1 + t * (A2 + t * (A3 + t * (A4 + t * A5))));
  ErfcParts r;
  r.gauss = __builtin_amdgcn_exp2f(x * x * (float)(-0.5 * kLog2e));
  r.half_erfc = poly * r.gauss;
  return r;
}
__device__ __forceinline__ float gelu_erf_fwd_fast(float x) {
  const ErfcParts e = half_erfc_abs(x);
  const float cdf = x < 0.f ? e.half_erfc : 1.0f - e.half_erfc;
  return x * cdf;
}
__device__ __forceinline__ float gelu_erf_bwd_fast(float dy, float x) {
  const ErfcParts e = half_erfc_abs(x);
  const float cdf = x < 0.f ? e.half_erfc : 1.0f - e.half_erfc;
  return dy * (cdf + x * (e.gauss * (float)kPdfScale));
}

template <typename T, int MODE>
__device__ __forceinline__ typename Acc<T>::type fwd_one(typename Acc<T>::type x) {
  if constexpr (MODE == CS_GELU_TANH) {
    if constexpr (sizeof(T) == 2) {
      return gelu_tanh_fwd_fast(x);
    } else {
      return gelu_tanh_fwd(x);
    }
  } else {
    if constexpr (sizeof(T) == 2) {
      return gelu_erf_fwd_fast(x);
    } else {
      return gelu_erf_fwd(x);
    }
  }
}
template <typename T, int MODE>
__device__ __forceinline__ typename Acc<T>::type bwd_one(typename Acc<T>::type dy,
                                                         typename Acc<T>::type x) {
  if constexpr (MODE == CS_GELU_TANH) {
    if constexpr (sizeof(T) == 2) {
      return gelu_tanh_bwd_fast(dy, x);
    } else {
      return gelu_tanh_bwd(dy, x);
    }
  } else {
    if constexpr (sizeof(T) == 2) {
      return gelu_erf_bwd_fast(dy, x);
    } else {
      return gelu_erf_bwd(dy, x);
    }
  }
}

constexpr int kThreads = 256;
// 16-byte vectors per lane per chunk, a workgroup apart.  Measured at [8192, 3072] bf16 (forward
// tanh / erf, backward tanh / erf, us): 1 -> 18.7 / 19.5 / 26.7 / 26.6, 2 -> 17.6 / 17.8 / 24.8 / 24.9,
// 3 -> 17.9 / 18.5 / 25.4 / 25.3, 4 -> 18.1 / 19.0 / 25.2 / 25.3; wave-contiguous kilobytes
// changed nothing here.
constexpr int kUnroll = 2;
__device__ __forceinline__ int vec_index(int u, int tid) { return u * kThreads + tid; }

template <typename T>
constexpr int64_t chunk_elems() {
  return (int64_t)kThreads * kUnroll * Vec16<T>::n;
}

template <typename T, int MODE, bool BACKWARD>
__global__ __launch_bounds__(kThreads) void gelu_kernel(const T *__restrict__ dy,
                                                        const T *__restrict__ x,
                                                        T *__restrict__ out, int64_t n,
                                                        bool vec_ok) {
  constexpr int VN = Vec16<T>::n;
  const int64_t begin = (int64_t)blockIdx.x * chunk_elems<T>();
  const int64_t end = begin + chunk_elems<T>() < n ? begin + chunk_elems<T>() : n;
  const int tid = threadIdx.x;
  if (vec_ok && end - begin == chunk_elems<T>()) {
    Vec16<T> vx[kUnroll], vd[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int64_t off = begin + (int64_t)vec_index(u, tid) * VN;
      vx[u] = load16_stream(x + off);
      if constexpr (BACKWARD) vd[u] = load16_stream(dy + off);
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int64_t off = begin + (int64_t)vec_index(u, tid) * VN;
      Vec16<T> r;
#pragma unroll
      for (int k = 0; k < VN; ++k) {
        if constexpr (BACKWARD) {
          r.e[k] = from_acc<T>(bwd_one<T, MODE>(to_acc(vd[u].e[k]), to_acc(vx[u].e[k])));
        } else {
          r.e[k] = from_acc<T>(fwd_one<T, MODE>(to_acc(vx[u].e[k])));
        }
      }
      store16_stream(out + off, r);
    }
    return;
  }
  for (int64_t i = begin + tid; i < end; i += kThreads) {
    if constexpr (BACKWARD) {
      out[i] = from_acc<T>(bwd_one<T, MODE>(to_acc(dy[i]), to_acc(x[i])));
    } else {
      out[i] = from_acc<T>(fwd_one<T, MODE>(to_acc(x[i])));
    }
  }
}

template <typename T, bool BACKWARD>
int launch(const void *dy, const void *x, void *out, int64_t n, int mode, hipStream_t s) {
  const int64_t blocks = ceil_div(n, chunk_elems<T>());
  if (blocks > 0x7fffffffLL) return CS_ERR_TOO_LARGE;
  const bool vec_ok = is_aligned16(x) && is_aligned16(out) && (!BACKWARD || is_aligned16(dy));
  const dim3 grid((unsigned)blocks), block(kThreads);
  if (mode == CS_GELU_TANH) {
    gelu_kernel<T, CS_GELU_TANH, BACKWARD>
        <<<grid, block, 0, s>>>((const T *)dy, (const T *)x, (T *)out, n, vec_ok);
  } else {
    gelu_kernel<T, CS_GELU_ERF, BACKWARD>
        <<<grid, block, 0, s>>>((const T *)dy, (const T *)x, (T *)out, n, vec_ok);
  }
  return launch_status();
}

template <bool BACKWARD>
int dispatch(const void *dy, const void *x, void *out, int64_t n, int dtype, int mode,
             void *stream) {
  if (n < 0 || (mode != CS_GELU_ERF && mode != CS_GELU_TANH)) return CS_ERR_INVALID_ARGUMENT;
  const size_t es = dtype_size(dtype);
  if (es == 0) return CS_ERR_UNSUPPORTED;
  if (n == 0) return CS_OK;
  if (!x || !out || (BACKWARD && !dy)) return CS_ERR_INVALID_ARGUMENT;
  if (!aligned_to(x, es) || !aligned_to(out, es) || (BACKWARD && !aligned_to(dy, es)))
    return CS_ERR_MISALIGNED;
  hipStream_t s = as_stream(stream);
  switch (dtype) {
    case CS_F32: return launch<float, BACKWARD>(dy, x, out, n, mode, s);
    case CS_F64: return launch<double, BACKWARD>(dy, x, out, n, mode, s);
    case CS_F16: return launch<f16_t, BACKWARD>(dy, x, out, n, mode, s);
    case CS_BF16: return launch<bf16_t, BACKWARD>(dy, x, out, n, mode, s);
  }
  return CS_ERR_UNSUPPORTED;
}

}  // namespace
}  // namespace cs_hip

extern "C" int cs_gelu_forward(const void *x, void *y, int64_t n, int dtype, int mode,
                               void *stream) {
  return cs_hip::dispatch<false>(nullptr, x, y, n, dtype, mode, stream);
}

extern "C" int cs_gelu_backward(const void *dy, const void *x, void *dx, int64_t n, int dtype,
                                int mode, void *stream) {
  return cs_hip::dispatch<true>(dy, x, dx, n, dtype, mode, stream);
}
