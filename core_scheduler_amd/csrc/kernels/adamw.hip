// AdamW step kernels for gfx950: a flat single-tensor step and a
// multi-tensor step that updates a whole parameter set in one launch.
//
// Arithmetic follows the reference kernel's operation order
// (src/optimizer/adamw.cu:45-59, amsgrad :72-89): math in float (double for
// double storage), m and v stored back in the storage type while the update
// continues from the unrounded values, bias corrections formed on the host in
// double and narrowed (adamw.cu:116-117).
//
// The op moves 28 B per fp32 parameter (read w, g, m, v; write w, m, v) and
// does ~20 flops, so it is bound by HBM: every lane moves 16 B per access
// (non-temporal: +6% over plain loads here),
// each workgroup owns one contiguous chunk, and nothing is read twice.
#include "common.hpp"

#include <math.h>

#include <cmath>

namespace cs_hip {
namespace {

template <typename U>
struct AdamHyper {
  U lr, beta1, beta2, inv_bc1, inv_bc2, eps, wd;
};

template <typename U>
__device__ __forceinline__ U dev_sqrt(U x);
template <>
__device__ __forceinline__ float dev_sqrt<float>(float x) {
  return sqrtf(x);
}
template <>
__device__ __forceinline__ double dev_sqrt<double>(double x) {
  return sqrt(x);
}

// One element, reference operation order.
// `gscale` is the gradient-clipping coefficient (1 when not clipping).  The scaled gradient
// is rounded to the storage type first, as the reference's in-place clip leaves it
// (src/compute/utils.cpp:733-736); multiplying by 1 changes nothing.
template <typename T, bool AMSGRAD>
__device__ __forceinline__ void adam_update(T &w, T &m, T &v, T &vmax, const T g_in,
                                            const AdamHyper<typename Acc<T>::type> &h,
                                            const typename Acc<T>::type gscale) {
  using U = typename Acc<T>::type;
  const U one = (U)1;
  const U g = round_through<T>(to_acc(g_in) * gscale);
  const U w0 = to_acc(w);
  const U theta = w0 - h.lr * h.wd * w0;
  const U m_t = h.beta1 * to_acc(m) + (one - h.beta1) * g;
  m = from_acc<T>(m_t);
  const U v_t = h.beta2 * to_acc(v) + (one - h.beta2) * g * g;
  v = from_acc<T>(v_t);
  const U m_hat = m_t * h.inv_bc1;
  U v_hat = v_t * h.inv_bc2;
  if constexpr (AMSGRAD) {
    const U vm = to_acc(vmax);
    v_hat = vm > v_hat ? vm : v_hat;
    vmax = from_acc<T>(v_hat);
  }
  w = from_acc<T>(theta - h.lr * m_hat / (dev_sqrt<U>(v_hat) + h.eps));
}

constexpr int kAdamThreads = 256;
// A chunk is what one workgroup updates: kAdamThreads lanes x U 16-byte vectors per array.
// One launch per tensor (cs_adamw_step, the reference's shape): U = 2 with a lane's accesses a
// workgroup apart; of 1, 2, 3, 4, 8 it measured best there (5.97 TB/s at 124M fp32 parameters
// against 5.36 - 5.72), and the many small launches of a model want small chunks.
// One launch for all tensors: U = 4 with every wave owning 4 consecutive kilobytes of each
// array.  The traffic alone (four arrays read, three rewritten) runs 568 us in that shape
// against 612 us in the other at 124M floats per array; the step gains 3% (620 -> 602 us,
// 7.96 -> 7.74 ms for 1.56G parameters).
constexpr int kAdamFlatUnroll = 2;
#ifndef CS_ADAM_MULTI_UNROLL
#define CS_ADAM_MULTI_UNROLL 4
#endif
constexpr int kAdamMultiUnroll = CS_ADAM_MULTI_UNROLL;

// Vector index inside a chunk for a lane's u-th access.
template <int U, bool WAVE_CONTIG>
__device__ __forceinline__ int adam_vec_index(int u, int tid) {
  if constexpr (WAVE_CONTIG) {
    return (tid >> 6) * (kWave * U) + u * kWave + (tid & (kWave - 1));
  } else {
    return u * kAdamThreads + tid;
  }
}

template <typename T, int U>
constexpr int64_t adam_chunk_elems() {
  return (int64_t)kAdamThreads * U * Vec16<T>::n;
}

// Updates elements [begin, end) of one tensor with this workgroup.  `vec_ok`
// says all five pointers are 16-byte aligned at element 0.
template <typename T, bool AMSGRAD, int U_, bool WAVE_CONTIG>
__device__ __forceinline__ void adam_chunk(T *__restrict__ w, const T *__restrict__ dw,
                                           T *__restrict__ m, T *__restrict__ v,
                                           T *__restrict__ vmax, int64_t begin, int64_t end,
                                           bool vec_ok,
                                           const AdamHyper<typename Acc<T>::type> &h,
                                           const typename Acc<T>::type gscale) {
  constexpr int VN = Vec16<T>::n;
  const int tid = threadIdx.x;
  if (vec_ok && end - begin == adam_chunk_elems<T, U_>()) {
    // full chunk: issue every load before the first use
    Vec16<T> vw[U_], vg[U_], vm[U_], vv[U_], vx[U_];
#pragma unroll
    for (int u = 0; u < U_; ++u) {
      const int64_t off = begin + (int64_t)adam_vec_index<U_, WAVE_CONTIG>(u, tid) * VN;
      vg[u] = load16_stream(dw + off);
      vw[u] = load16_stream(w + off);
      vm[u] = load16_stream(m + off);
      vv[u] = load16_stream(v + off);
      if constexpr (AMSGRAD) vx[u] = load16_stream(vmax + off);
    }
#pragma unroll
    for (int u = 0; u < U_; ++u) {
      const int64_t off = begin + (int64_t)adam_vec_index<U_, WAVE_CONTIG>(u, tid) * VN;
#pragma unroll
      for (int k = 0; k < VN; ++k) {
        adam_update<T, AMSGRAD>(vw[u].e[k], vm[u].e[k], vv[u].e[k], vx[u].e[k], vg[u].e[k], h, gscale);
      }
      store16_stream(w + off, vw[u]);
      store16_stream(m + off, vm[u]);
      store16_stream(v + off, vv[u]);
      if constexpr (AMSGRAD) store16_stream(vmax + off, vx[u]);
    }
    return;
  }
  // ragged chunk (tensor tail, small tensors, or unaligned pointers)
  for (int64_t i = begin + tid; i < end; i += kAdamThreads) {
    T wi = w[i], mi = m[i], vi = v[i], xi{};
    if constexpr (AMSGRAD) xi = vmax[i];
    adam_update<T, AMSGRAD>(wi, mi, vi, xi, dw[i], h, gscale);
    w[i] = wi;
    m[i] = mi;
    v[i] = vi;
    if constexpr (AMSGRAD) vmax[i] = xi;
  }
}

template <typename T, bool AMSGRAD>
__global__ __launch_bounds__(kAdamThreads) void adamw_flat_kernel(
    T *__restrict__ w, const T *__restrict__ dw, T *__restrict__ m, T *__restrict__ v,
    T *__restrict__ vmax, int64_t n, bool vec_ok, AdamHyper<typename Acc<T>::type> h) {
  const int64_t chunk = adam_chunk_elems<T, kAdamFlatUnroll>();
  const int64_t begin = (int64_t)blockIdx.x * chunk;
  const int64_t end = begin + chunk < n ? begin + chunk : n;
  adam_chunk<T, AMSGRAD, kAdamFlatUnroll, false>(w, dw, m, v, vmax, begin, end, vec_ok, h,
                                                 (typename Acc<T>::type)1);
}

// ---------------------------------------------------------- multi-tensor
// Device table: int64 first_slot[n_tensors + 1] (padded to a multiple of 8
// entries), then one DevTensor per tensor.  Workgroup slot s belongs to the
// tensor i with first_slot[i] <= s < first_slot[i+1] and updates that
// tensor's chunk number s - first_slot[i].
struct DevTensor {
  void *w;
  const void *dw;
  void *m;
  void *v;
  void *vmax;
  int64_t n;
  int64_t vec_ok;
  int64_t pad;
};
static_assert(sizeof(DevTensor) == 64, "table layout");

__host__ __device__ inline int64_t slot_array_len(int64_t n_tensors) {
  return (n_tensors + 1 + 7) / 8 * 8;
}

// The tensor that owns workgroup slot `slot`: binary search over the prefix array;
// wave-uniform, so it runs on the scalar unit out of the constant cache.
__device__ __forceinline__ int tensor_of_slot(const int64_t *__restrict__ table, int n_tensors,
                                              int64_t slot) {
  int lo = 0, hi = n_tensors;  // invariant: first_slot[lo] <= slot < first_slot[hi]
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (table[mid] <= slot) {
      lo = mid;
    } else {
      hi = mid;
    }
  }
  return lo;
}

// `clip` points at the clipping coefficient in device memory (written by the norm launches
// that precede this one on the stream), or is null.
template <typename T, bool AMSGRAD>
__global__ __launch_bounds__(kAdamThreads) void adamw_multi_kernel(
    const int64_t *__restrict__ table, int n_tensors, AdamHyper<typename Acc<T>::type> h,
    const float *__restrict__ clip) {
  using U = typename Acc<T>::type;
  const int64_t slot = blockIdx.x;
  const int lo = tensor_of_slot(table, n_tensors, slot);
  const DevTensor *desc =
      reinterpret_cast<const DevTensor *>(table + slot_array_len(n_tensors)) + lo;
  const int64_t chunk = adam_chunk_elems<T, kAdamMultiUnroll>();
  const int64_t begin = (slot - table[lo]) * chunk;
  const int64_t n = desc->n;
  const int64_t end = begin + chunk < n ? begin + chunk : n;
  const U gscale = clip ? (U)*clip : (U)1;
  adam_chunk<T, AMSGRAD, kAdamMultiUnroll, true>(
      static_cast<T *>(desc->w), static_cast<const T *>(desc->dw), static_cast<T *>(desc->m),
      static_cast<T *>(desc->v), static_cast<T *>(desc->vmax), begin, end, desc->vec_ok != 0, h, gscale);
}

// ------------------------------------------------- global gradient norm
// Utils::clip_grad_norm_ (src/compute/utils.cpp:700-746): total = ||all gradients||_p,
// coefficient = min(1, max_norm / (total + 1e-6)), gradients *= coefficient.
// Pass 1 walks the same table as the step: each workgroup reduces its chunk of one
// gradient to a partial (sum of squares, or largest magnitude for the infinity norm).
// Pass 2 adds the partials in slot order in double, so the result does not depend on
// scheduling, and writes the norm and the coefficient.
template <typename T, bool INF>
__global__ __launch_bounds__(kAdamThreads) void grad_norm_partial_kernel(
    const int64_t *__restrict__ table, int n_tensors, float *__restrict__ partial) {
  constexpr int VN = Vec16<T>::n;
  const int64_t slot = blockIdx.x;
  const int lo = tensor_of_slot(table, n_tensors, slot);
  const DevTensor *desc =
      reinterpret_cast<const DevTensor *>(table + slot_array_len(n_tensors)) + lo;
  const T *g = static_cast<const T *>(desc->dw);
  const int64_t chunk = adam_chunk_elems<T, kAdamMultiUnroll>();
  const int64_t begin = (slot - table[lo]) * chunk;
  const int64_t n = desc->n;
  const int64_t end = begin + chunk < n ? begin + chunk : n;
  const int tid = threadIdx.x;
  float acc = 0.f;
  auto take = [&](const T x) {
    const float f = (float)to_acc(x);
    if constexpr (INF) {
      acc = fmaxf(acc, fabsf(f));
    } else {
      acc += f * f;
    }
  };
  if (is_aligned16(g) && end - begin == chunk) {
    Vec16<T> v[kAdamMultiUnroll];
#pragma unroll
    for (int u = 0; u < kAdamMultiUnroll; ++u)
      v[u] = load16(g + begin + (int64_t)adam_vec_index<kAdamMultiUnroll, true>(u, tid) * VN);  // read again by the step: keep it cached
#pragma unroll
    for (int u = 0; u < kAdamMultiUnroll; ++u)
#pragma unroll
      for (int k = 0; k < VN; ++k) take(v[u].e[k]);
  } else {
    for (int64_t i = begin + tid; i < end; i += kAdamThreads) take(g[i]);
  }
  __shared__ float scratch[kAdamThreads / kWave];
  float total;
  if constexpr (INF) {
    total = block_reduce(acc, MaxOp{}, 0.f, scratch);
  } else {
    total = block_reduce(acc, SumOp{}, 0.f, scratch);
  }
  if (tid == 0) partial[slot] = total;
}

template <bool INF>
__global__ __launch_bounds__(1024) void grad_norm_final_kernel(const float *__restrict__ partial,
                                                               int64_t n_slots, float max_norm,
                                                               float *__restrict__ total_norm,
                                                               float *__restrict__ clip) {
  __shared__ double scratch[1024 / kWave];
  const int tid = threadIdx.x;
  // thread t adds slots t, t + 1024, ... (coalesced reads) into four interleaved sums, so four
  // loads are in flight; the order is fixed, whatever the scheduling
  double a4[4] = {0., 0., 0., 0.};
  int64_t i = tid;
  for (; i + 3 * 1024 < n_slots; i += 4 * 1024) {
    const float p0 = partial[i], p1 = partial[i + 1024], p2 = partial[i + 2048], p3 = partial[i + 3072];
    const float p[4] = {p0, p1, p2, p3};
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if constexpr (INF) {
        a4[u] = (double)p[u] > a4[u] ? (double)p[u] : a4[u];
      } else {
        a4[u] += (double)p[u];
      }
    }
  }
  for (; i < n_slots; i += 1024) {
    const double p = (double)partial[i];
    if constexpr (INF) {
      a4[0] = p > a4[0] ? p : a4[0];
    } else {
      a4[0] += p;
    }
  }
  double acc;
  if constexpr (INF) {
    const double m01 = a4[0] > a4[1] ? a4[0] : a4[1], m23 = a4[2] > a4[3] ? a4[2] : a4[3];
    acc = m01 > m23 ? m01 : m23;
  } else {
    acc = (a4[0] + a4[1]) + (a4[2] + a4[3]);
  }
  double total;
  if constexpr (INF) {
    total = block_reduce(acc, MaxOp{}, 0., scratch);
  } else {
    total = block_reduce(acc, SumOp{}, 0., scratch);
  }
  if (tid == 0) {
    const float norm = INF ? (float)total : (float)sqrt(total);
    *total_norm = norm;
    // in float, as the reference's tensor ops are: max_norm / (norm + 1e-6), clamped to 1
    const float coef = max_norm / (norm + 1e-6f);
    *clip = coef < 1.0f ? coef : 1.0f;
  }
}

// gradients *= coefficient, in place (what the reference's clip leaves behind)
template <typename T>
__global__ __launch_bounds__(kAdamThreads) void grad_scale_kernel(const int64_t *__restrict__ table,
                                                                  int n_tensors,
                                                                  const float *__restrict__ clip) {
  using U = typename Acc<T>::type;
  constexpr int VN = Vec16<T>::n;
  const int64_t slot = blockIdx.x;
  const int lo = tensor_of_slot(table, n_tensors, slot);
  const DevTensor *desc =
      reinterpret_cast<const DevTensor *>(table + slot_array_len(n_tensors)) + lo;
  T *g = static_cast<T *>(const_cast<void *>(desc->dw));
  const int64_t chunk = adam_chunk_elems<T, kAdamMultiUnroll>();
  const int64_t begin = (slot - table[lo]) * chunk;
  const int64_t n = desc->n;
  const int64_t end = begin + chunk < n ? begin + chunk : n;
  const int tid = threadIdx.x;
  const U scale = (U)*clip;
  if (is_aligned16(g) && end - begin == chunk) {
#pragma unroll
    for (int u = 0; u < kAdamMultiUnroll; ++u) {
      T *p = g + begin + (int64_t)adam_vec_index<kAdamMultiUnroll, true>(u, tid) * VN;
      Vec16<T> v = load16(p);
#pragma unroll
      for (int k = 0; k < VN; ++k) v.e[k] = from_acc<T>(to_acc(v.e[k]) * scale);
      store16(p, v);
    }
  } else {
    for (int64_t i = begin + tid; i < end; i += kAdamThreads) g[i] = from_acc<T>(to_acc(g[i]) * scale);
  }
}

template <typename U>
AdamHyper<U> make_hyper(double lr, double beta1, double beta2, double eps, double wd, int64_t t) {
  AdamHyper<U> h;
  h.lr = (U)lr;
  h.beta1 = (U)beta1;
  h.beta2 = (U)beta2;
  // host double, then narrowed: adamw.cu:116-117
  h.inv_bc1 = (U)(1. / (1. - pow(beta1, (double)t)));
  h.inv_bc2 = (U)(1. / (1. - pow(beta2, (double)t)));
  h.eps = (U)eps;
  h.wd = (U)wd;
  return h;
}

// workgroup slots a tensor of n elements takes in the multi-tensor table
template <typename T>
int64_t chunks_for(int64_t n) {
  return ceil_div(n, adam_chunk_elems<T, kAdamMultiUnroll>());
}

int64_t chunks_for_dtype(int dtype, int64_t n) {
  switch (dtype) {
    case CS_F32: return chunks_for<float>(n);
    case CS_F64: return chunks_for<double>(n);
    case CS_F16: return chunks_for<f16_t>(n);
    case CS_BF16: return chunks_for<bf16_t>(n);
    default: return -1;
  }
}

template <typename T>
int launch_flat(void *w, const void *dw, void *m, void *v, void *vmax, int64_t n, double lr,
                double beta1, double beta2, double eps, double wd, int64_t t, hipStream_t s) {
  using U = typename Acc<T>::type;
  const int64_t blocks = ceil_div(n, adam_chunk_elems<T, kAdamFlatUnroll>());
  if (blocks > 0x7fffffffLL) return CS_ERR_TOO_LARGE;
  const bool vec_ok = is_aligned16(w) && is_aligned16(dw) && is_aligned16(m) && is_aligned16(v) &&
                      (vmax == nullptr || is_aligned16(vmax));
  const AdamHyper<U> h = make_hyper<U>(lr, beta1, beta2, eps, wd, t);
  if (vmax) {
    adamw_flat_kernel<T, true><<<dim3((unsigned)blocks), dim3(kAdamThreads), 0, s>>>(
        (T *)w, (const T *)dw, (T *)m, (T *)v, (T *)vmax, n, vec_ok, h);
  } else {
    adamw_flat_kernel<T, false><<<dim3((unsigned)blocks), dim3(kAdamThreads), 0, s>>>(
        (T *)w, (const T *)dw, (T *)m, (T *)v, nullptr, n, vec_ok, h);
  }
  return launch_status();
}

template <typename T>
int launch_multi(const void *table, int64_t n_tensors, int64_t n_slots, int amsgrad, double lr,
                 double beta1, double beta2, double eps, double wd, int64_t t, const float *clip,
                 hipStream_t s) {
  using U = typename Acc<T>::type;
  const AdamHyper<U> h = make_hyper<U>(lr, beta1, beta2, eps, wd, t);
  const int64_t *tab = static_cast<const int64_t *>(table);
  if (amsgrad) {
    adamw_multi_kernel<T, true>
        <<<dim3((unsigned)n_slots), dim3(kAdamThreads), 0, s>>>(tab, (int)n_tensors, h, clip);
  } else {
    adamw_multi_kernel<T, false>
        <<<dim3((unsigned)n_slots), dim3(kAdamThreads), 0, s>>>(tab, (int)n_tensors, h, clip);
  }
  return launch_status();
}

}  // namespace
}  // namespace cs_hip

using namespace cs_hip;

extern "C" int cs_adamw_step(void *w, const void *dw, void *m, void *v, void *v_max, int64_t n,
                             int dtype, double lr, double beta1, double beta2, double eps,
                             double weight_decay, int64_t t, void *stream) {
  if (n < 0) return CS_ERR_INVALID_ARGUMENT;
  const size_t es = dtype_size(dtype);
  if (es == 0) return CS_ERR_UNSUPPORTED;
  if (n == 0) return CS_OK;
  if (!w || !dw || !m || !v) return CS_ERR_INVALID_ARGUMENT;
  if (!aligned_to(w, es) || !aligned_to(dw, es) || !aligned_to(m, es) || !aligned_to(v, es) ||
      (v_max && !aligned_to(v_max, es)))
    return CS_ERR_MISALIGNED;
  hipStream_t s = as_stream(stream);
  switch (dtype) {
    case CS_F32:
      return launch_flat<float>(w, dw, m, v, v_max, n, lr, beta1, beta2, eps, weight_decay, t, s);
    case CS_F64:
      return launch_flat<double>(w, dw, m, v, v_max, n, lr, beta1, beta2, eps, weight_decay, t, s);
    case CS_F16:
      return launch_flat<f16_t>(w, dw, m, v, v_max, n, lr, beta1, beta2, eps, weight_decay, t, s);
    case CS_BF16:
      return launch_flat<bf16_t>(w, dw, m, v, v_max, n, lr, beta1, beta2, eps, weight_decay, t, s);
  }
  return CS_ERR_UNSUPPORTED;
}

extern "C" size_t cs_adamw_multi_table_bytes(int64_t n_tensors) {
  if (n_tensors <= 0) return 0;
  return (size_t)slot_array_len(n_tensors) * sizeof(int64_t) +
         (size_t)n_tensors * sizeof(DevTensor);
}

// The chunk size depends on the element type, so a table is built for one
// dtype and must be used with the same dtype in cs_adamw_multi_step.
extern "C" int cs_adamw_multi_build_table(const cs_adamw_tensor *tensors, int64_t n_tensors,
                                          int dtype, void *host_table, size_t table_bytes,
                                          int64_t *n_slots) {
  if (!tensors || !host_table || !n_slots || n_tensors <= 0) return CS_ERR_INVALID_ARGUMENT;
  const size_t es = dtype_size(dtype);
  if (es == 0) return CS_ERR_UNSUPPORTED;
  if (table_bytes < cs_adamw_multi_table_bytes(n_tensors)) return CS_ERR_WORKSPACE;
  int64_t *first_slot = static_cast<int64_t *>(host_table);
  DevTensor *desc = reinterpret_cast<DevTensor *>(first_slot + slot_array_len(n_tensors));
  int64_t slots = 0;
  for (int64_t i = 0; i < n_tensors; ++i) {
    const cs_adamw_tensor &t = tensors[i];
    if (t.n < 0) return CS_ERR_INVALID_ARGUMENT;
    if (t.n > 0) {
      if (!t.w || !t.dw || !t.m || !t.v) return CS_ERR_INVALID_ARGUMENT;
      if (!aligned_to(t.w, es) || !aligned_to(t.dw, es) || !aligned_to(t.m, es) ||
          !aligned_to(t.v, es) || (t.v_max && !aligned_to(t.v_max, es)))
        return CS_ERR_MISALIGNED;
    }
    first_slot[i] = slots;
    desc[i].w = t.w;
    desc[i].dw = t.dw;
    desc[i].m = t.m;
    desc[i].v = t.v;
    desc[i].vmax = t.v_max;
    desc[i].n = t.n;
    desc[i].vec_ok = is_aligned16(t.w) && is_aligned16(t.dw) && is_aligned16(t.m) &&
                     is_aligned16(t.v) && (t.v_max == nullptr || is_aligned16(t.v_max));
    desc[i].pad = 0;
    slots += chunks_for_dtype(dtype, t.n);
  }
  for (int64_t i = n_tensors; i < slot_array_len(n_tensors); ++i) first_slot[i] = slots;
  if (slots > 0x7fffffffLL) return CS_ERR_TOO_LARGE;
  *n_slots = slots;
  return CS_OK;
}

namespace {
int multi_step(const void *device_table, int64_t n_tensors, int64_t n_slots, int dtype, int amsgrad,
               double lr, double beta1, double beta2, double eps, double weight_decay, int64_t t,
               const float *clip, void *stream) {
  if (n_tensors < 0 || n_slots < 0) return CS_ERR_INVALID_ARGUMENT;
  if (n_tensors == 0 || n_slots == 0) return CS_OK;
  if (!device_table || !aligned_to(device_table, 16)) return CS_ERR_INVALID_ARGUMENT;
  if (n_slots > 0x7fffffffLL || n_tensors > 0x7fffffffLL) return CS_ERR_TOO_LARGE;
  hipStream_t s = as_stream(stream);
  switch (dtype) {
    case CS_F32:
      return launch_multi<float>(device_table, n_tensors, n_slots, amsgrad, lr, beta1, beta2, eps,
                                 weight_decay, t, clip, s);
    case CS_F64:
      return launch_multi<double>(device_table, n_tensors, n_slots, amsgrad, lr, beta1, beta2, eps,
                                  weight_decay, t, clip, s);
    case CS_F16:
      return launch_multi<f16_t>(device_table, n_tensors, n_slots, amsgrad, lr, beta1, beta2, eps,
                                 weight_decay, t, clip, s);
    case CS_BF16:
      return launch_multi<bf16_t>(device_table, n_tensors, n_slots, amsgrad, lr, beta1, beta2, eps,
                                  weight_decay, t, clip, s);
  }
  return CS_ERR_UNSUPPORTED;
}

template <typename T>
int launch_norm(const void *table, int64_t n_tensors, int64_t n_slots, bool inf, float max_norm,
                float *partial, float *total_norm, float *clip, hipStream_t s) {
  const int64_t *tab = static_cast<const int64_t *>(table);
  const dim3 grid((unsigned)n_slots), block(kAdamThreads);
  if (inf) {
    grad_norm_partial_kernel<T, true><<<grid, block, 0, s>>>(tab, (int)n_tensors, partial);
    grad_norm_final_kernel<true><<<dim3(1), dim3(1024), 0, s>>>(partial, n_slots, max_norm, total_norm, clip);
  } else {
    grad_norm_partial_kernel<T, false><<<grid, block, 0, s>>>(tab, (int)n_tensors, partial);
    grad_norm_final_kernel<false><<<dim3(1), dim3(1024), 0, s>>>(partial, n_slots, max_norm, total_norm, clip);
  }
  return launch_status();
}
}  // namespace

extern "C" int cs_adamw_multi_step(const void *device_table, int64_t n_tensors, int64_t n_slots,
                                   int dtype, int amsgrad, double lr, double beta1, double beta2,
                                   double eps, double weight_decay, int64_t t, void *stream) {
  return multi_step(device_table, n_tensors, n_slots, dtype, amsgrad, lr, beta1, beta2, eps,
                    weight_decay, t, nullptr, stream);
}

extern "C" int cs_adamw_multi_step_clipped(const void *device_table, int64_t n_tensors,
                                           int64_t n_slots, int dtype, int amsgrad, double lr,
                                           double beta1, double beta2, double eps,
                                           double weight_decay, int64_t t, const float *clip_coef,
                                           void *stream) {
  if (!clip_coef || !aligned_to(clip_coef, 4)) return CS_ERR_INVALID_ARGUMENT;
  return multi_step(device_table, n_tensors, n_slots, dtype, amsgrad, lr, beta1, beta2, eps,
                    weight_decay, t, clip_coef, stream);
}

extern "C" size_t cs_grad_norm_multi_workspace_bytes(int64_t n_slots) {
  if (n_slots <= 0) return 0;
  return ((size_t)n_slots * sizeof(float) + 255) / 256 * 256;
}

extern "C" int cs_grad_norm_multi(const void *device_table, int64_t n_tensors, int64_t n_slots,
                                  int dtype, double norm_type, double max_norm, void *workspace,
                                  size_t workspace_bytes, float *total_norm, float *clip_coef,
                                  void *stream) {
  if (n_tensors <= 0 || n_slots <= 0) return CS_ERR_INVALID_ARGUMENT;
  const bool inf = std::isinf(norm_type) && norm_type > 0;
  if (!inf && norm_type != 2.0) return CS_ERR_UNSUPPORTED;
  if (!device_table || !aligned_to(device_table, 16) || !total_norm || !clip_coef ||
      !aligned_to(total_norm, 4) || !aligned_to(clip_coef, 4))
    return CS_ERR_INVALID_ARGUMENT;
  if (n_slots > 0x7fffffffLL || n_tensors > 0x7fffffffLL) return CS_ERR_TOO_LARGE;
  if (!workspace || workspace_bytes < cs_grad_norm_multi_workspace_bytes(n_slots) ||
      !aligned_to(workspace, 16))
    return CS_ERR_WORKSPACE;
  hipStream_t s = as_stream(stream);
  float *partial = static_cast<float *>(workspace);
  const float mx = (float)max_norm;
  switch (dtype) {
    case CS_F32:
      return launch_norm<float>(device_table, n_tensors, n_slots, inf, mx, partial, total_norm, clip_coef, s);
    case CS_F64:
      return launch_norm<double>(device_table, n_tensors, n_slots, inf, mx, partial, total_norm, clip_coef, s);
    case CS_F16:
      return launch_norm<f16_t>(device_table, n_tensors, n_slots, inf, mx, partial, total_norm, clip_coef, s);
    case CS_BF16:
      return launch_norm<bf16_t>(device_table, n_tensors, n_slots, inf, mx, partial, total_norm, clip_coef, s);
  }
  return CS_ERR_UNSUPPORTED;
}

extern "C" int cs_grad_scale_multi(const void *device_table, int64_t n_tensors, int64_t n_slots,
                                   int dtype, const float *clip_coef, void *stream) {
  if (n_tensors <= 0 || n_slots <= 0) return CS_ERR_INVALID_ARGUMENT;
  if (!device_table || !aligned_to(device_table, 16) || !clip_coef || !aligned_to(clip_coef, 4))
    return CS_ERR_INVALID_ARGUMENT;
  if (n_slots > 0x7fffffffLL || n_tensors > 0x7fffffffLL) return CS_ERR_TOO_LARGE;
  hipStream_t s = as_stream(stream);
  const int64_t *tab = static_cast<const int64_t *>(device_table);
  const dim3 grid((unsigned)n_slots), block(kAdamThreads);
  switch (dtype) {
    case CS_F32: grad_scale_kernel<float><<<grid, block, 0, s>>>(tab, (int)n_tensors, clip_coef); break;
    case CS_F64: grad_scale_kernel<double><<<grid, block, 0, s>>>(tab, (int)n_tensors, clip_coef); break;
    case CS_F16: grad_scale_kernel<f16_t><<<grid, block, 0, s>>>(tab, (int)n_tensors, clip_coef); break;
    case CS_BF16: grad_scale_kernel<bf16_t><<<grid, block, 0, s>>>(tab, (int)n_tensors, clip_coef); break;
    default: return CS_ERR_UNSUPPORTED;
  }
  return launch_status();
}
