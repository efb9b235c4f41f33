// Fused classifier for gfx950: row softmax + cross-entropy loss + dlogits in
// one pass over the logits.
//
// Replaces at::log_softmax + at::nll_loss_forward
// (src/compute/cross_entropy.cpp:57-63) and at::nll_loss_backward +
// at::_log_softmax_backward_data (:103-109), which between them make about
// five passes over [N, V] and keep three [N, V] temporaries:
//   loss_i    = logsumexp(x_i) - x_i[t_i]            (0 for ignored rows)
//   loss      = sum_i loss_i / #{not ignored}        (MEAN)  |  sum_i loss_i (SUM)
//   dlogits_i = (softmax(x_i) - onehot(t_i)) * s,    s = dloss / #{not ignored} (MEAN) | dloss
//
// A row is read from HBM once and its gradient written once: 2 accesses per
// element.  Which kernel does that depends on the row's width:
//   up to 2048 vectors of 16 bytes   ce_rows_kernel: one workgroup per row, the row in
//                                    registers, exact two-step max and sum (wave64
//                                    butterfly, then LDS across the waves)
//   up to 7168 (8192 at fp32)        ce_rows_stream_kernel: one persistent workgroup per
//                                    CU that loads the next row while it works on the
//                                    current one (50257 bf16 = 6283 vectors = 7 per lane)
//   wider, or rows that do not       ce_rows_wide_kernel: two sweeps over the row, the
//   start on 16-byte boundaries      second one served by the cache
//   fp64, unaligned base pointers    ce_rows_general_kernel
// Probabilities are 2^(x*log2e - max*log2e) / sum with one fma and one hardware exp2 per
// element; the row loss is ln(sum) - (x_t - max).
#include "common.hpp"

#include <math.h>

#include <atomic>
#include <type_traits>

namespace cs_hip {
namespace {

constexpr float kLog2e = 1.44269504088896340736f;
constexpr float kLn2 = 0.69314718055994530942f;

// workspace: [0] int32 count of rows not ignored, [1] float the same number,
// then (from byte 256) N floats of row loss when the caller keeps none.
constexpr size_t kWsHeader = 256;

__device__ __forceinline__ bool target_counts(int64_t t, int64_t V, int64_t ignore_index) {
  return t != ignore_index && t >= 0 && t < V;
}

// Both one-workgroup kernels below keep kSmallInFlight loads per lane in flight: with one load
// at a time a quarter of a million rows took 75 us each.
constexpr int kSmallInFlight = 8;

__global__ __launch_bounds__(1024) void ce_count_kernel(const int64_t *__restrict__ targets,
                                                        int64_t N, int64_t V,
                                                        int64_t ignore_index,
                                                        int *__restrict__ ws_count,
                                                        float *__restrict__ ws_weight,
                                                        const float *__restrict__ class_weight) {
  __shared__ int scratch[16];
  __shared__ float wscratch[16];
  const int tid = threadIdx.x;
  int c = 0;
  float wsum[kSmallInFlight];  // per-class weights of the rows that count: interleaved sums, fixed order
#pragma unroll
  for (int u = 0; u < kSmallInFlight; ++u) wsum[u] = 0.f;
  for (int64_t i0 = tid; i0 < N; i0 += (int64_t)1024 * kSmallInFlight) {
    int64_t t[kSmallInFlight];
#pragma unroll
    for (int u = 0; u < kSmallInFlight; ++u) {
      const int64_t i = i0 + (int64_t)u * 1024;
      t[u] = i < N ? targets[i] : ignore_index;
    }
#pragma unroll
    for (int u = 0; u < kSmallInFlight; ++u) c += target_counts(t[u], V, ignore_index);
    if (class_weight != nullptr) {  // block-uniform
      float w[kSmallInFlight];
#pragma unroll
      for (int u = 0; u < kSmallInFlight; ++u) w[u] = class_weight[target_counts(t[u], V, ignore_index) ? t[u] : 0];
#pragma unroll
      for (int u = 0; u < kSmallInFlight; ++u) wsum[u] += target_counts(t[u], V, ignore_index) ? w[u] : 0.f;
    }
  }
  c = block_reduce(c, SumOp{}, 0, scratch);
  float total = (float)c;  // without class weights every row that counts weighs 1
  if (class_weight != nullptr) {
    float ws_ = 0.f;
#pragma unroll
    for (int u = 0; u < kSmallInFlight; ++u) ws_ += wsum[u];
    total = block_reduce(ws_, SumOp{}, 0.f, wscratch);
  }
  if (tid == 0) {
    *ws_count = c;
    *ws_weight = total;
  }
}

// Fixed-order sum of the row losses: thread t adds rows t, t+1024, ... into kSmallInFlight
// interleaved sums, which are then added in order; the 1024 sub-sums are folded by the
// butterfly.  Independent of scheduling.
__global__ __launch_bounds__(1024) void ce_reduce_kernel(const float *__restrict__ row_loss,
                                                         int64_t N, const int *__restrict__ ws_count,
                                                         int reduction, float *__restrict__ loss,
                                                         float *__restrict__ total_weight) {
  __shared__ float scratch[16];
  const int tid = threadIdx.x;
  float part[kSmallInFlight];
#pragma unroll
  for (int u = 0; u < kSmallInFlight; ++u) part[u] = 0.f;
  for (int64_t i0 = tid; i0 < N; i0 += (int64_t)1024 * kSmallInFlight) {
    float v[kSmallInFlight];
#pragma unroll
    for (int u = 0; u < kSmallInFlight; ++u) {
      const int64_t i = i0 + (int64_t)u * 1024;
      v[u] = i < N ? row_loss[i] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < kSmallInFlight; ++u) part[u] += v[u];
  }
  float s = 0.f;
#pragma unroll
  for (int u = 0; u < kSmallInFlight; ++u) s += part[u];
  s = block_reduce(s, SumOp{}, 0.f, scratch);
  if (tid == 0) {
    // the float next to the count: the number of rows that count, or the sum of their class weights
    const float total = reinterpret_cast<const float *>(ws_count)[1];
    if (loss) *loss = reduction == CS_REDUCTION_MEAN ? s / total : s;
    if (total_weight) *total_weight = total;
  }
}

template <typename T>
__device__ __forceinline__ float vec_get(const Vec16<T> &v, int k) {
  return to_acc(v.e[k]);
}

// TD is the dlogits storage: T, or float when the caller wants fp32 gradients
// for 16-bit logits.
template <typename T, typename TD, int N_ELEMS>
__device__ __forceinline__ void store_out(TD *p, const float (&o)[N_ELEMS]) {
  constexpr int DN = Vec16<TD>::n;
#pragma unroll
  for (int q = 0; q < N_ELEMS / DN; ++q) {
    Vec16<TD> v;
#pragma unroll
    for (int k = 0; k < DN; ++k) v.e[k] = from_acc<TD>(o[q * DN + k]);
    store16_stream(p + q * DN, v);
  }
}

template <typename T, typename TD, int BLOCK, int VPT>
__global__ __launch_bounds__(BLOCK) void ce_rows_kernel(
    const T *__restrict__ logits, TD *__restrict__ dlogits, const int64_t *__restrict__ targets,
    float *__restrict__ row_loss, const int *__restrict__ ws_count, int64_t V, int64_t row_stride,
    int64_t ignore_index, int reduction, float dloss) {
  constexpr int VN = Vec16<T>::n;
  __shared__ float scratch[(BLOCK + kWave - 1) / kWave];
  const int64_t row = blockIdx.x;
  const int tid = threadIdx.x;
  const int nvec = (int)(row_stride / VN);  // whole row incl. padding, in vectors
  const int iV = (int)V;
  const T *x = logits + row * row_stride;
  const int64_t target = targets[row];
  const bool counts = target_counts(target, V, ignore_index);  // block-uniform

  if (!counts) {
    if (tid == 0 && row_loss) row_loss[row] = 0.f;
    if (dlogits) {
      float z[VN];
#pragma unroll
      for (int k = 0; k < VN; ++k) z[k] = 0.f;
      for (int idx = tid; idx < nvec; idx += BLOCK)
        store_out<T, TD, VN>(dlogits + row * row_stride + (int64_t)idx * VN, z);
    }
    return;
  }

  Vec16<T> xr[VPT];
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int idx = tid + BLOCK * j;
    // every lane loads (lanes past the row read its last vector, which nothing below uses): a
    // load under the lane's own condition makes the compiler wait for it before the next one
    xr[j] = load16_stream(x + (int64_t)(idx < nvec ? idx : nvec - 1) * VN);
  }
  const float x_t = tid == 0 ? to_acc(x[target]) : 0.f;

  // ---- row maximum
  float m = -INFINITY;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int c0 = (tid + BLOCK * j) * VN;
    if (c0 + VN <= iV) {
#pragma unroll
      for (int k = 0; k < VN; ++k) m = fmaxf(m, vec_get(xr[j], k));
    } else if (c0 < iV) {
#pragma unroll
      for (int k = 0; k < VN; ++k)
        if (c0 + k < iV) m = fmaxf(m, vec_get(xr[j], k));
    }
  }
  m = block_reduce(m, MaxOp{}, -INFINITY, scratch);
  const float m2 = m * kLog2e;

  // ---- sum of exponentials
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int c0 = (tid + BLOCK * j) * VN;
    if (c0 + VN <= iV) {
#pragma unroll
      for (int k = 0; k < VN; ++k) s += __builtin_amdgcn_exp2f(__builtin_fmaf(vec_get(xr[j], k), kLog2e, -m2));
    } else if (c0 < iV) {
#pragma unroll
      for (int k = 0; k < VN; ++k)
        if (c0 + k < iV) s += __builtin_amdgcn_exp2f(__builtin_fmaf(vec_get(xr[j], k), kLog2e, -m2));
    }
  }
  s = block_reduce(s, SumOp{}, 0.f, scratch);

  const float log2_s = __builtin_amdgcn_logf(s);  // v_log_f32 is log2
  // loss = ln(sum exp(x - max)) - (x_t - max): the difference to the maximum is formed with one
  // fused multiply-add against the same rounded m2 the sum used, so a loss near 0 keeps its digits
  if (tid == 0 && row_loss) row_loss[row] = (log2_s - __builtin_fmaf(x_t, kLog2e, -m2)) * kLn2;
  if (dlogits == nullptr) return;

  // ---- dlogits = (p - onehot) * scale with p = 2^(x*log2e - m2) / s.  The exponent is taken
  // relative to the row maximum with one fused multiply-add, the same expression the sum above
  // used, so the rounding of m2 cancels between numerator and denominator and p keeps fp32
  // accuracy; folding log2(s) and log2(scale) into the exponent instead costs ~1e-6 relative,
  // which the subtraction at the target column amplifies when p is close to 1.
  float scale = dloss;
  if (reduction == CS_REDUCTION_MEAN) scale = dloss / (float)(*ws_count);
  const float factor = scale / s;  // s >= 1: the maximum contributes 2^0
  const int t_vec = (int)(target / VN), t_sub = (int)(target % VN);
  TD *d = dlogits + row * row_stride;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int idx = tid + BLOCK * j;
    if (idx < nvec) {
      const int c0 = idx * VN;
      float o[VN];
#pragma unroll
      for (int k = 0; k < VN; ++k)
        o[k] = __builtin_amdgcn_exp2f(__builtin_fmaf(vec_get(xr[j], k), kLog2e, -m2)) * factor;
      if (c0 + VN > iV) {  // last class vector and the padding
#pragma unroll
        for (int k = 0; k < VN; ++k)
          if (c0 + k >= iV) o[k] = 0.f;
      }
      if (idx == t_vec) {
#pragma unroll
        for (int k = 0; k < VN; ++k)
          if (k == t_sub) o[k] -= scale;
      }
      store_out<T, TD, VN>(d + (int64_t)c0, o);
    }
  }
}

// EPV elements of T in one 8- or 16-byte access.  The streaming kernel reads 16-bit logits 8
// bytes per lane when it writes fp32 gradients, so that every store is a full 16 bytes per lane
// and a wave's store covers one contiguous kilobyte (with 16-byte loads each lane would own 32
// output bytes and every store instruction would touch only half of each 64-byte line).
template <typename T, int EPV>
struct alignas(EPV * sizeof(T)) VecE {
  T e[EPV];
};
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
template <typename T, int EPV>
__device__ __forceinline__ VecE<T, EPV> load_e_stream(const T *p) {
  static_assert(EPV * sizeof(T) == 16 || EPV * sizeof(T) == 8, "8- or 16-byte accesses");
  if constexpr (EPV * sizeof(T) == 16) {
    const u32x4 raw = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
    return __builtin_bit_cast(VecE<T, EPV>, raw);
  } else {
    const u32x2 raw = __builtin_nontemporal_load(reinterpret_cast<const u32x2 *>(p));
    return __builtin_bit_cast(VecE<T, EPV>, raw);
  }
}

// Element k of v as fp32.  fp16 is converted straight out of its half of the 32-bit register
// (the sub-dword select of the conversion instruction): shifting the upper half down first
// costs a temporary register per element, which the 13 x 4 plan does not have (the plans with
// 16-byte loads have, and keep the compiler's own sequence).
template <typename T, int EPV>
__device__ __forceinline__ float widen(const VecE<T, EPV> &v, int k) {
  if constexpr (std::is_same_v<T, f16_t> && EPV == 4) {
    typedef uint32_t words_t __attribute__((ext_vector_type(EPV / 2)));
    const words_t w = __builtin_bit_cast(words_t, v);
    const uint32_t word = w[k >> 1];
    float f;
    if (k & 1) {
      asm("v_cvt_f32_f16_sdwa %0, %1 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:WORD_1" : "=v"(f) : "v"(word));
    } else {
      asm("v_cvt_f32_f16_e32 %0, %1" : "=v"(f) : "v"(word));
    }
    return f;
  } else {
    return to_acc(v.e[k]);
  }
}

// Streaming variant for wide rows (the GPT-2 vocabulary): one 1024-lane
// workgroup per CU walks rows blockIdx.x, blockIdx.x + gridDim.x, ... and
// loads the next row into a second register set before it starts on the
// current one, so the CU's memory pipe stays busy while its VALUs work; the
// stores of a finished row drain under the next row's arithmetic.  Without
// this, all workgroups load, compute and store in lockstep and HBM idles for
// the whole compute phase.
//
// Each element costs one hardware exp2: lane-local max first, then
// e = 2^((x - m_lane) log2e) is kept in registers, one exchange of (max, sum)
// pairs across the 16 waves gives the row's max and sum, and the output is
// e * f with one per-lane factor f = 2^(m_lane*log2e - log2(sum) - max*log2e) * scale.
//
// HAS_W: per-class weights (nll_loss's `weight`): a row's gradient and loss carry w[target], and
// the mean divides by the sum of those weights, which the count launch left next to the count.
template <typename T, typename TD, int VPT, int EPV, bool HAS_W>
__global__ __launch_bounds__(1024) void ce_rows_stream_kernel(
    const T *logits, TD *dlogits, const int64_t *__restrict__ targets, float *__restrict__ row_loss,
    const int *__restrict__ ws_count, int64_t N, int64_t V, int64_t row_stride,
    int64_t ignore_index, int reduction, float dloss, const float *__restrict__ class_weight) {
  constexpr int BLOCK = 1024;
  constexpr int VN = EPV;  // elements per lane per access
  constexpr int kWaves = BLOCK / kWave;
  __shared__ float red_m[2][kWaves], red_s[2][kWaves];
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid >> 6;
  const int nvec = (int)(row_stride / VN);
  const int iV = (int)V;

  float scale0 = dloss;
  if (reduction == CS_REDUCTION_MEAN)
    scale0 = HAS_W ? dloss / reinterpret_cast<const float *>(ws_count)[1] : dloss / (float)(*ws_count);
  const float log2_scale0 = __builtin_amdgcn_logf(fabsf(scale0));  // -inf for 0: every output 0

  // Workgroups go round the eight XCDs in launch order.  The workgroups of one XCD take
  // neighbouring rows of each round of gridDim rows (XCD 0 the first eighth, and so on) rather
  // than every eighth row: [8192,50257] bf16 282.7 us per call against 285.2, with fp32 gradients
  // 444.5 against 450.8.
  int64_t row = (gridDim.x % 8 == 0) ? (int64_t)(blockIdx.x % 8) * (gridDim.x / 8) + blockIdx.x / 8 : blockIdx.x;
  VecE<T, EPV> cur[VPT];
  int64_t tgt = 0;
  bool live = false;
  float x_t = 0.f, wt = 1.f;
  if (row < N) {
    tgt = targets[row];
    live = target_counts(tgt, V, ignore_index);
    if (live) {
      if constexpr (HAS_W) wt = class_weight[tgt];
      const T *x = logits + row * row_stride;
#pragma unroll
      for (int j = 0; j < VPT; ++j) {
        const int idx = tid + BLOCK * j;
        if (idx < nvec) cur[j] = load_e_stream<T, EPV>(x + (int64_t)idx * VN);
      }
      if (tid == 0) x_t = to_acc(x[tgt]);
    }
  }
  int parity = 0;
  while (row < N) {
    // ---- issue the next row's loads
    const int64_t nrow = row + gridDim.x;
    VecE<T, EPV> nxt[VPT];
    int64_t ntgt = 0;
    bool nlive = false;
    float nx_t = 0.f, nwt = 1.f;
    if (nrow < N) {
      ntgt = targets[nrow];
      nlive = target_counts(ntgt, V, ignore_index);
      if (nlive) {
        if constexpr (HAS_W) nwt = class_weight[ntgt];
        const T *x = logits + nrow * row_stride;
#pragma unroll
        for (int j = 0; j < VPT; ++j) {
          const int idx = tid + BLOCK * j;
          // (kept under the lane's condition here: the compiler issues these back to back as they
          // are, and the unconditional form spills 56 bytes per lane: 283 -> 305 us)
          if (idx < nvec) nxt[j] = load_e_stream<T, EPV>(x + (int64_t)idx * VN);
        }
        if (tid == 0) nx_t = to_acc(x[ntgt]);
      }
    }

    if (!live) {
      if (tid == 0 && row_loss) row_loss[row] = 0.f;
      if (dlogits) {
        float z[VN];
#pragma unroll
        for (int k = 0; k < VN; ++k) z[k] = 0.f;
        for (int idx = tid; idx < nvec; idx += BLOCK)
          store_out<T, TD, VN>(dlogits + row * row_stride + (int64_t)idx * VN, z);
      }
    } else {
      // ---- widen, mask what is not a class column to -inf, lane-local max
      float e[VPT][VN];
      float m = -INFINITY;
#pragma unroll
      for (int j = 0; j < VPT; ++j) {
        const int c0 = (tid + BLOCK * j) * VN;
        if (c0 + VN <= iV) {
#pragma unroll
          for (int k = 0; k < VN; ++k) {
            e[j][k] = widen(cur[j], k);
            m = fmaxf(m, e[j][k]);
          }
        } else {
#pragma unroll
          for (int k = 0; k < VN; ++k) {
            e[j][k] = c0 + k < iV ? widen(cur[j], k) : -INFINITY;
            m = fmaxf(m, e[j][k]);
          }
        }
      }
      // a lane without any class column: any finite stand-in keeps 2^(-inf - m) = 0
      const float ml2 = (m == -INFINITY ? 0.f : m) * kLog2e;
      float s = 0.f;
#pragma unroll
      for (int j = 0; j < VPT; ++j)
#pragma unroll
        for (int k = 0; k < VN; ++k) {
          e[j][k] = __builtin_amdgcn_exp2f(e[j][k] * kLog2e - ml2);
          s += e[j][k];
        }
      // ---- (max, sum) across the wave, then across the 16 waves.  A lane without a finite
      // value takes no part: its stand-in maximum must not pass for a real one (the real ones
      // may all lie far below it), and its empty sum must not meet an overflowed 2^(0 - max)
      const bool empty = m == -INFINITY;
      const float mw2 = wave_reduce(empty ? -INFINITY : ml2, MaxOp{});
      const float sw = wave_reduce(empty ? 0.f : s * __builtin_amdgcn_exp2f(ml2 - mw2), SumOp{});
      if (lane == 0) {
        red_m[parity][wave] = mw2;
        red_s[parity][wave] = sw;
      }
      __syncthreads();
      const float pm = lane < kWaves ? red_m[parity][lane] : -INFINITY;
      const float ps = lane < kWaves ? red_s[parity][lane] : 0.f;
      const float M2 = wave_reduce(pm, MaxOp{});
      const float S = wave_reduce(pm == -INFINITY ? 0.f : ps * __builtin_amdgcn_exp2f(pm - M2), SumOp{});
      parity ^= 1;  // the other pair of arrays next time: one barrier per row is enough
      const float log2_S = __builtin_amdgcn_logf(S);
      // loss = ln(sum exp(x - max)) - (x_t - max), the difference to the maximum formed with one
      // fused multiply-add against the rounded M2 the sum was taken with
      {
        const float l = (log2_S - __builtin_fmaf(x_t, kLog2e, -M2)) * kLn2;
        if (tid == 0 && row_loss) row_loss[row] = HAS_W ? l * wt : l;
      }
      // the row's scale: the call's, times the weight of the row's class
      const float scale = HAS_W ? scale0 * wt : scale0;
      const float log2_scale = HAS_W ? log2_scale0 + __builtin_amdgcn_logf(fabsf(wt)) : log2_scale0;
      const bool negate = scale < 0.f;

      if (dlogits) {
        // a lane that holds no class column has e = 0 everywhere; give it f = 0 so that
        // 0 * f cannot meet an overflowed factor
        float f = empty ? 0.f : __builtin_amdgcn_exp2f(ml2 - M2 - log2_S + log2_scale);
        f = negate ? -f : f;
        const int t_vec = (int)(tgt / VN), t_sub = (int)(tgt % VN);
        TD *d = dlogits + row * row_stride;
#pragma unroll
        for (int j = 0; j < VPT; ++j) {
          const int idx = tid + BLOCK * j;
          if (idx < nvec) {
            float o[VN];
#pragma unroll
            for (int k = 0; k < VN; ++k) o[k] = e[j][k] * f;
            if (idx == t_vec) {
              // the exponent-folded factor f is good to ~1e-6 relative (its logarithms are),
              // which subtracting `scale` amplifies when p is close to 1: the target element
              // is formed as a product instead
              const float exact = __builtin_amdgcn_exp2f(ml2 - M2) * (scale * __builtin_amdgcn_rcpf(S));
#pragma unroll
              for (int k = 0; k < VN; ++k)
                if (k == t_sub) o[k] = e[j][k] * exact - scale;
            }
            store_out<T, TD, VN>(d + (int64_t)idx * VN, o);
          }
        }
      }
    }
#pragma unroll
    for (int j = 0; j < VPT; ++j) cur[j] = nxt[j];
    live = nlive;
    tgt = ntgt;
    x_t = nx_t;
    wt = nwt;
    row = nrow;
  }
}

// Rows too wide for registers (more than 8192 16-byte vectors: vocabularies beyond 65536 at 16
// bit, 32768 at fp32), and rows whose stride is not a multiple of the vector width (a
// vocabulary used unpadded).  Persistent workgroups walk rows.  A row is split into a head of
// single elements up to the first 16-byte boundary, a body of whole vectors and a tail; the
// base pointers are 16-byte aligned, so gradient rows split at the same columns.  The body is
// read twice in chunks of kWideU vectors per lane: the first sweep keeps a running (max, sum)
// per lane (rescaling the sum when the maximum moves: one exp2 per element plus one per
// chunk), the second sweep re-reads the row, which the first one left in the L2 / last-level
// cache, and writes the gradient.  Only a handful of scalars is carried between the sweeps,
// so two workgroups share a CU and cover each other's waits.
constexpr int kWideU = 2;  // 16-byte vectors per lane and chunk
static_assert(kWideU == 2, "the chunk sum below adds two vector sums");

template <typename T, typename TD, int BLOCK>
__global__ __launch_bounds__(BLOCK, 8) void ce_rows_wide_kernel(
    const T *logits, TD *dlogits, const int64_t *__restrict__ targets, float *__restrict__ row_loss,
    const int *__restrict__ ws_count, int64_t N, int64_t V, int64_t row_stride,
    int64_t ignore_index, int reduction, float dloss, const float *__restrict__ class_weight) {
  constexpr int VN = Vec16<T>::n;
  constexpr int kWaves = BLOCK / kWave;
  constexpr int kTailLane = 32;  // lanes [0, VN) own head elements, [32, 32 + VN) tail elements
  static_assert(VN <= kTailLane, "head and tail lanes overlap");
  __shared__ float red_m[kWaves], red_s[kWaves];
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid >> 6;
  const int stride = (int)row_stride;  // the host checks that it fits
  const int vcols = (int)V;
  // per-class weights (at::nll_loss's `weight`): a row's loss and gradient are scaled by the
  // weight of its target, and the mean is over the sum of those weights
  float scale0 = dloss;
  if (reduction == CS_REDUCTION_MEAN)
    scale0 = class_weight ? dloss / reinterpret_cast<const float *>(ws_count)[1] : dloss / (float)(*ws_count);

  for (int64_t row = blockIdx.x; row < N; row += gridDim.x) {
    const int64_t tgt = targets[row];
    const T *x = logits + row * row_stride;
    TD *d = dlogits ? dlogits + row * row_stride : nullptr;
    // columns [0, head) before the first aligned vector, nvec vectors, then the rest
    int head = (int)((VN - (row * row_stride) % VN) % VN);
    head = head < stride ? head : stride;
    const int nvec = (stride - head) / VN;
    const int tail0 = head + nvec * VN;
    int ecol = -1;  // the single element this lane owns, if any
    if (tid < head) ecol = tid;
    if (tid >= kTailLane && tail0 + (tid - kTailLane) < stride) ecol = tail0 + (tid - kTailLane);
    const T *xb = x + head;
    TD *db = d ? d + head : nullptr;

    if (!target_counts(tgt, V, ignore_index)) {  // block-uniform
      if (tid == 0 && row_loss) row_loss[row] = 0.f;
      if (d) {
        float z[VN];
#pragma unroll
        for (int k = 0; k < VN; ++k) z[k] = 0.f;
        for (int idx = tid; idx < nvec; idx += BLOCK) store_out<T, TD, VN>(db + (int64_t)idx * VN, z);
        if (ecol >= 0) d[ecol] = from_acc<TD>(0.f);
      }
      continue;
    }
    // ---- sweep 1: running maximum (times log2 e) and the sum relative to it
    float xe = -INFINITY;
    if (ecol >= 0 && ecol < vcols) xe = to_acc(x[ecol]);
    float m2 = xe * kLog2e;
    // the same expression as in the second sweep (the fma sees the product unrounded, so this is not exactly 1)
    float s = xe == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(__builtin_fmaf(xe, kLog2e, -m2));
    for (int base = tid; base < nvec + tid; base += BLOCK * kWideU) {
      Vec16<T> v[kWideU];
#pragma unroll
      for (int u = 0; u < kWideU; ++u) {
        const int idx = base + BLOCK * u;
        // cached: read again below.  Every lane loads, see ce_rows_kernel.
        v[u] = load16(xb + (int64_t)(idx < nvec ? idx : nvec - 1) * VN);
      }
      float xs[kWideU][VN];
      float cm = -INFINITY;
#pragma unroll
      for (int u = 0; u < kWideU; ++u) {
        const int idx = base + BLOCK * u;
        const int c0 = head + idx * VN;
#pragma unroll
        for (int k = 0; k < VN; ++k) {
          xs[u][k] = (idx < nvec && c0 + k < vcols) ? vec_get(v[u], k) : -INFINITY;  // padding, lanes past the row
          cm = fmaxf(cm, xs[u][k]);
        }
      }
      const float cm2 = cm * kLog2e;
      if (cm2 > m2) {
        s *= __builtin_amdgcn_exp2f(m2 - cm2);  // 0 the first time (m2 = -inf, s = 0)
        m2 = cm2;
      }
      if (m2 != -INFINITY) {
        // pairwise within the chunk, one add onto the running sum: once a dominant term sits
        // in s, every further add rounds at its size, so there should be few of them
        float part[kWideU];
#pragma unroll
        for (int u = 0; u < kWideU; ++u) {
          float e[VN];
#pragma unroll
          for (int k = 0; k < VN; ++k) e[k] = __builtin_amdgcn_exp2f(__builtin_fmaf(xs[u][k], kLog2e, -m2));
#pragma unroll
          for (int w = VN / 2; w > 0; w /= 2)
#pragma unroll
            for (int k = 0; k < w; ++k) e[k] += e[k + w];
          part[u] = e[0];
        }
        s += part[0] + part[1];
      }
    }
    // ---- (max, sum) across the wave, then across the waves
    const float mw2 = wave_reduce(m2, MaxOp{});
    const float sw = wave_reduce(m2 == -INFINITY ? 0.f : s * __builtin_amdgcn_exp2f(m2 - mw2), SumOp{});
    __syncthreads();  // the previous row's readers are done with red_m / red_s
    if (lane == 0) {
      red_m[wave] = mw2;
      red_s[wave] = sw;
    }
    __syncthreads();
    const float pm = lane < kWaves ? red_m[lane] : -INFINITY;
    const float ps = lane < kWaves ? red_s[lane] : 0.f;
    const float M2 = wave_reduce(pm, MaxOp{});
    const float S = wave_reduce(pm == -INFINITY ? 0.f : ps * __builtin_amdgcn_exp2f(pm - M2), SumOp{});
    const float wt = class_weight ? class_weight[tgt] : 1.0f;
    const float scale = class_weight ? scale0 * wt : scale0;
    if (tid == 0 && row_loss) {
      const float x_t = to_acc(x[tgt]);
      const float l = (__builtin_amdgcn_logf(S) - __builtin_fmaf(x_t, kLog2e, -M2)) * kLn2;
      row_loss[row] = class_weight ? l * wt : l;
    }
    if (!d) continue;
    // ---- sweep 2: p = 2^(x log2e - M2) / S, gradient (p - onehot) * scale
    const float factor = scale / S;
    const int t_vec = tgt >= head ? (int)((tgt - head) / VN) : -1;  // past the body if in the tail
    const int t_sub = (int)((tgt - head) % VN);
    if (ecol >= 0) {
      float o = 0.f;
      if (ecol < vcols) {
        o = __builtin_amdgcn_exp2f(__builtin_fmaf(xe, kLog2e, -M2)) * factor;
        if (ecol == tgt) o -= scale;
      }
      d[ecol] = from_acc<TD>(o);
    }
    for (int base = tid; base < nvec + tid; base += BLOCK * kWideU) {
      Vec16<T> v[kWideU];
#pragma unroll
      for (int u = 0; u < kWideU; ++u) {
        const int idx = base + BLOCK * u;
        v[u] = load16_stream(xb + (int64_t)(idx < nvec ? idx : nvec - 1) * VN);
      }
#pragma unroll
      for (int u = 0; u < kWideU; ++u) {
        const int idx = base + BLOCK * u;
        if (idx < nvec) {
          const int c0 = head + idx * VN;
          float o[VN];
#pragma unroll
          for (int k = 0; k < VN; ++k)
            o[k] = c0 + k < vcols ? __builtin_amdgcn_exp2f(__builtin_fmaf(vec_get(v[u], k), kLog2e, -M2)) * factor : 0.f;
          if (idx == t_vec) {
#pragma unroll
            for (int k = 0; k < VN; ++k)
              if (k == t_sub) o[k] -= scale;
          }
          store_out<T, TD, VN>(db + (int64_t)idx * VN, o);
        }
      }
    }
  }
}

// Any V, stride and alignment; fp64 too.  Three sweeps over the row, the
// later ones served by the cache.
template <typename T, typename TD>
__global__ __launch_bounds__(256) void ce_rows_general_kernel(
    const T *__restrict__ logits, TD *__restrict__ dlogits, const int64_t *__restrict__ targets,
    float *__restrict__ row_loss, const int *__restrict__ ws_count, int64_t V, int64_t row_stride,
    int64_t ignore_index, int reduction, float dloss, const float *__restrict__ class_weight) {
  using U = typename Acc<T>::type;
  __shared__ U scratch[4];
  const int64_t row = blockIdx.x;
  const T *x = logits + row * row_stride;
  const int64_t target = targets[row];
  const bool counts = target_counts(target, V, ignore_index);
  if (!counts) {
    if (threadIdx.x == 0 && row_loss) row_loss[row] = 0.f;
    if (dlogits)
      for (int64_t c = threadIdx.x; c < row_stride; c += 256)
        dlogits[row * row_stride + c] = from_acc<TD>((typename Acc<TD>::type)0);
    return;
  }
  U m = -INFINITY;
  for (int64_t c = threadIdx.x; c < V; c += 256) {
    const U v = to_acc(x[c]);
    m = v > m ? v : m;
  }
  m = block_reduce(m, MaxOp{}, (U)-INFINITY, scratch);
  U s = 0;
  for (int64_t c = threadIdx.x; c < V; c += 256) s += exp((U)to_acc(x[c]) - m);
  s = block_reduce(s, SumOp{}, (U)0, scratch);
  const U lse = m + log(s);
  const U wt = class_weight ? (U)class_weight[target] : (U)1;
  if (threadIdx.x == 0 && row_loss) row_loss[row] = (float)((lse - (U)to_acc(x[target])) * wt);
  if (!dlogits) return;
  U scale = (U)dloss;
  if (reduction == CS_REDUCTION_MEAN)
    scale = class_weight ? (U)dloss / (U) reinterpret_cast<const float *>(ws_count)[1] : (U)dloss / (U)(*ws_count);
  scale *= wt;
  for (int64_t c = threadIdx.x; c < row_stride; c += 256) {
    U o = 0;
    if (c < V) {
      o = exp((U)to_acc(x[c]) - lse);
      if (c == target) o -= (U)1;
      o *= scale;
    }
    dlogits[row * row_stride + c] = from_acc<TD>((typename Acc<TD>::type)o);
  }
}

// CUs of the current device, asked once per device (threads may race to fill a slot: they
// store the same value).
int64_t compute_units() {
  static std::atomic<int> cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  int n = cached[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    cached[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

// Two-sweep kernel: workgroups of 1024 lanes, two per CU, for wide rows; of 256 lanes, eight
// per CU, where a row has too few vectors to occupy 1024.
template <typename T, typename TD>
void launch_wide(const void *logits, void *dlogits, const int64_t *targets, float *row_loss,
                 const int *ws_count, int64_t N, int64_t V, int64_t row_stride, int64_t ignore_index,
                 int reduction, float dloss, const float *class_weight, hipStream_t s) {
  const int64_t cus = compute_units();
  const int64_t nvec = row_stride / Vec16<T>::n;
  if (nvec > 256 * kWideU * 2) {
    const dim3 grid((unsigned)(N < 2 * cus ? N : 2 * cus));
    ce_rows_wide_kernel<T, TD, 1024><<<grid, dim3(1024), 0, s>>>(
        (const T *)logits, (TD *)dlogits, targets, row_loss, ws_count, N, V, row_stride, ignore_index,
        reduction, dloss, class_weight);
  } else {
    const dim3 grid((unsigned)(N < 8 * cus ? N : 8 * cus));
    ce_rows_wide_kernel<T, TD, 256><<<grid, dim3(256), 0, s>>>(
        (const T *)logits, (TD *)dlogits, targets, row_loss, ws_count, N, V, row_stride, ignore_index,
        reduction, dloss, class_weight);
  }
}

template <typename T, typename TD>
int launch_rows(const void *logits, void *dlogits, const int64_t *targets, float *row_loss,
                const int *ws_count, int64_t N, int64_t V, int64_t row_stride,
                int64_t ignore_index, int reduction, float dloss, const float *class_weight, hipStream_t s) {
  constexpr int VN = Vec16<T>::n;
  const bool base_ok = !std::is_same_v<T, double> && is_aligned16(logits) &&
                       (!dlogits || is_aligned16(dlogits)) && row_stride <= (int64_t(1) << 30);
  const bool vec_ok = base_ok && row_stride % VN == 0;
  const dim3 grid((unsigned)N);
  if constexpr (!std::is_same_v<T, double>) {
    // per-class weights: the streaming kernel, the two-sweep kernel (any aligned row) and the
    // general one take them; the small row-in-registers kernels do not (no caller of the reference
    // sets weights), so weighted calls on narrow rows go to the two-sweep kernel
    const int64_t nvec_all = row_stride / VN;
    const bool streams = nvec_all > 256 * 8 &&
                         nvec_all <= (sizeof(T) == 4 ? 1024 * 8 : sizeof(TD) == 4 ? 512 * 13 : 1024 * 7);
    if (vec_ok && (class_weight == nullptr || streams)) {
      const int64_t nvec = row_stride / VN;
#define CS_CE(BLOCK, VPT)                                                                   \
  ce_rows_kernel<T, TD, BLOCK, VPT><<<grid, dim3(BLOCK), 0, s>>>(                           \
      (const T *)logits, (TD *)dlogits, targets, row_loss, ws_count, V, row_stride,         \
      ignore_index, reduction, dloss)
      if (nvec <= 64 * 8) {
        CS_CE(64, 8);
      } else if (nvec <= 256 * 8) {
        CS_CE(256, 8);
      } else if (nvec <= (sizeof(T) == 4 ? 1024 * 8 : sizeof(TD) == 4 ? 512 * 13 : 1024 * 7)) {
        // one persistent workgroup per CU, the row in registers.  The widest plans (8 vectors
        // per lane at 16 bit, 16 half vectors with fp32 gradients) measured slower than the
        // two-sweep kernel and are not built.
        const int64_t cus = compute_units();
        const dim3 pgrid((unsigned)(N < cus ? N : cus));
#define CS_CE_STREAM(VPT, EPV)                                                                    \
  if (class_weight != nullptr) {                                                                  \
    ce_rows_stream_kernel<T, TD, VPT, EPV, true><<<pgrid, dim3(1024), 0, s>>>(                    \
        (const T *)logits, (TD *)dlogits, targets, row_loss, ws_count, N, V, row_stride,          \
        ignore_index, reduction, dloss, class_weight);                                            \
  } else {                                                                                        \
    ce_rows_stream_kernel<T, TD, VPT, EPV, false><<<pgrid, dim3(1024), 0, s>>>(                   \
        (const T *)logits, (TD *)dlogits, targets, row_loss, ws_count, N, V, row_stride,          \
        ignore_index, reduction, dloss, nullptr);                                                 \
  }
        if constexpr (sizeof(T) == 2 && sizeof(TD) == 4) {
          CS_CE_STREAM(13, 4);  // 16-bit logits, fp32 gradients (autocast): 4 elements per lane per access
        } else if (nvec <= 1024 * 4) {
          CS_CE_STREAM(4, VN);
        } else if (nvec <= 1024 * 7) {
          CS_CE_STREAM(7, VN);
        } else {
          if constexpr (sizeof(T) == 4) {
            CS_CE_STREAM(8, VN);
          }
        }
#undef CS_CE_STREAM
      } else if (sizeof(T) == 4 && nvec <= 1024 * 16) {
        // fp32 rows up to 65536 columns still fit in registers (at 16 bit this plan spills)
        if constexpr (sizeof(T) == 4) CS_CE(1024, 16);
      } else {
        launch_wide<T, TD>(logits, dlogits, targets, row_loss, ws_count, N, V, row_stride, ignore_index,
                           reduction, dloss, class_weight, s);
      }
#undef CS_CE
      return launch_status();
    }
    if (base_ok && sizeof(TD) >= sizeof(T)) {
      // rows that start off a 16-byte boundary: split per row into head, vectors and tail
      launch_wide<T, TD>(logits, dlogits, targets, row_loss, ws_count, N, V, row_stride, ignore_index,
                         reduction, dloss, class_weight, s);
      return launch_status();
    }
  }
  ce_rows_general_kernel<T, TD><<<grid, dim3(256), 0, s>>>((const T *)logits, (TD *)dlogits,
                                                            targets, row_loss, ws_count, V,
                                                            row_stride, ignore_index, reduction,
                                                            dloss, class_weight);
  return launch_status();
}

}  // namespace
}  // namespace cs_hip

using namespace cs_hip;

extern "C" size_t cs_fused_classifier_workspace_bytes(int64_t N) {
  if (N < 0) return 0;
  return kWsHeader + ((size_t)N * sizeof(float) + 255) / 256 * 256;
}

namespace {

struct CeArgs {
  const void *logits;
  void *dlogits;
  const int64_t *targets;
  float *row_loss;
  float *loss;
  float *total_weight;
  void *workspace;
  size_t workspace_bytes;
  int64_t N, V, row_stride, ignore_index;
  int reduction;
  float dloss;
  int dtype, dlogits_dtype;
  const float *class_weight = nullptr;  // [V] fp32, or NULL: every class weighs 1
};

int ce_validate(const CeArgs &a) {
  if (a.N < 0 || a.V <= 0 || a.row_stride < a.V) return CS_ERR_INVALID_ARGUMENT;
  if (a.reduction != CS_REDUCTION_NONE && a.reduction != CS_REDUCTION_MEAN &&
      a.reduction != CS_REDUCTION_SUM)
    return CS_ERR_INVALID_ARGUMENT;
  const size_t es = dtype_size(a.dtype), ds = dtype_size(a.dlogits_dtype);
  if (es == 0 || ds == 0) return CS_ERR_UNSUPPORTED;
  if (a.dlogits_dtype != a.dtype && !(a.dlogits_dtype == CS_F32 && es == 2))
    return CS_ERR_UNSUPPORTED;
  if (a.N > 0x7fffffffLL || a.V > 0x7fffffffLL || a.row_stride > 0x7fffffffLL)
    return CS_ERR_TOO_LARGE;
  if (!a.workspace || a.workspace_bytes < cs_fused_classifier_workspace_bytes(a.N) ||
      !aligned_to(a.workspace, 256))
    return CS_ERR_WORKSPACE;
  if (a.reduction == CS_REDUCTION_NONE && !a.row_loss) return CS_ERR_INVALID_ARGUMENT;
  if (a.reduction != CS_REDUCTION_NONE && !a.loss) return CS_ERR_INVALID_ARGUMENT;
  if (a.N > 0 && (!a.logits || !a.targets)) return CS_ERR_INVALID_ARGUMENT;
  if ((a.logits && !aligned_to(a.logits, es)) || (a.dlogits && !aligned_to(a.dlogits, ds)) ||
      (a.targets && !aligned_to(a.targets, 8)) || (a.row_loss && !aligned_to(a.row_loss, 4)) ||
      (a.loss && !aligned_to(a.loss, 4)) || (a.total_weight && !aligned_to(a.total_weight, 4)) ||
      (a.class_weight && !aligned_to(a.class_weight, 4)))
    return CS_ERR_MISALIGNED;
  if (a.dlogits == a.logits && a.dlogits_dtype != a.dtype) return CS_ERR_INVALID_ARGUMENT;
  return CS_OK;
}

// phases: 1 = count the rows that are not ignored, 2 = the row pass,
// 4 = reduce the row losses
int ce_run(const CeArgs &a, int phases, void *stream) {
  int st = ce_validate(a);
  if (st != CS_OK) return st;
  hipStream_t s = as_stream(stream);
  char *ws = static_cast<char *>(a.workspace);
  int *ws_count = reinterpret_cast<int *>(ws);
  float *ws_weight = reinterpret_cast<float *>(ws) + 1;
  float *rows = a.row_loss ? a.row_loss : reinterpret_cast<float *>(ws + kWsHeader);
  if (phases & 1) {
    ce_count_kernel<<<dim3(1), dim3(1024), 0, s>>>(a.targets, a.N, a.V, a.ignore_index, ws_count,
                                                   ws_weight, a.class_weight);
    st = launch_status();
    if (st != CS_OK) return st;
  }
  if ((phases & 2) && a.N > 0) {
#define CS_CALL(T, TD)                                                                      \
  st = launch_rows<T, TD>(a.logits, a.dlogits, a.targets, rows, ws_count, a.N, a.V,         \
                          a.row_stride, a.ignore_index, a.reduction, a.dloss, a.class_weight, s)
    const bool wide = a.dlogits_dtype != a.dtype;
    switch (a.dtype) {
      case CS_F32: CS_CALL(float, float); break;
      case CS_F64: CS_CALL(double, double); break;
      case CS_F16:
        if (wide) {
          CS_CALL(f16_t, float);
        } else {
          CS_CALL(f16_t, f16_t);
        }
        break;
      case CS_BF16:
        if (wide) {
          CS_CALL(bf16_t, float);
        } else {
          CS_CALL(bf16_t, bf16_t);
        }
        break;
    }
#undef CS_CALL
    if (st != CS_OK) return st;
  }
  if (phases & 4) {
    ce_reduce_kernel<<<dim3(1), dim3(1024), 0, s>>>(
        rows, a.N, ws_count, a.reduction, a.reduction == CS_REDUCTION_NONE ? nullptr : a.loss,
        a.total_weight);
    st = launch_status();
  }
  return st;
}

}  // namespace

extern "C" int cs_fused_classifier(const void *logits, void *dlogits, const int64_t *targets,
                                   float *row_loss, float *loss, float *total_weight,
                                   void *workspace, size_t workspace_bytes, int64_t N, int64_t V,
                                   int64_t row_stride, int64_t ignore_index, int reduction,
                                   float dloss, int dtype, int dlogits_dtype, void *stream) {
  const CeArgs a{logits, dlogits, targets,      row_loss,  loss,  total_weight, workspace,
                 workspace_bytes, N, V, row_stride, ignore_index, reduction, dloss, dtype,
                 dlogits_dtype};
  return ce_run(a, 1 | 2 | 4, stream);
}

extern "C" int cs_fused_classifier_weighted(const void *logits, void *dlogits, const int64_t *targets,
                                            const float *class_weight, float *row_loss, float *loss,
                                            float *total_weight, void *workspace, size_t workspace_bytes,
                                            int64_t N, int64_t V, int64_t row_stride, int64_t ignore_index,
                                            int reduction, float dloss, int dtype, int dlogits_dtype,
                                            void *stream) {
  CeArgs a{logits, dlogits, targets,      row_loss,  loss,  total_weight, workspace,
           workspace_bytes, N, V, row_stride, ignore_index, reduction, dloss, dtype,
           dlogits_dtype};
  a.class_weight = class_weight;
  return ce_run(a, 1 | 2 | 4, stream);
}

// ------------------------------------------------- the call that allocates nothing
// Device memory that belongs to the library, one copy per GPU, held until the process ends:
// the workspace of cs_fused_classifier_static.  In host code this name is only a handle for
// hipGetSymbolAddress; the address that kernels and the host use is the one that call returns.
static __device__ __align__(256) unsigned char scratch[CS_FUSED_CLASSIFIER_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
// the scratch array's address on each device, looked up once per device (threads may race to
// fill a slot: they store the same value)
std::atomic<void *> scratch_ptr[kMaxDevices];

int static_scratch(void **out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kMaxDevices) return CS_ERR_UNSUPPORTED;
  void *p = scratch_ptr[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    // the current device's copy of the array
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (p == nullptr) return CS_ERR_WORKSPACE;
    scratch_ptr[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return CS_OK;
}
}  // namespace

extern "C" int64_t cs_fused_classifier_static_max_rows(void) {
  return ((int64_t)CS_FUSED_CLASSIFIER_STATIC_SCRATCH_BYTES - (int64_t)kWsHeader) / (int64_t)sizeof(float);
}

extern "C" int cs_fused_classifier_static(const void *logits, void *dlogits, const int64_t *targets,
                                          float *row_loss, float *loss, float *total_weight,
                                          int64_t N, int64_t V, int64_t row_stride,
                                          int64_t ignore_index, int reduction, float dloss,
                                          int dtype, int dlogits_dtype, void *stream) {
  if (N > cs_fused_classifier_static_max_rows()) return CS_ERR_STATIC_LIMIT;
  void *ws = nullptr;
  const int st = static_scratch(&ws);
  if (st != CS_OK) return st;
  // Nothing in the scratch has to start at zero: the counting launch overwrites the header and
  // the row pass overwrites the N row losses that the reduction then reads.
  const CeArgs a{logits, dlogits, targets, row_loss, loss, total_weight, ws,
                 (size_t)CS_FUSED_CLASSIFIER_STATIC_SCRATCH_BYTES, N, V, row_stride, ignore_index,
                 reduction, dloss, dtype, dlogits_dtype};
  return ce_run(a, 1 | 2 | 4, stream);
}

extern "C" int cs_fused_classifier_phases(const void *logits, void *dlogits,
                                          const int64_t *targets, float *row_loss, float *loss,
                                          float *total_weight, void *workspace,
                                          size_t workspace_bytes, int64_t N, int64_t V,
                                          int64_t row_stride, int64_t ignore_index, int reduction,
                                          float dloss, int dtype, int dlogits_dtype, int phases,
                                          void *stream) {
  if (phases <= 0 || phases > 7) return CS_ERR_INVALID_ARGUMENT;
  const CeArgs a{logits, dlogits, targets,      row_loss,  loss,  total_weight, workspace,
                 workspace_bytes, N, V, row_stride, ignore_index, reduction, dloss, dtype,
                 dlogits_dtype};
  return ce_run(a, phases, stream);
}
