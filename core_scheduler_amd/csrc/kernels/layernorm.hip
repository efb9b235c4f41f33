// LayerNorm forward / backward over the last dimension for gfx950.
//
// Replaces at::native_layer_norm (src/compute/layer_norm.cpp:163-169,
// :198-204) and the two at::native_layer_norm_backward calls (:263-266 for
// dx, :321-334 / :375-383 for dgamma and dbeta).  Statistics and all
// arithmetic are fp32 for f32/f16/bf16 storage (fp64 for f64):
//   mean = sum(x)/C, var = sum((x-mean)^2)/C (biased), rstd = 1/sqrt(var+eps)
//   y    = (x-mean)*rstd*gamma + beta
//   dx   = rstd * (g - mean_C(g) - xhat*mean_C(g*xhat)),  g = dy*gamma
//   dgamma = sum_rows(dy*xhat), dbeta = sum_rows(dy)
//
// Fast path: one wavefront owns whole rows.  A row lives in registers as
// 16-byte vectors (lane l holds vectors l, l+64, ...), the two row sums are
// wave64 butterflies, and nothing is read twice: forward moves x once in and
// y once out, backward reads dy and x once and produces dx and the
// per-column partial sums in the same pass.  Each lane keeps the partial
// dgamma/dbeta of its own columns in registers across all rows its wave
// visits; a workgroup folds its waves through LDS and writes one partial row
// per workgroup, and a second small kernel adds the partial rows in a fixed
// order, so the result does not depend on scheduling and uses no atomics.
//
// Anything the fast path cannot take (C not a multiple of the vector width,
// C beyond the register budget, unaligned pointers, fp64) goes through a
// plain one-workgroup-per-row path.
#include "common.hpp"

#include <math.h>

#include <atomic>
#include <type_traits>

// Every product and sum below is rounded as written: no multiply-add contraction, so that the
// template variants of one kernel (with and without the fused residual adds, every output
// mask) produce the same bits for the same row.
#pragma clang fp contract(off)

namespace cs_hip {
namespace {

// ------------------------------------------------------------ n-wide access
// N consecutive elements of T (N * sizeof(T) is 16 or 32 bytes) <-> fp32.
template <typename T, int N>
__device__ __forceinline__ void load_n(const T *p, float (&out)[N]) {
  constexpr int VN = Vec16<T>::n;
  static_assert(N % VN == 0, "whole 16-byte pieces");
#pragma unroll
  for (int q = 0; q < N / VN; ++q) {
    const Vec16<T> v = load16(p + q * VN);
#pragma unroll
    for (int k = 0; k < VN; ++k) out[q * VN + k] = to_acc(v.e[k]);
  }
}
template <typename T, int N>
__device__ __forceinline__ void store_n(T *p, const float (&in)[N]) {
  constexpr int VN = Vec16<T>::n;
  static_assert(N % VN == 0, "whole 16-byte pieces");
#pragma unroll
  for (int q = 0; q < N / VN; ++q) {
    Vec16<T> v;
#pragma unroll
    for (int k = 0; k < VN; ++k) v.e[k] = from_acc<T>(in[q * VN + k]);
    store16_stream(p + q * VN, v);
  }
}
// raw (still packed) row pieces, so a row costs 4 VGPRs per 16 bytes
template <typename T, int N>
struct Raw {
  Vec16<T> v[N / Vec16<T>::n];
};
template <typename T, int N>
__device__ __forceinline__ Raw<T, N> load_raw(const T *p) {
  Raw<T, N> r;
#pragma unroll
  for (int q = 0; q < N / Vec16<T>::n; ++q) r.v[q] = load16_stream(p + q * Vec16<T>::n);
  return r;
}
// Makes the compiler forget what it derived from the packed values, so code after
// this point unpacks them again instead of keeping the unpacked floats in registers.
template <typename T, int N>
__device__ __forceinline__ void forget_unpacked(Raw<T, N> &r) {
#pragma unroll
  for (int q = 0; q < N / Vec16<T>::n; ++q) {
    u32x4 w = __builtin_bit_cast(u32x4, r.v[q]);
    asm volatile("" : "+v"(w));
    r.v[q] = __builtin_bit_cast(Vec16<T>, w);
  }
}
template <typename T, int N>
__device__ __forceinline__ Raw<T, N> zero_raw() {
  Raw<T, N> r;
#pragma unroll
  for (int q = 0; q < N / Vec16<T>::n; ++q)
#pragma unroll
    for (int k = 0; k < Vec16<T>::n; ++k) r.v[q].e[k] = T{};
  return r;
}
template <typename T, int N>
__device__ __forceinline__ float raw_get(const Raw<T, N> &r, int i) {
  return to_acc(r.v[i / Vec16<T>::n].e[i % Vec16<T>::n]);
}

constexpr int kHalf = kWave / 2;

// Sum over the LPR lanes that share a row (all 64, or each half of the wave on its own).
template <int LPR>
__device__ __forceinline__ float row_lanes_sum(float v, bool upper) {
  v += dpp_f32<kDppQuadXor1>(v);
  v += dpp_f32<kDppQuadXor2>(v);
  v += dpp_f32<kDppHalfMirror>(v);
  v += dpp_f32<kDppRowMirror>(v);
  const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
  const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 16));
  const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
  const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 48));
  if constexpr (LPR == kWave) return (r0 + r1) + (r2 + r3);
  return upper ? r2 + r3 : r0 + r1;
}

// forward launch shape (rows a wave normalises per step, next step's rows prefetched or not)
#ifndef CS_LN_FWD_ROWS_VPL1
#define CS_LN_FWD_ROWS_VPL1 4
#endif
#ifndef CS_LN_FWD_ROWS_VPL2
#define CS_LN_FWD_ROWS_VPL2 4
#endif
#ifndef CS_LN_FWD_ROWS_VPL4
#define CS_LN_FWD_ROWS_VPL4 2
#endif
#ifndef CS_LN_FWD_PF
#define CS_LN_FWD_PF true
#endif
#ifndef CS_LN_ADD_ROWS_VPL1
#define CS_LN_ADD_ROWS_VPL1 4
#endif
#ifndef CS_LN_ADD_ROWS_VPL2
#define CS_LN_ADD_ROWS_VPL2 4
#endif
#ifndef CS_LN_ADD_ROWS_VPL4
#define CS_LN_ADD_ROWS_VPL4 2
#endif
// two rows per wave (rows of up to 32, and of 65-96, vectors): row pairs a wave normalises per step
#ifndef CS_LN_FWD_HALF
#define CS_LN_FWD_HALF 1
#endif
#ifndef CS_LN_FWD_ROWS_H1
#define CS_LN_FWD_ROWS_H1 4
#endif
#ifndef CS_LN_FWD_ROWS_H3
#define CS_LN_FWD_ROWS_H3 2
#endif
#ifndef CS_LN_ADD_ROWS_H1
#define CS_LN_ADD_ROWS_H1 4
#endif
#ifndef CS_LN_ADD_ROWS_H3
#define CS_LN_ADD_ROWS_H3 2
#endif
#ifndef CS_LN_THREADS
#define CS_LN_THREADS 256
#endif
constexpr int kLnThreads = CS_LN_THREADS;  // 4 waves
// backward launch shape; the defaults are the measured best, the macros exist for tuning runs
#ifndef CS_LN_BWD_THREADS
#define CS_LN_BWD_THREADS 512
#endif
// grid caps of the backward row kernel, by 16-byte vectors per lane (the partial rows the
// launch leaves behind are one per workgroup): 512 workgroups of 8 waves, four waves per SIMD,
// for rows of up to 128 vectors; 256, two per SIMD, beyond (their accumulators take twice the
// registers)
#ifndef CS_LN_BWD_MAX_BLOCKS_VPL2
#define CS_LN_BWD_MAX_BLOCKS_VPL2 512
#endif
#ifndef CS_LN_BWD_MAX_BLOCKS
#define CS_LN_BWD_MAX_BLOCKS 256
#endif
constexpr int kLnBwdThreads = CS_LN_BWD_THREADS;

// ------------------------------------------------------------ fast forward
// VPL: 16-byte x vectors per lane; R: rows a wave handles per step.  A wave
// keeps gamma and beta for its columns in registers and walks rows
// gw*R, (gw + n_waves)*R, ...; the next step's rows are loaded before the
// current ones are normalised, so loads overlap the arithmetic and the
// parameters are read once per wave, not once per row.
// VN is the column count per vector position (set by x's type); T may be wider.
template <typename T, int VN, int VPL, int R>
struct RowSet {
  Raw<T, VN> v[R][VPL];
};

template <typename T, int VN, int VPL, int R, int LPR = kWave>
__device__ __forceinline__ void load_rows(RowSet<T, VN, VPL, R> &dst, const T *__restrict__ src,
                                          int64_t row0, int64_t rows, int C, int nvec, int lane) {
  // LPR lanes per row: with 32, the wave's halves hold rows row0 + 2r and row0 + 2r + 1
  constexpr int RPW = kWave / LPR;
  const int sub = lane / LPR, hl = lane % LPR;
#pragma unroll
  for (int r = 0; r < R; ++r) {
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
      const int idx = hl + LPR * j;
      const int64_t row = row0 + r * RPW + sub;
      if (idx < nvec && row < rows) {
        dst.v[r][j] = load_raw<T, VN>(src + row * C + (int64_t)idx * VN);
      } else {
        dst.v[r][j] = zero_raw<T, VN>();
      }
    }
  }
}

// One row, every lane loading: lanes past the end of the row read its last vector again.  A load
// under a lane-dependent condition can make the compiler wait for it before it issues the next
// one (it did for the third input of the backward kernel: two extra round trips per row), an
// unconditional one cannot.  What the extra lanes hold is masked where it matters (zero_past_row).
template <typename T, int VN, int VPL>
__device__ __forceinline__ void load_row_all_lanes(RowSet<T, VN, VPL, 1> &dst, const T *__restrict__ src,
                                                   int64_t row, int C, int nvec, int lane) {
#pragma unroll
  for (int j = 0; j < VPL; ++j) {
    const int idx = lane + kWave * j;
    dst.v[0][j] = load_raw<T, VN>(src + row * C + (int64_t)(idx < nvec ? idx : nvec - 1) * VN);
  }
}
template <typename T, int VN, int VPL>
__device__ __forceinline__ void zero_past_row(RowSet<T, VN, VPL, 1> &r, int nvec, int lane) {
#pragma unroll
  for (int j = 0; j < VPL; ++j) {
    const bool past = lane + kWave * j >= nvec;
#pragma unroll
    for (int q = 0; q < VN / Vec16<T>::n; ++q) {
      u32x4 w = __builtin_bit_cast(u32x4, r.v[0][j].v[q]);
      w.x = past ? 0u : w.x;
      w.y = past ? 0u : w.y;
      w.z = past ? 0u : w.z;
      w.w = past ? 0u : w.w;
      r.v[0][j].v[q] = __builtin_bit_cast(Vec16<T>, w);
    }
  }
}

// HAS_RES: the rows that are normalised are x + residual, rounded to x's type (the sum is also
// written to sum_out, which may be x or residual itself): the residual add in front of the
// LayerNorm of a transformer block without a [rows, C] round trip between two launches.
template <typename TX, typename TY, typename TP, int VPL, int R, bool PF, bool HAS_RES, int LPR = kWave>
__global__ __launch_bounds__(kLnThreads) void ln_fwd_rows_kernel(
    const TX *x /* sum_out may be x: not restrict */, const TP *__restrict__ gamma, const TP *__restrict__ beta,
    TY *__restrict__ y, float *__restrict__ mean, float *__restrict__ rstd, int64_t rows, int C,
    float eps, const TX *res, TX *sum_out) {
  constexpr int VN = Vec16<TX>::n;
  constexpr int RPW = kWave / LPR;  // rows side by side in a wave: R * RPW rows per wave and step
  const int lane = threadIdx.x & (kWave - 1);
  const int sub = lane / LPR, hl = lane % LPR;
  const bool upper = sub != 0;
  const int64_t gw = (int64_t)blockIdx.x * (kLnThreads / kWave) + (threadIdx.x >> 6);
  const int64_t step = (int64_t)gridDim.x * (kLnThreads / kWave) * R * RPW;
  const int nvec = C / VN;
  int64_t row0 = gw * R * RPW;
  if (row0 >= rows) return;  // wave-uniform

  RowSet<TX, VN, VPL, R> cur, rcur;
  if constexpr (PF) {
    load_rows<TX, VN, VPL, R, LPR>(cur, x, row0, rows, C, nvec, lane);
    if constexpr (HAS_RES) load_rows<TX, VN, VPL, R, LPR>(rcur, res, row0, rows, C, nvec, lane);
  }
  float g[VPL][VN], b[VPL][VN];
#pragma unroll
  for (int j = 0; j < VPL; ++j) {
    const int idx = hl + LPR * j;
#pragma unroll
    for (int k = 0; k < VN; ++k) {
      g[j][k] = 0.f;
      b[j][k] = 0.f;
    }
    if (idx < nvec) {
      load_n<TP, VN>(gamma + idx * VN, g[j]);
      if (beta) load_n<TP, VN>(beta + idx * VN, b[j]);
    }
  }
  const float inv_c = 1.0f / (float)C;
  for (; row0 < rows; row0 += step) {
    RowSet<TX, VN, VPL, R> nxt, rnxt;
    if constexpr (PF) {
      if (row0 + step < rows) {
        load_rows<TX, VN, VPL, R, LPR>(nxt, x, row0 + step, rows, C, nvec, lane);
        if constexpr (HAS_RES) load_rows<TX, VN, VPL, R, LPR>(rnxt, res, row0 + step, rows, C, nvec, lane);
      }
    } else {
      load_rows<TX, VN, VPL, R, LPR>(cur, x, row0, rows, C, nvec, lane);
      if constexpr (HAS_RES) load_rows<TX, VN, VPL, R, LPR>(rcur, res, row0, rows, C, nvec, lane);
    }
    if constexpr (HAS_RES) {
      // cur = x + residual, one fp32 add and one rounding per element, as an add launch would give
#pragma unroll
      for (int r = 0; r < R; ++r) {
#pragma unroll
        for (int j = 0; j < VPL; ++j) {
          Vec16<TX> sum;
#pragma unroll
          for (int k = 0; k < VN; ++k)
            sum.e[k] = from_acc<TX>(raw_get<TX, VN>(cur.v[r][j], k) + raw_get<TX, VN>(rcur.v[r][j], k));
          cur.v[r][j].v[0] = sum;
          const int idx = hl + LPR * j;
          const int64_t row = row0 + r * RPW + sub;
          if (idx < nvec && row < rows) store16_stream(sum_out + row * C + (int64_t)idx * VN, sum);
        }
      }
    }
    // the R rows are independent: their reductions interleave
    float mu[R], rs[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float s = 0.f;
#pragma unroll
      for (int j = 0; j < VPL; ++j)
#pragma unroll
        for (int k = 0; k < VN; ++k) s += raw_get<TX, VN>(cur.v[r][j], k);
      mu[r] = s;
    }
#pragma unroll
    for (int r = 0; r < R; ++r) mu[r] = row_lanes_sum<LPR>(mu[r], upper) * inv_c;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float q = 0.f;
#pragma unroll
      for (int j = 0; j < VPL; ++j) {
        if (hl + LPR * j < nvec) {
#pragma unroll
          for (int k = 0; k < VN; ++k) {
            const float d = raw_get<TX, VN>(cur.v[r][j], k) - mu[r];
            q += d * d;
          }
        }
      }
      rs[r] = q;
    }
#pragma unroll
    for (int r = 0; r < R; ++r) rs[r] = 1.0f / sqrtf(row_lanes_sum<LPR>(rs[r], upper) * inv_c + eps);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      if (row0 + r * RPW >= rows) break;  // wave-uniform
      const int64_t row = row0 + r * RPW + sub;
      const bool row_ok = row < rows;
      if (hl == 0 && row_ok) {
        mean[row] = mu[r];
        rstd[row] = rs[r];
      }
#pragma unroll
      for (int j = 0; j < VPL; ++j) {
        const int idx = hl + LPR * j;
        if (idx < nvec && row_ok) {
          float o[VN];
#pragma unroll
          for (int k = 0; k < VN; ++k)
            o[k] = (raw_get<TX, VN>(cur.v[r][j], k) - mu[r]) * rs[r] * g[j][k] + b[j][k];
          store_n<TY, VN>(y + row * C + (int64_t)idx * VN, o);
        }
      }
    }
    if constexpr (PF) {
      cur = nxt;
      if constexpr (HAS_RES) rcur = rnxt;
    }
  }
}

// ------------------------------------------------- column sums of partial rows
// What a launch of the row kernel may do on the side: the column sums of an EARLIER call's partial
// rows (written by a launch that is complete when this one starts).  The first `blocks`
// workgroups of the grid do that and leave; the row work starts at workgroup `blocks`.
struct LnPending {
  const float *partial;  // nullptr: nothing pending
  void *dgamma, *dbeta;  // of the earlier call; either may be nullptr
  int nparts, accumulate, blocks;
};

// Adds `nparts` partial rows in a fixed order.  Partial rows are permuted: position
// p = k*nvec + idx holds column idx*vn + k (nvec = C/vn).  One tile = 32 positions of dgamma or
// dbeta: thread (cx, ry) of 32 x 16 sums partial rows ry, ry+16, ... for one position, sixteen
// loads in flight and none of them under a condition (this work waits for a row kernel and is all
// latency), then row 0 adds the 16 sub-sums in order.  `sub` is 16 x 32 floats of LDS.
constexpr int kLnFinCols = 32, kLnFinRows = 16, kLnFinInFlight = 16;

template <typename TP, int THREADS = kLnFinCols * kLnFinRows>
__device__ __forceinline__ void ln_finalize_tile(const float *__restrict__ partial, int nparts, TP *__restrict__ out,
                                                 int which, int tile, int C, int vn, int accumulate, float *sub,
                                                 int tid) {
  static_assert(THREADS >= kLnFinCols * kLnFinRows, "a tile takes 512 threads; further ones only join the barrier");
  const int cx = tid % kLnFinCols, ry = tid / kLnFinCols;
  const int col = tile * kLnFinCols + cx;  // a position in the permuted row
  float s = 0.f;
  if (col < C && ry < kLnFinRows) {
    const float *src = partial + (int64_t)which * C + col;
    const int64_t stride = 2 * (int64_t)C;
    for (int p0 = ry; p0 < nparts; p0 += kLnFinRows * kLnFinInFlight) {
      float v[kLnFinInFlight];
#pragma unroll
      for (int u = 0; u < kLnFinInFlight; ++u) {
        const int p = p0 + u * kLnFinRows;
        v[u] = src[(int64_t)(p < nparts ? p : nparts - 1) * stride];
      }
#pragma unroll
      for (int u = 0; u < kLnFinInFlight; ++u) s += p0 + u * kLnFinRows < nparts ? v[u] : 0.f;
    }
  }
  if (ry < kLnFinRows) sub[ry * kLnFinCols + cx] = s;
  __syncthreads();
  if (ry == 0 && col < C) {
    float t = 0.f;
#pragma unroll
    for (int r = 0; r < kLnFinRows; ++r) t += sub[r * kLnFinCols + cx];
    const int nvec = C / vn;
    const int real = (col % nvec) * vn + col / nvec;  // the column this position stands for
    if (accumulate) t += to_acc(out[real]);
    out[real] = from_acc<TP>(t);
  }
}
// workgroup b of the 2 * ceil(C/32) that cover a pending call: even b dgamma, odd b dbeta
template <typename TP, int THREADS = kLnFinCols * kLnFinRows>
__device__ __forceinline__ void ln_finalize_pending(const LnPending &pend, int b, int C, int vn, float *sub, int tid) {
  const int which = b & 1;
  TP *out = (TP *)(which == 0 ? pend.dgamma : pend.dbeta);
  if (out == nullptr) return;  // block-uniform
  ln_finalize_tile<TP, THREADS>(pend.partial, pend.nparts, out, which, b >> 1, C, vn, pend.accumulate, sub, tid);
}

// ----------------------------------------------------------- fast backward
// One wave per row, the row (dy and x) in registers, gamma and the per-column partial sums in
// registers for all rows a wave visits (rows gw, gw + n_waves, ...).  No software prefetch:
// WPE waves per SIMD are resident (the launch bound asks the compiler for that), so while one
// wave waits for its row the others compute; measured on MI355X this beats two rows per wave
// with the next step's rows prefetched ([8192,768] bf16: 12.3 -> 9.8 us, [16384,1600]: 32.8 ->
// 30.3 us) because twice as many waves are in flight with half the registers each.
// The arithmetic uses explicit fused multiply-adds (contraction is off in this file, so every
// variant of the kernel rounds alike): 17 VALU operations per element instead of 27, which
// matters because at 16-bit storage this kernel is as close to its VALU limit as to HBM's.
// HAS_DRES: dx_out = dx + dresidual, the gradient add that follows LayerNorm::backward on the
// residual stream; dx is rounded to its type first, then the sum, as two kernels would.  Only
// instantiated for the 2-vectors-per-lane plan: wider rows have no registers left for a third
// input, and there the add runs as its own launch.
template <typename TDY, typename TX, typename TDX, typename TP, int VPL, int WPE, bool HAS_DX,
          bool HAS_DP, bool HAS_DRES>
__global__ __launch_bounds__(kLnBwdThreads, WPE) void ln_bwd_rows_kernel(
    const TDY *__restrict__ dy, const TX *__restrict__ x, const float *__restrict__ mean,
    const float *__restrict__ rstd, const TP *__restrict__ gamma, TDX *dx,
    float *__restrict__ partial, int64_t rows, int C, const TDX *dres /* dx may be dres */,
    const LnPending pend) {
  constexpr int VN = Vec16<TX>::n;
  extern __shared__ float lds[];  // [waves per block][C], at least 16 x 32 floats with pending sums
  if ((int)blockIdx.x < pend.blocks) {
    ln_finalize_pending<TP>(pend, blockIdx.x, C, VN, lds, threadIdx.x);
    return;
  }
  const int bid = blockIdx.x - pend.blocks;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  constexpr int kWaves = kLnBwdThreads / kWave;
  const int64_t step = (int64_t)(gridDim.x - pend.blocks) * kWaves;
  const int nvec = C / VN;
  const float inv_c = 1.0f / (float)C;

  float acc_g[VPL][VN], acc_b[VPL][VN], g[VPL][VN];
#pragma unroll
  for (int j = 0; j < VPL; ++j) {
#pragma unroll
    for (int k = 0; k < VN; ++k) {
      acc_g[j][k] = 0.f;
      acc_b[j][k] = 0.f;
      g[j][k] = 0.f;
    }
    if (HAS_DX && lane + kWave * j < nvec) load_n<TP, VN>(gamma + (lane + kWave * j) * VN, g[j]);
  }

  for (int64_t row = (int64_t)bid * kWaves + wave; row < rows; row += step) {
    RowSet<TDY, VN, VPL, 1> dcur;
    RowSet<TX, VN, VPL, 1> xcur;
    RowSet<TDX, VN, VPL, 1> rcur;  // this row of dresidual, in flight during the reductions
    if constexpr (HAS_DRES) {
      // three inputs: with loads under the lane's own condition the compiler waits for each
      // piece of the third before it issues the next (two extra round trips per row at
      // [8192,768]: 21.0 -> 19.7 us, 53.1 -> 46.4 us at [16384,1600]); every lane loads instead
      load_row_all_lanes<TDY, VN, VPL>(dcur, dy, row, C, nvec, lane);
      load_row_all_lanes<TX, VN, VPL>(xcur, x, row, C, nvec, lane);
      load_row_all_lanes<TDX, VN, VPL>(rcur, dres, row, C, nvec, lane);
      zero_past_row<TDY, VN, VPL>(dcur, nvec, lane);  // so that lanes past the row add nothing below
    } else {
      // two inputs: the conditional form has no such waits and needs half the registers
      // (13.9 against 14.8 us, 34.0 against 36.4 us)
      load_rows<TDY, VN, VPL, 1>(dcur, dy, row, rows, C, nvec, lane);
      load_rows<TX, VN, VPL, 1>(xcur, x, row, rows, C, nvec, lane);
    }
    const float mu = mean[row], rs = rstd[row];
    float s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
#pragma unroll
      for (int k = 0; k < VN; ++k) {
        // lanes past the row hold zeros in dy, so they add nothing
        const float xh = (raw_get<TX, VN>(xcur.v[0][j], k) - mu) * rs;
        const float dv = raw_get<TDY, VN>(dcur.v[0][j], k);
        if constexpr (HAS_DP) {
          acc_g[j][k] = __builtin_fmaf(dv, xh, acc_g[j][k]);
          acc_b[j][k] += dv;
        }
        if constexpr (HAS_DX) {
          const float gd = dv * g[j][k];
          s1 += gd;
          s2 = __builtin_fmaf(gd, xh, s2);
        }
      }
    }
    if constexpr (HAS_DX) {
      s1 = wave_reduce(s1, SumOp{}) * inv_c;
      s2 = wave_reduce(s2, SumOp{}) * inv_c;
      // x-hat and dy are unpacked again from the packed row rather than kept as floats across
      // the reduction: half the registers, a few more VALU ops
#pragma unroll
      for (int j = 0; j < VPL; ++j) {
        forget_unpacked(xcur.v[0][j]);
        forget_unpacked(dcur.v[0][j]);
        // also keeps the load of this piece up where it was issued: without a use outside the
        // branch below the compiler moves it into the branch, behind the reductions
        if constexpr (HAS_DRES) forget_unpacked(rcur.v[0][j]);
        const int idx = lane + kWave * j;
        if (idx < nvec) {
          float o[VN];
#pragma unroll
          for (int k = 0; k < VN; ++k) {
            const float xh = (raw_get<TX, VN>(xcur.v[0][j], k) - mu) * rs;
            const float dv = raw_get<TDY, VN>(dcur.v[0][j], k);
            // rstd * (dy gamma - mean(dy gamma) - xhat mean(dy gamma xhat))
            o[k] = rs * __builtin_fmaf(-xh, s2, __builtin_fmaf(dv, g[j][k], -s1));
            if constexpr (HAS_DRES)
              o[k] = round_through<TDX>(o[k]) + raw_get<TDX, VN>(rcur.v[0][j], k);
          }
          store_n<TDX, VN>(dx + row * C + (int64_t)idx * VN, o);
        }
      }
    }
  }

  if constexpr (HAS_DP) {
    // fold the block's waves, dgamma first, then dbeta through the same LDS.  Column
    // idx*VN + k is kept at position k*nvec + idx, in the LDS and in the partial rows: lanes
    // then write consecutive words (no bank conflicts); the last kernel undoes the permutation.
#pragma unroll
    for (int which = 0; which < 2; ++which) {
#pragma unroll
      for (int j = 0; j < VPL; ++j) {
        const int idx = lane + kWave * j;
        if (idx < nvec) {
#pragma unroll
          for (int k = 0; k < VN; ++k)
            lds[wave * C + k * nvec + idx] = which == 0 ? acc_g[j][k] : acc_b[j][k];
        }
      }
      __syncthreads();
      for (int c = threadIdx.x; c < C; c += kLnBwdThreads) {
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) s += lds[w * C + c];
        partial[((int64_t)bid * 2 + which) * C + c] = s;
      }
      __syncthreads();
    }
  }
}

// --------------------------------- rows on whole waves or on halves of a wave
// LPR lanes per row: 64 (a wave per row) or 32: two rows per wave, side by side, lanes 0-31 on row
// 2p, lanes 32-63 on row 2p + 1, for rows of at most 32 * VPL vectors.  A 768-column row of 16-bit
// data is 96 vectors = 32 lanes x 3, so every lane slot is used (on whole waves it takes two
// vectors per lane and leaves a quarter of them empty), a wave finishes two rows per round trip to
// memory, and the same number of waves leaves half as many rows behind them.  The two row sums
// are reduced per half; the column sums of the halves meet in the LDS fold at the end.
template <typename T, int VN, int VPL>
struct Strip {
  Raw<T, VN> v[VPL];
};
// every lane loads (from the last vector of the row again where it has none of its own)
template <typename T, int VN, int VPL, int LPR>
__device__ __forceinline__ void load_strip(Strip<T, VN, VPL> &dst, const T *src, int64_t row, int C, int nvec,
                                           int hl) {
#pragma unroll
  for (int j = 0; j < VPL; ++j) {
    const int idx = hl + LPR * j;
    dst.v[j] = load_raw<T, VN>(src + row * C + (int64_t)(idx < nvec ? idx : nvec - 1) * VN);
  }
}
template <typename T, int VN, int VPL, int LPR>
__device__ __forceinline__ void zero_strip_unless(Strip<T, VN, VPL> &r, bool row_ok, int nvec, int hl) {
#pragma unroll
  for (int j = 0; j < VPL; ++j) {
    const bool keep = row_ok && hl + LPR * j < nvec;
#pragma unroll
    for (int q = 0; q < VN / Vec16<T>::n; ++q) {
      u32x4 w = __builtin_bit_cast(u32x4, r.v[j].v[q]);
      w.x = keep ? w.x : 0u;
      w.y = keep ? w.y : 0u;
      w.z = keep ? w.z : 0u;
      w.w = keep ? w.w : 0u;
      r.v[j].v[q] = __builtin_bit_cast(Vec16<T>, w);
    }
  }
}

#ifndef CS_LN_PAIR_FOLD
#define CS_LN_PAIR_FOLD 1
#endif

// PF: the next step's rows are requested before the current ones are worked on.
// KEEP: x-hat and dy*gamma stay unpacked across the two row sums instead of being unpacked and
// normalised again for the second pass (at 16-bit storage the kernel is as close to the VALU
// limit as to the memory's); takes VPL * 2 * VN more registers.
template <typename TDY, typename TX, typename TDX, typename TP, int THREADS, int LPR, int VPL, int WPE, bool PF,
          bool KEEP,
          bool HAS_DX, bool HAS_DP, bool HAS_DRES>
__global__ __launch_bounds__(THREADS, WPE) void ln_bwd_kernel(
    const TDY *__restrict__ dy, const TX *__restrict__ x, const float *__restrict__ mean,
    const float *__restrict__ rstd, const TP *__restrict__ gamma, TDX *dx /* may be dres */,
    float *__restrict__ partial, int64_t rows, int C, const TDX *dres, const LnPending pend) {
  constexpr int VN = Vec16<TX>::n;
  constexpr int RPW = kWave / LPR;  // rows a wave works on side by side
  extern __shared__ float lds[];    // [RPW * waves per block][C], at least 16 x 32 floats
  if ((int)blockIdx.x < pend.blocks) {
    ln_finalize_pending<TP, THREADS>(pend, blockIdx.x, C, VN, lds, threadIdx.x);
    return;
  }
  const int bid = blockIdx.x - pend.blocks, nblocks = gridDim.x - pend.blocks;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  const bool upper = LPR == kHalf && lane >= kHalf;
  const int hl = lane & (LPR - 1);
  constexpr int kWaves = THREADS / kWave;
  const int64_t step = (int64_t)nblocks * kWaves;
  const int64_t nsteps = (rows + RPW - 1) / RPW;  // row groups: one per wave and step
  const int nvec = C / VN;
  const float inv_c = 1.0f / (float)C;

  float acc_g[VPL][VN], acc_b[VPL][VN], g[VPL][VN];
#pragma unroll
  for (int j = 0; j < VPL; ++j) {
    const int idx = hl + LPR * j;
#pragma unroll
    for (int k = 0; k < VN; ++k) {
      acc_g[j][k] = 0.f;
      acc_b[j][k] = 0.f;
    }
    if constexpr (HAS_DX) load_n<TP, VN>(gamma + (idx < nvec ? idx : nvec - 1) * VN, g[j]);
  }

  Strip<TDY, VN, VPL> dcur, dnxt;
  Strip<TX, VN, VPL> xcur, xnxt;
  Strip<TDX, VN, VPL> rcur, rnxt;  // this row of dresidual, in flight during the reductions
  float mu = 0.f, rs = 0.f, nmu = 0.f, nrs = 0.f;
  int64_t p = (int64_t)bid * kWaves + wave;
  auto issue = [&](int64_t p_, Strip<TDY, VN, VPL> &d, Strip<TX, VN, VPL> &xx, Strip<TDX, VN, VPL> &rr, float &m_,
                   float &r_) {
    const int64_t row = RPW * p_ + (upper ? 1 : 0);
    const int64_t rowc = row < rows ? row : rows - 1;
    load_strip<TDY, VN, VPL, LPR>(d, dy, rowc, C, nvec, hl);
    load_strip<TX, VN, VPL, LPR>(xx, x, rowc, C, nvec, hl);
    if constexpr (HAS_DRES) load_strip<TDX, VN, VPL, LPR>(rr, dres, rowc, C, nvec, hl);
    m_ = mean[rowc];
    r_ = rstd[rowc];
  };
  if constexpr (PF) {
    if (p < nsteps) issue(p, dcur, xcur, rcur, mu, rs);
  }
  for (; p < nsteps; p += step) {
    if constexpr (PF) {
      if (p + step < nsteps) issue(p + step, dnxt, xnxt, rnxt, nmu, nrs);
    } else {
      issue(p, dcur, xcur, rcur, mu, rs);
    }
    const int64_t row = RPW * p + (upper ? 1 : 0);
    const bool row_ok = row < rows;
    zero_strip_unless<TDY, VN, VPL, LPR>(dcur, row_ok, nvec, hl);  // lanes without data add nothing below
    float s1 = 0.f, s2 = 0.f;
    float xh[KEEP ? VPL : 1][VN], gd[KEEP ? VPL : 1][VN];
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
      const int jj = KEEP ? j : 0;
#pragma unroll
      for (int k = 0; k < VN; ++k) {
        xh[jj][k] = (raw_get<TX, VN>(xcur.v[j], k) - mu) * rs;
        const float dv = raw_get<TDY, VN>(dcur.v[j], k);
        if constexpr (HAS_DP) {
          acc_g[j][k] = __builtin_fmaf(dv, xh[jj][k], acc_g[j][k]);
          acc_b[j][k] += dv;
        }
        if constexpr (HAS_DX) {
          gd[jj][k] = dv * g[j][k];
          s1 += gd[jj][k];
          s2 = __builtin_fmaf(gd[jj][k], xh[jj][k], s2);
        }
      }
    }
    if constexpr (HAS_DX) {
      // rstd * (dy gamma - mean(dy gamma) - xhat mean(dy gamma xhat)) with the row's three
      // factors folded first: two operations per element
      const float cb = -(row_lanes_sum<LPR>(s1, upper) * inv_c) * rs;
      const float cc = -(row_lanes_sum<LPR>(s2, upper) * inv_c) * rs;
#pragma unroll
      for (int j = 0; j < VPL; ++j) {
        const int jj = KEEP ? j : 0;
        if constexpr (!KEEP) {
          // unpacked again from the packed row rather than kept as floats across the reduction
          forget_unpacked(xcur.v[j]);
          forget_unpacked(dcur.v[j]);
        }
        if constexpr (HAS_DRES) forget_unpacked(rcur.v[j]);  // keeps its load where it was issued
        const int idx = hl + LPR * j;
        float o[VN];
#pragma unroll
        for (int k = 0; k < VN; ++k) {
          if constexpr (!KEEP) {
            xh[jj][k] = (raw_get<TX, VN>(xcur.v[j], k) - mu) * rs;
            gd[jj][k] = raw_get<TDY, VN>(dcur.v[j], k) * g[j][k];
          }
          o[k] = __builtin_fmaf(xh[jj][k], cc, __builtin_fmaf(gd[jj][k], rs, cb));
          if constexpr (HAS_DRES) o[k] = round_through<TDX>(o[k]) + raw_get<TDX, VN>(rcur.v[j], k);
        }
        if (row_ok && idx < nvec) store_n<TDX, VN>(dx + row * C + (int64_t)idx * VN, o);
      }
    }
    if constexpr (PF) {
      dcur = dnxt;
      xcur = xnxt;
      if constexpr (HAS_DRES) rcur = rnxt;
      mu = nmu;
      rs = nrs;
    }
  }

#if CS_LN_PAIR_FOLD <= 0
  if constexpr (HAS_DP) {
    float t = 0.f;
#pragma unroll
    for (int j = 0; j < VPL; ++j)
#pragma unroll
      for (int k = 0; k < VN; ++k) t += acc_g[j][k] * acc_b[j][k];
    if (t == 12345.678f) partial[threadIdx.x] = t;
  }
#endif
  if constexpr (HAS_DP && CS_LN_PAIR_FOLD > 0) {
    // Fold the block's waves (half-waves), dgamma first, then dbeta through the same LDS.  Column
    // idx*VN + k is kept at position k*nvec + idx, in the LDS and in the partial rows: lanes
    // then write consecutive words (no bank conflicts); the finalize step undoes the permutation.
    // (Measured against 16-byte LDS writes in a layout that suits them, with 16-byte or 4-byte
    // reads: 0.3-0.9 us slower per launch at [8192,768] than these 4-byte accesses.)
    const int hw = wave * RPW + (upper ? 1 : 0);
#pragma unroll
    for (int which = 0; which < 2; ++which) {
#pragma unroll
      for (int j = 0; j < VPL; ++j) {
        const int idx = hl + LPR * j;
        if (idx < nvec) {
#pragma unroll
          for (int k = 0; k < VN; ++k) lds[hw * C + k * nvec + idx] = which == 0 ? acc_g[j][k] : acc_b[j][k];
        }
      }
      lds_barrier();
      for (int c = threadIdx.x; c < C; c += THREADS) {
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < RPW * kWaves; ++w) s += lds[w * C + c];
        partial[((int64_t)bid * 2 + which) * C + c] = s;
      }
      if (which == 0) lds_barrier();
    }
  }
}

// ------------------------------------------------- wide rows: two waves per row
// Rows of 5 to 8 vectors per lane do not fit one wave's registers once the dgamma/dbeta
// accumulators are there, so a pair of waves shares a row: wave h of the pair (h = 0, 1) owns
// vectors lane + 64*(2j + h), j < VPLH.  The two halves of the row sums meet in the LDS (one
// barrier per row; every pair makes the same number of steps so that all waves reach it).
template <typename T, int VN, int VPLH>
struct HalfRow {
  Raw<T, VN> v[VPLH];
};
template <typename T, int VN, int VPLH>
__device__ __forceinline__ void load_half_row(HalfRow<T, VN, VPLH> &dst, const T *__restrict__ src,
                                              int64_t row, bool valid, int C, int nvec, int lane, int h) {
#pragma unroll
  for (int j = 0; j < VPLH; ++j) {
    const int idx = lane + kWave * (2 * j + h);
    if (valid && idx < nvec) {
      dst.v[j] = load_raw<T, VN>(src + row * C + (int64_t)idx * VN);
    } else {
      dst.v[j] = zero_raw<T, VN>();
    }
  }
}

template <typename TDY, typename TX, typename TDX, typename TP, int VPLH, bool HAS_DX, bool HAS_DP>
__global__ __launch_bounds__(kLnBwdThreads) void ln_bwd_split_rows_kernel(
    const TDY *__restrict__ dy, const TX *__restrict__ x, const float *__restrict__ mean,
    const float *__restrict__ rstd, const TP *__restrict__ gamma, TDX *__restrict__ dx,
    float *__restrict__ partial, int64_t rows, int C) {
  constexpr int VN = Vec16<TX>::n;
  constexpr int kWaves = kLnBwdThreads / kWave;
  constexpr int kPairs = kWaves / 2;
  constexpr int kRegion = VPLH * kWave * VN;  // floats one wave contributes to the fold
  extern __shared__ float lds[];              // [kPairs][kRegion], one half of the row at a time
  __shared__ float halves[2][kPairs][2][2];   // [parity][pair][half][s1, s2]
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  const int pair = wave >> 1, h = wave & 1;
  const int64_t n_pairs = (int64_t)gridDim.x * kPairs;
  const int64_t gp = (int64_t)blockIdx.x * kPairs + pair;
  const int64_t steps = (rows + n_pairs - 1) / n_pairs;  // the same for every pair
  const int nvec = C / VN;
  const float inv_c = 1.0f / (float)C;

  float acc_g[VPLH][VN], acc_b[VPLH][VN], g[VPLH][VN];
#pragma unroll
  for (int j = 0; j < VPLH; ++j) {
    const int idx = lane + kWave * (2 * j + h);
#pragma unroll
    for (int k = 0; k < VN; ++k) {
      acc_g[j][k] = 0.f;
      acc_b[j][k] = 0.f;
      g[j][k] = 0.f;
    }
    if (HAS_DX && idx < nvec) load_n<TP, VN>(gamma + idx * VN, g[j]);
  }

  HalfRow<TDY, VN, VPLH> dcur;
  HalfRow<TX, VN, VPLH> xcur;
  int64_t row = gp;
  load_half_row<TDY, VN, VPLH>(dcur, dy, row, row < rows, C, nvec, lane, h);
  load_half_row<TX, VN, VPLH>(xcur, x, row, row < rows, C, nvec, lane, h);
  float mu = row < rows ? mean[row] : 0.f, rs = row < rows ? rstd[row] : 0.f;
  int parity = 0;
  for (int64_t it = 0; it < steps; ++it, row += n_pairs) {
    const int64_t nrow = row + n_pairs;
    HalfRow<TDY, VN, VPLH> dnxt;
    HalfRow<TX, VN, VPLH> xnxt;
    load_half_row<TDY, VN, VPLH>(dnxt, dy, nrow, nrow < rows, C, nvec, lane, h);
    load_half_row<TX, VN, VPLH>(xnxt, x, nrow, nrow < rows, C, nvec, lane, h);
    const float nmu = nrow < rows ? mean[nrow] : 0.f, nrs = nrow < rows ? rstd[nrow] : 0.f;

    // a row past the end is all zeros here: it adds nothing and stores nothing
    float s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int j = 0; j < VPLH; ++j) {
#pragma unroll
      for (int k = 0; k < VN; ++k) {
        const float xh = (raw_get<TX, VN>(xcur.v[j], k) - mu) * rs;
        const float dv = raw_get<TDY, VN>(dcur.v[j], k);
        if constexpr (HAS_DP) {
          acc_g[j][k] = __builtin_fmaf(dv, xh, acc_g[j][k]);
          acc_b[j][k] += dv;
        }
        if constexpr (HAS_DX) {
          const float gd = dv * g[j][k];
          s1 += gd;
          s2 = __builtin_fmaf(gd, xh, s2);
        }
      }
    }
    if constexpr (HAS_DX) {
      s1 = wave_reduce(s1, SumOp{});
      s2 = wave_reduce(s2, SumOp{});
      if (lane == 0) {
        halves[parity][pair][h][0] = s1;
        halves[parity][pair][h][1] = s2;
      }
      __syncthreads();
      // both waves of the pair add the halves in the same order
      s1 = (halves[parity][pair][0][0] + halves[parity][pair][1][0]) * inv_c;
      s2 = (halves[parity][pair][0][1] + halves[parity][pair][1][1]) * inv_c;
      parity ^= 1;  // the other buffer next step: one barrier per row is enough
      if (row < rows) {
#pragma unroll
        for (int j = 0; j < VPLH; ++j) {
          forget_unpacked(xcur.v[j]);
          forget_unpacked(dcur.v[j]);
          const int idx = lane + kWave * (2 * j + h);
          if (idx < nvec) {
            float o[VN];
#pragma unroll
            for (int k = 0; k < VN; ++k) {
              const float xh = (raw_get<TX, VN>(xcur.v[j], k) - mu) * rs;
              const float dv = raw_get<TDY, VN>(dcur.v[j], k);
              o[k] = rs * __builtin_fmaf(-xh, s2, __builtin_fmaf(dv, g[j][k], -s1));
            }
            store_n<TDX, VN>(dx + row * C + (int64_t)idx * VN, o);
          }
        }
      }
    }
    dcur = dnxt;
    xcur = xnxt;
    mu = nmu;
    rs = nrs;
  }

  if constexpr (HAS_DP) {
    // fold the four waves that own the same half, one half at a time; positions inside a wave's
    // region are k*(64 VPLH) + lane + 64 j (conflict-free writes); the partial rows use the
    // permuted layout of the narrow kernel, position k*nvec + idx for column idx*VN + k
#pragma unroll
    for (int which = 0; which < 2; ++which) {
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        if (h == hh) {
#pragma unroll
          for (int j = 0; j < VPLH; ++j)
#pragma unroll
            for (int k = 0; k < VN; ++k)
              lds[pair * kRegion + k * (kWave * VPLH) + lane + kWave * j] = which == 0 ? acc_g[j][k] : acc_b[j][k];
        }
        __syncthreads();
        for (int local = threadIdx.x; local < kRegion; local += kLnBwdThreads) {
          const int k = local / (kWave * VPLH), li = local % (kWave * VPLH);
          const int idx = (li % kWave) + kWave * (2 * (li / kWave) + hh);
          if (idx < nvec) {
            float sum = 0.f;
#pragma unroll
            for (int pp = 0; pp < kPairs; ++pp) sum += lds[pp * kRegion + local];
            partial[((int64_t)blockIdx.x * 2 + which) * C + k * nvec + idx] = sum;
          }
        }
        __syncthreads();
      }
    }
  }
}

// The column sums as a launch of their own: grid 2 * ceil(C/32) workgroups of 32 x 16 threads, even
// ones dgamma, odd ones dbeta (the same tiles, in the same order of additions, as the pending
// form inside the row kernel's launch).
template <typename TP>
__global__ __launch_bounds__(kLnFinCols *kLnFinRows) void ln_bwd_finalize_kernel(
    const float *__restrict__ partial, int nparts, TP *__restrict__ dgamma, TP *__restrict__ dbeta,
    int C, int vn, int accumulate) {
  __shared__ float sub[kLnFinRows * kLnFinCols];
  const LnPending pend{partial, dgamma, dbeta, nparts, accumulate, (int)gridDim.x};
  ln_finalize_pending<TP>(pend, blockIdx.x, C, vn, sub, threadIdx.x);
}

// ------------------------------------------------------ elementwise add
// out = a + b, one fp32 (fp64) add and one rounding per element; out may be a or b.
constexpr int kAddUnroll = 2;  // 16-byte vectors per lane, all requested before the first use

template <typename T>
__global__ __launch_bounds__(kLnThreads) void ew_add_kernel(const T *a, const T *b, T *out, int64_t n,
                                                            bool vec_ok) {
  constexpr int VN = Vec16<T>::n;
  using U = typename Acc<T>::type;
  constexpr int64_t kChunk = (int64_t)kLnThreads * kAddUnroll * VN;
  const int64_t begin = (int64_t)blockIdx.x * kChunk;
  const int64_t end = begin + kChunk < n ? begin + kChunk : n;
  if (vec_ok && end - begin == kChunk) {
    Vec16<T> va[kAddUnroll], vb[kAddUnroll];
#pragma unroll
    for (int u = 0; u < kAddUnroll; ++u) {
      const int64_t off = begin + ((int64_t)u * kLnThreads + threadIdx.x) * VN;
      va[u] = load16_stream(a + off);
      vb[u] = load16_stream(b + off);
    }
#pragma unroll
    for (int u = 0; u < kAddUnroll; ++u) {
      const int64_t off = begin + ((int64_t)u * kLnThreads + threadIdx.x) * VN;
      Vec16<T> vo;
#pragma unroll
      for (int k = 0; k < VN; ++k) vo.e[k] = from_acc<T>((U)(to_acc(va[u].e[k]) + to_acc(vb[u].e[k])));
      store16(out + off, vo);  // read again by the kernel that follows: keep it cached
    }
    return;
  }
  for (int64_t i = begin + threadIdx.x; i < end; i += kLnThreads)
    out[i] = from_acc<T>((U)(to_acc(a[i]) + to_acc(b[i])));
}

template <typename T>
int launch_add(const void *a, const void *b, void *out, int64_t n, hipStream_t s) {
  if (n <= 0) return CS_OK;
  const bool vec_ok = is_aligned16(a) && is_aligned16(b) && is_aligned16(out);
  const int64_t blocks = ceil_div(n, (int64_t)kLnThreads * kAddUnroll * Vec16<T>::n);
  if (blocks > 0x7fffffffLL) return CS_ERR_TOO_LARGE;
  ew_add_kernel<T><<<dim3((unsigned)blocks), dim3(kLnThreads), 0, s>>>((const T *)a, (const T *)b, (T *)out, n,
                                                                      vec_ok);
  return launch_status();
}

int launch_add_dtype(int dtype, const void *a, const void *b, void *out, int64_t n, hipStream_t s) {
  switch (dtype) {
    case CS_F32: return launch_add<float>(a, b, out, n, s);
    case CS_F64: return launch_add<double>(a, b, out, n, s);
    case CS_F16: return launch_add<f16_t>(a, b, out, n, s);
    case CS_BF16: return launch_add<bf16_t>(a, b, out, n, s);
  }
  return CS_ERR_UNSUPPORTED;
}

// ------------------------------------------------------------ general path
// One workgroup per row, any C, any alignment, fp64 included.
template <typename TX, typename TY, typename TP>
__global__ __launch_bounds__(kLnThreads) void ln_fwd_general_kernel(
    const TX *__restrict__ x, const TP *__restrict__ gamma, const TP *__restrict__ beta,
    TY *__restrict__ y, typename Acc<TX>::type *__restrict__ mean,
    typename Acc<TX>::type *__restrict__ rstd, int64_t C, typename Acc<TX>::type eps) {
  using U = typename Acc<TX>::type;
  __shared__ U scratch[kLnThreads / kWave];
  const int64_t row = blockIdx.x;
  const TX *xr = x + row * C;
  U s = 0;
  for (int64_t c = threadIdx.x; c < C; c += kLnThreads) s += to_acc(xr[c]);
  const U mu = block_reduce(s, SumOp{}, (U)0, scratch) / (U)C;
  U q = 0;
  for (int64_t c = threadIdx.x; c < C; c += kLnThreads) {
    const U d = to_acc(xr[c]) - mu;
    q += d * d;
  }
  const U var = block_reduce(q, SumOp{}, (U)0, scratch) / (U)C;
  const U rs = (U)1 / sqrt(var + eps);
  if (threadIdx.x == 0) {
    mean[row] = mu;
    rstd[row] = rs;
  }
  for (int64_t c = threadIdx.x; c < C; c += kLnThreads) {
    const U bb = beta ? (U)to_acc(beta[c]) : (U)0;
    y[row * C + c] = from_acc<TY>((U)((to_acc(xr[c]) - mu) * rs * (U)to_acc(gamma[c]) + bb));
  }
}

template <typename TDY, typename TX, typename TDX, typename TP>
__global__ __launch_bounds__(kLnThreads) void ln_bwd_dx_general_kernel(
    const TDY *__restrict__ dy, const TX *__restrict__ x,
    const typename Acc<TX>::type *__restrict__ mean,
    const typename Acc<TX>::type *__restrict__ rstd, const TP *__restrict__ gamma,
    TDX *__restrict__ dx, int64_t C, const TDX *__restrict__ dres) {
  using U = typename Acc<TX>::type;
  __shared__ U scratch[kLnThreads / kWave];
  const int64_t row = blockIdx.x;
  const U mu = mean[row], rs = rstd[row];
  U s1 = 0, s2 = 0;
  for (int64_t c = threadIdx.x; c < C; c += kLnThreads) {
    const U gd = (U)to_acc(dy[row * C + c]) * (U)to_acc(gamma[c]);
    const U xh = ((U)to_acc(x[row * C + c]) - mu) * rs;
    s1 += gd;
    s2 += gd * xh;
  }
  s1 = block_reduce(s1, SumOp{}, (U)0, scratch) / (U)C;
  s2 = block_reduce(s2, SumOp{}, (U)0, scratch) / (U)C;
  for (int64_t c = threadIdx.x; c < C; c += kLnThreads) {
    const U gd = (U)to_acc(dy[row * C + c]) * (U)to_acc(gamma[c]);
    const U xh = ((U)to_acc(x[row * C + c]) - mu) * rs;
    TDX o = from_acc<TDX>((U)(rs * (gd - s1 - xh * s2)));
    if (dres) o = from_acc<TDX>((U)(round_through<TDX>((U)to_acc(o)) + (U)to_acc(dres[row * C + c])));
    dx[row * C + c] = o;
  }
}

// grid ceil(C/64) blocks of (64, 4): thread (cx, ry) walks rows ry, ry+4, ...  A thread adds
// rows/4 terms one after the other, so the running sums are kept in double: in float the
// rounding of a sum of thousands of O(1) terms reaches several 1e-5.
template <typename TDY, typename TX, typename TP>
__global__ __launch_bounds__(256) void ln_bwd_param_general_kernel(
    const TDY *__restrict__ dy, const TX *__restrict__ x,
    const typename Acc<TX>::type *__restrict__ mean,
    const typename Acc<TX>::type *__restrict__ rstd, TP *__restrict__ dgamma,
    TP *__restrict__ dbeta, int64_t rows, int64_t C, int accumulate) {
  using U = typename Acc<TX>::type;
  __shared__ double sg[4][64], sb[4][64];
  const int64_t col = (int64_t)blockIdx.x * 64 + threadIdx.x;
  double ag = 0, ab = 0;
  if (col < C) {
    for (int64_t r = threadIdx.y; r < rows; r += 4) {
      const U d = to_acc(dy[r * C + col]);
      ag += (double)(d * (((U)to_acc(x[r * C + col]) - mean[r]) * rstd[r]));
      ab += (double)d;
    }
  }
  sg[threadIdx.y][threadIdx.x] = ag;
  sb[threadIdx.y][threadIdx.x] = ab;
  __syncthreads();
  if (threadIdx.y == 0 && col < C) {
    double tg = 0, tb = 0;
    for (int r = 0; r < 4; ++r) {
      tg += sg[r][threadIdx.x];
      tb += sb[r][threadIdx.x];
    }
    if (dgamma) {
      if (accumulate) tg += (double)to_acc(dgamma[col]);
      dgamma[col] = from_acc<TP>((typename Acc<TP>::type)tg);
    }
    if (dbeta) {
      if (accumulate) tb += (double)to_acc(dbeta[col]);
      dbeta[col] = from_acc<TP>((typename Acc<TP>::type)tb);
    }
  }
}

// ---------------------------------------------------------------- dispatch
struct FastPlan {
  int vpl = 0;       // 0: not eligible
  int fwd_rows = 1;  // rows a wave normalises per step, forward
};
// The widest plan whose backward kernel still has registers for a third input per row
// (dresidual); wider rows get dx + dresidual from a second launch.
constexpr int kMaxVplWithResidual = 4;

// x vectors per lane needed for C columns of x_dtype; the fast kernels are
// instantiated for 1, 2, 4 and 8.
FastPlan fast_plan(int64_t C, int x_dtype) {
  FastPlan p;
  const int vn = 16 / (int)dtype_size(x_dtype);
  if (x_dtype == CS_F64 || C <= 0 || C % vn != 0) return p;
  const int64_t nvec = C / vn;
  const int64_t per_lane = ceil_div(nvec, (int64_t)kWave);
  if (per_lane <= 1) {
    p.vpl = 1;
    p.fwd_rows = CS_LN_FWD_ROWS_VPL1;
  } else if (per_lane <= 2) {
    p.vpl = 2;
    p.fwd_rows = CS_LN_FWD_ROWS_VPL2;
  } else if (per_lane <= 4) {
    p.vpl = 4;
    p.fwd_rows = CS_LN_FWD_ROWS_VPL4;
  } else if (per_lane <= 8) {
    p.vpl = 8;
    p.fwd_rows = 1;
  }
  return p;
}

// Grid caps: beyond these the waves loop over rows (with prefetch) instead of
// the grid growing, which keeps the parameters in registers for many rows
// and bounds the number of partial rows the backward pass leaves behind.
#ifndef CS_LN_FWD_MAX_BLOCKS
#define CS_LN_FWD_MAX_BLOCKS 1024
#endif
constexpr int kLnFwdMaxBlocks = CS_LN_FWD_MAX_BLOCKS;
constexpr int kLnBwdMaxBlocks = CS_LN_BWD_MAX_BLOCKS;
constexpr int kLnBwdMaxBlocksNarrow = CS_LN_BWD_MAX_BLOCKS_VPL2;

int ln_blocks(int64_t rows, int rows_per_wave, int cap, int threads = kLnThreads) {
  const int64_t rows_per_block = (int64_t)(threads / kWave) * rows_per_wave;
  const int64_t b = ceil_div(rows, rows_per_block);
  return (int)(b < cap ? b : cap);
}

template <typename TX, typename TY, typename TP>
int fwd_typed(const void *x, const void *gamma, const void *beta, void *y, void *mean, void *rstd,
              int64_t rows, int64_t C, double eps, bool aligned, int x_dtype, const void *res,
              void *sum_out, hipStream_t s) {
  const FastPlan p = aligned ? fast_plan(C, x_dtype) : FastPlan{};
  if constexpr (!std::is_same_v<TX, double>) {
    if (p.vpl != 0) {
      // rows of up to 32 vectors, and of 65 to 96 (C = 768 at 16 bit), go two to a wave: no lane
      // slot stays empty
      const int64_t nvec = C / Vec16<TX>::n;
      const int half_vpl = !CS_LN_FWD_HALF ? 0 : nvec <= kHalf ? 1 : (nvec > kWave && nvec <= 3 * kHalf) ? 3 : 0;
      if (half_vpl != 0) {
        const int groups = res ? (half_vpl == 1 ? CS_LN_ADD_ROWS_H1 : CS_LN_ADD_ROWS_H3)
                               : (half_vpl == 1 ? CS_LN_FWD_ROWS_H1 : CS_LN_FWD_ROWS_H3);
        const dim3 grid((unsigned)ln_blocks(rows, 2 * groups, kLnFwdMaxBlocks)), block(kLnThreads);
#define CS_LN_FWD_H(VPL, R, HAS_RES)                                                                 \
  ln_fwd_rows_kernel<TX, TY, TP, VPL, R, CS_LN_FWD_PF, HAS_RES, kHalf><<<grid, block, 0, s>>>(       \
      (const TX *)x, (const TP *)gamma, (const TP *)beta, (TY *)y, (float *)mean, (float *)rstd, rows, \
      (int)C, (float)eps, (const TX *)res, (TX *)sum_out)
        if (res && half_vpl == 1) {
          CS_LN_FWD_H(1, CS_LN_ADD_ROWS_H1, true);
        } else if (res) {
          CS_LN_FWD_H(3, CS_LN_ADD_ROWS_H3, true);
        } else if (half_vpl == 1) {
          CS_LN_FWD_H(1, CS_LN_FWD_ROWS_H1, false);
        } else {
          CS_LN_FWD_H(3, CS_LN_FWD_ROWS_H3, false);
        }
#undef CS_LN_FWD_H
        return launch_status();
      }
      // with the residual stream a wave holds two inputs per row: half the rows per step
      const int r_rows = res ? (p.vpl == 1   ? CS_LN_ADD_ROWS_VPL1
                                : p.vpl == 2 ? CS_LN_ADD_ROWS_VPL2
                                : p.vpl == 4 ? CS_LN_ADD_ROWS_VPL4
                                             : 1)
                             : p.fwd_rows;
      const dim3 grid((unsigned)ln_blocks(rows, r_rows, kLnFwdMaxBlocks)), block(kLnThreads);
#define CS_LN_FWD(VPL, R, HAS_RES)                                                          \
  ln_fwd_rows_kernel<TX, TY, TP, VPL, R, CS_LN_FWD_PF, HAS_RES><<<grid, block, 0, s>>>(     \
      (const TX *)x, (const TP *)gamma, (const TP *)beta, (TY *)y, (float *)mean,           \
      (float *)rstd, rows, (int)C, (float)eps, (const TX *)res, (TX *)sum_out)
      if (res) {
        if (p.vpl == 1) {
          CS_LN_FWD(1, CS_LN_ADD_ROWS_VPL1, true);
        } else if (p.vpl == 2) {
          CS_LN_FWD(2, CS_LN_ADD_ROWS_VPL2, true);
        } else if (p.vpl == 4) {
          CS_LN_FWD(4, CS_LN_ADD_ROWS_VPL4, true);
        } else {
          CS_LN_FWD(8, 1, true);
        }
      } else if (p.vpl == 1) {
        CS_LN_FWD(1, CS_LN_FWD_ROWS_VPL1, false);
      } else if (p.vpl == 2) {
        CS_LN_FWD(2, CS_LN_FWD_ROWS_VPL2, false);
      } else if (p.vpl == 4) {
        CS_LN_FWD(4, CS_LN_FWD_ROWS_VPL4, false);
      } else {
        CS_LN_FWD(8, 1, false);
      }
#undef CS_LN_FWD
      return launch_status();
    }
  }
  using U = typename Acc<TX>::type;
  if (rows > 0x7fffffffLL) return CS_ERR_TOO_LARGE;
  if (res) {
    // no fast plan: the sum as its own launch, then the general kernel on it
    const int st = launch_add<TX>(x, res, sum_out, rows * C, s);
    if (st != CS_OK) return st;
    x = sum_out;
  }
  ln_fwd_general_kernel<TX, TY, TP><<<dim3((unsigned)rows), dim3(kLnThreads), 0, s>>>(
      (const TX *)x, (const TP *)gamma, (const TP *)beta, (TY *)y, (U *)mean, (U *)rstd, C,
      (U)eps);
  return launch_status();
}

// ---- backward plans.  Which row kernel takes a shape, with what launch: one function, used by
// the launches, the workspace sizes and the partial-row counts alike.
#ifndef CS_LN_PAIRS
#define CS_LN_PAIRS 1
#endif
#ifndef CS_LN_H3_ALONE_PF
#define CS_LN_H3_ALONE_PF 1
#endif
#ifndef CS_LN_H3_WPE
#define CS_LN_H3_WPE 2
#endif
#ifndef CS_LN_PAIR_PF
#define CS_LN_PAIR_PF false
#endif
#ifndef CS_LN_PAIR_KEEP
#define CS_LN_PAIR_KEEP true
#endif
#ifndef CS_LN_PAIR_MAX_BLOCKS
#define CS_LN_PAIR_MAX_BLOCKS 256
#endif
// Rows of 4 vectors per lane (the 1600-column row at 16 bit) on ln_bwd_kernel, a wave per row:
// 0 never, 1 when only dgamma/dbeta are asked for, 2 always.  Measured at [16384,1600] bf16 with
// 512 threads, against ln_bwd_rows_kernel: dgamma/dbeta alone 22.4 against 45.8 us (every lane
// loads: nothing serialises the loads), dx alone 29.0 against 28.4 us, all three 33.3 against
// 33.7 us; with the next row prefetched, or 1024 threads, the kernel spills.  The two kernels give
// the same partial rows bit for bit (same rows per wave, same order of additions).
#ifndef CS_LN_W4_NEW
#define CS_LN_W4_NEW 1
#endif
#ifndef CS_LN_W4_THREADS
#define CS_LN_W4_THREADS 512
#endif
#ifndef CS_LN_W4_WPE
#define CS_LN_W4_WPE 2
#endif
#ifndef CS_LN_W4_PF
#define CS_LN_W4_PF false
#endif
#ifndef CS_LN_W4_KEEP
#define CS_LN_W4_KEEP false
#endif
enum BwdKind {
  kBwdNone = 0,  // no row-in-registers plan: the general kernels
  kBwdHalf1,     // ln_bwd_kernel, two rows per wave, 1 vector per lane (rows of up to 32 vectors)
  kBwdHalf3,     // ln_bwd_kernel, two rows per wave, 3 vectors per lane (65 to 96 vectors: C = 768 at 16 bit)
  kBwdWave4,     // ln_bwd_kernel, a wave per row, 4 vectors per lane
  kBwdRows,      // ln_bwd_rows_kernel, 1 / 2 / 4 / 8 (no parameter gradients) vectors per lane
  kBwdSplit,     // ln_bwd_split_rows_kernel: 8 vectors per lane with parameter gradients
};
struct BwdPlan {
  BwdKind kind = kBwdNone;
  int vpl = 0;
  int threads = kLnBwdThreads;
  int blocks = 0;         // workgroups of row work = partial rows left behind when dgamma/dbeta are wanted
  size_t fold_lds = 0;    // LDS of the column-sum fold
};
constexpr int kLnMaxPartialRows = 512;
static_assert(kLnBwdMaxBlocksNarrow <= kLnMaxPartialRows && kLnBwdMaxBlocks <= kLnMaxPartialRows &&
                  CS_LN_PAIR_MAX_BLOCKS <= kLnMaxPartialRows,
              "every plan's grid cap fits the finalize step's row limit");

BwdPlan bwd_plan(int64_t rows, int64_t C, int x_dtype, bool want_dp, bool want_dx = true) {
  BwdPlan b;
  const FastPlan p = fast_plan(C, x_dtype);
  if (p.vpl == 0) return b;
  const int vn = 16 / (int)dtype_size(x_dtype);
  const int64_t nvec = C / vn;
  b.vpl = p.vpl;
  if (CS_LN_PAIRS && (nvec <= kHalf || (nvec > kWave && nvec <= 3 * kHalf))) {
    b.kind = nvec <= kHalf ? kBwdHalf1 : kBwdHalf3;
    b.vpl = nvec <= kHalf ? 1 : 3;
    const int64_t n = ceil_div((rows + 1) / 2, (int64_t)(kLnBwdThreads / kWave));
    b.blocks = (int)(n < CS_LN_PAIR_MAX_BLOCKS ? n : CS_LN_PAIR_MAX_BLOCKS);
    b.fold_lds = (size_t)(kLnBwdThreads / kWave) * 2 * C * sizeof(float);
  } else if (p.vpl == 4 && (CS_LN_W4_NEW == 2 || (CS_LN_W4_NEW == 1 && !want_dx))) {
    b.kind = kBwdWave4;
    b.threads = CS_LN_W4_THREADS;
    b.blocks = ln_blocks(rows, 1, kLnBwdMaxBlocks, b.threads);
    b.fold_lds = (size_t)(b.threads / kWave) * C * sizeof(float);
  } else if (p.vpl == 8 && want_dp) {
    // with the dgamma/dbeta accumulators a row no longer fits one wave's registers (a single-wave
    // kernel spilled ~1 KB per lane), so two waves share each row
    b.kind = kBwdSplit;
    b.blocks = ln_blocks(rows, 1, kLnBwdMaxBlocks, kLnBwdThreads / 2);
    b.fold_lds = (size_t)(kLnBwdThreads / kWave / 2) * 4 * kWave * vn * sizeof(float);
  } else {
    b.kind = kBwdRows;
    b.blocks = ln_blocks(rows, 1, p.vpl <= 2 ? kLnBwdMaxBlocksNarrow : kLnBwdMaxBlocks, kLnBwdThreads);
    b.fold_lds = (size_t)(kLnBwdThreads / kWave) * C * sizeof(float);
  }
  return b;
}

// Column order inside a partial row, as the `vn` of ln_finalize_tile: every row kernel leaves
// column idx*vn + k at position k*(C/vn) + idx.
int partial_vn(int x_dtype) { return 16 / (int)dtype_size(x_dtype); }

enum BwdPhase { kBwdWhole = 0, kBwdRowsOnly = 1 };

// An earlier call's partial rows whose column sums ride in this call's launch (host side of
// LnPending); partial == nullptr: none.
struct PendingSums {
  const void *partial = nullptr;
  int64_t nparts = 0;
  void *dgamma = nullptr, *dbeta = nullptr;
  int accumulate = 0;
};

template <typename TP>
int launch_finalize(const void *partial, int64_t nparts, void *dgamma, void *dbeta, int64_t C, int vn,
                    int accumulate, hipStream_t s) {
  ln_bwd_finalize_kernel<TP><<<dim3(2 * (unsigned)ceil_div(C, (int64_t)kLnFinCols)), dim3(kLnFinCols * kLnFinRows), 0, s>>>(
      (const float *)partial, (int)nparts, (TP *)dgamma, (TP *)dbeta, (int)C, vn, accumulate);
  return launch_status();
}

// A launch may ask for more dynamic LDS than the 64 KB it gets by default once the kernel's limit
// has been raised; once per kernel and device.
template <typename K>
int allow_lds(K kernel, size_t bytes, size_t most, std::atomic<bool> *done) {
  if (bytes <= 64 * 1024) return CS_OK;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return (int)hipErrorInvalidDevice;
  if (!done[dev].load(std::memory_order_acquire)) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)most);
    if (e != hipSuccess) return (int)e;
    done[dev].store(true, std::memory_order_release);
  }
  return CS_OK;
}

template <typename TDY, typename TX, typename TDX, typename TP, int THREADS, int LPR, int VPL, int WPE, bool PF,
          bool KEEP, bool HAS_DX, bool HAS_DP, bool HAS_DRES>
int launch_bwd_kernel(const void *dy, const void *x, const void *mean, const void *rstd, const void *gamma,
                      void *dx, void *workspace, int64_t rows, int64_t C, const void *dres, const LnPending &pend,
                      int blocks, size_t lds, hipStream_t s) {
  static std::atomic<bool> lds_allowed[64];
  auto kernel = ln_bwd_kernel<TDY, TX, TDX, TP, THREADS, LPR, VPL, WPE, PF, KEEP, HAS_DX, HAS_DP, HAS_DRES>;
  // the fold of the widest row this instantiation takes: [rows side by side x waves][C] floats
  constexpr size_t kMostLds = (size_t)THREADS * VPL * Vec16<TX>::n * sizeof(float);
  const int st = allow_lds(kernel, lds, kMostLds, lds_allowed);
  if (st != CS_OK) return st;
  kernel<<<dim3((unsigned)(blocks + pend.blocks)), dim3(THREADS), lds, s>>>(
      (const TDY *)dy, (const TX *)x, (const float *)mean, (const float *)rstd, (const TP *)gamma, (TDX *)dx,
      (float *)workspace, rows, (int)C, (const TDX *)dres, pend);
  return launch_status();
}

template <typename TDY, typename TX, typename TDX, typename TP>
int bwd_typed(const void *dy, const void *x, const void *mean, const void *rstd,
              const void *gamma, void *dx, void *dgamma, void *dbeta, void *workspace,
              size_t workspace_bytes, int64_t rows, int64_t C, bool aligned, int x_dtype,
              int accumulate, const void *dres, hipStream_t s, BwdPhase phase = kBwdWhole,
              PendingSums pending = PendingSums{}) {
  // rows only: the partial rows are the product, the parameter gradients come from a later
  // cs_layernorm_backward_finalize (or ride in a later call's launch)
  const bool want_dp = phase == kBwdRowsOnly || dgamma != nullptr || dbeta != nullptr;
  const BwdPlan plan = aligned ? bwd_plan(rows, C, x_dtype, want_dp, dx != nullptr) : BwdPlan{};
  if (phase == kBwdRowsOnly && (plan.kind == kBwdNone || std::is_same_v<TX, double>))
    return aligned ? CS_ERR_UNSUPPORTED : CS_ERR_MISALIGNED;
  // dx + dresidual inside the kernel where it fits (rows of up to 4 vectors per lane), as a
  // second, in-place launch elsewhere
  const bool fuse_dres = dres != nullptr && plan.kind != kBwdNone && plan.vpl <= kMaxVplWithResidual && is_aligned16(dres);
  const void *late_dres = fuse_dres ? nullptr : dres;
  if (!fuse_dres) dres = nullptr;
  if constexpr (!std::is_same_v<TX, double>) {
    if (plan.kind != kBwdNone) {
      const int blocks = plan.blocks;
      const size_t need = want_dp ? (size_t)blocks * 2 * C * sizeof(float) : 0;
      if (want_dp && (workspace == nullptr || workspace_bytes < need)) return CS_ERR_WORKSPACE;
      // the split kernel carries no pending sums: those get their own launch first
      LnPending pend{nullptr, nullptr, nullptr, 0, 0, 0};
      if (pending.partial != nullptr && (pending.dgamma != nullptr || pending.dbeta != nullptr)) {
        if (plan.kind == kBwdSplit) {
          const int st = launch_finalize<TP>(pending.partial, pending.nparts, pending.dgamma, pending.dbeta, C,
                                             partial_vn(x_dtype), pending.accumulate, s);
          if (st != CS_OK) return st;
        } else {
          pend = LnPending{(const float *)pending.partial, pending.dgamma, pending.dbeta, (int)pending.nparts,
                           pending.accumulate, 2 * (int)ceil_div(C, (int64_t)kLnFinCols)};
        }
      }
      size_t lds = want_dp ? plan.fold_lds : 0;
      const size_t pend_lds = (size_t)kLnFinRows * kLnFinCols * sizeof(float);
      if (pend.blocks != 0 && lds < pend_lds) lds = pend_lds;
      const dim3 grid((unsigned)(blocks + pend.blocks)), block(kLnBwdThreads);
      int st = CS_OK;
#define CS_LN_BWD(VPL, WPE, HAS_DX, HAS_DP, HAS_DRES)                                       \
  ln_bwd_rows_kernel<TDY, TX, TDX, TP, VPL, WPE, HAS_DX, HAS_DP, HAS_DRES>                  \
      <<<grid, block, lds, s>>>((const TDY *)dy, (const TX *)x, (const float *)mean,        \
                                (const float *)rstd, (const TP *)gamma, (TDX *)dx,          \
                                (float *)workspace, rows, (int)C, (const TDX *)dres, pend)
#define CS_LN_K32(VPL, WPE, HAS_DX, HAS_DP, HAS_DRES)                                                          \
  st = launch_bwd_kernel<TDY, TX, TDX, TP, kLnBwdThreads, 32, VPL, WPE, CS_LN_PAIR_PF, CS_LN_PAIR_KEEP, HAS_DX, \
                         HAS_DP, HAS_DRES>(dy, x, mean, rstd, gamma, dx, workspace, rows, C, dres, pend, blocks, \
                                           lds, s)
#define CS_LN_K32PF(VPL, WPE, HAS_DX, HAS_DP, HAS_DRES)                                                        \
  st = launch_bwd_kernel<TDY, TX, TDX, TP, kLnBwdThreads, 32, VPL, WPE, true, CS_LN_PAIR_KEEP, HAS_DX, HAS_DP,   \
                         HAS_DRES>(dy, x, mean, rstd, gamma, dx, workspace, rows, C, dres, pend, blocks, lds, s)
#define CS_LN_K64(VPL, WPE, HAS_DX, HAS_DP, HAS_DRES)                                                          \
  st = launch_bwd_kernel<TDY, TX, TDX, TP, CS_LN_W4_THREADS, 64, VPL, WPE, CS_LN_W4_PF, CS_LN_W4_KEEP, HAS_DX,  \
                         HAS_DP, HAS_DRES>(dy, x, mean, rstd, gamma, dx, workspace, rows, C, dres, pend, blocks, \
                                           lds, s)
#define CS_LN_BWD_MASK(K, VPL, WPE)             \
  if (dx && want_dp && dres) {                  \
    K(VPL, WPE, true, true, true);              \
  } else if (dx && dres) {                      \
    K(VPL, WPE, true, false, true);             \
  } else if (dx && want_dp) {                   \
    K(VPL, WPE, true, true, false);             \
  } else if (dx) {                              \
    K(VPL, WPE, true, false, false);            \
  } else {                                      \
    K(VPL, WPE, false, true, false);            \
  }
      if (plan.kind == kBwdHalf1) {
        CS_LN_BWD_MASK(CS_LN_K32, 1, 4)
      } else if (plan.kind == kBwdHalf3) {
        // On its own a launch is one workgroup per CU, so a wave may take twice the registers and
        // load its next two rows while it works on the current ones ([8192,768]: 13.7 -> 13.1 us, with
        // dresidual 16.1 -> 15.7).  With an earlier call's sums in the launch their workgroups must
        // fit next to a row workgroup on the same CU, which the larger register budget rules out
        // (11.3 -> 12.1 us), so that form keeps two workgroups per CU and no prefetch.
        if (pend.blocks == 0 && dx != nullptr && CS_LN_H3_ALONE_PF) {  // sums alone: 10.9 us without, 11.3 with
          CS_LN_BWD_MASK(CS_LN_K32PF, 3, 1)
        } else {
          CS_LN_BWD_MASK(CS_LN_K32, 3, CS_LN_H3_WPE)
        }
      } else if (plan.kind == kBwdWave4) {
#if CS_LN_W4_NEW == 2
        CS_LN_BWD_MASK(CS_LN_K64, 4, CS_LN_W4_WPE)
#else
        CS_LN_K64(4, CS_LN_W4_WPE, false, true, false);
#endif
      } else if (plan.kind == kBwdSplit) {
        if (dx) {
          ln_bwd_split_rows_kernel<TDY, TX, TDX, TP, 4, true, true><<<dim3((unsigned)blocks), block, lds, s>>>(
              (const TDY *)dy, (const TX *)x, (const float *)mean, (const float *)rstd, (const TP *)gamma,
              (TDX *)dx, (float *)workspace, rows, (int)C);
        } else {
          ln_bwd_split_rows_kernel<TDY, TX, TDX, TP, 4, false, true><<<dim3((unsigned)blocks), block, lds, s>>>(
              (const TDY *)dy, (const TX *)x, (const float *)mean, (const float *)rstd, (const TP *)gamma,
              (TDX *)dx, (float *)workspace, rows, (int)C);
        }
      } else if (plan.vpl == 1) {
        CS_LN_BWD_MASK(CS_LN_BWD, 1, 4)
      } else if (plan.vpl == 2 && dres && want_dp) {
        CS_LN_BWD(2, 3, true, true, true);  // four per SIMD would spill
      } else if (plan.vpl == 2) {
        CS_LN_BWD_MASK(CS_LN_BWD, 2, 4)
      } else if (plan.vpl == 4) {
        CS_LN_BWD_MASK(CS_LN_BWD, 4, 2)
      } else {
        CS_LN_BWD(8, 2, true, false, false);
      }
#undef CS_LN_BWD_MASK
#undef CS_LN_K32
#undef CS_LN_K32PF
#undef CS_LN_K64
#undef CS_LN_BWD
      if (st == CS_OK) st = launch_status();
      if (st == CS_OK && want_dp && phase == kBwdWhole)
        st = launch_finalize<TP>(workspace, blocks, dgamma, dbeta, C, partial_vn(x_dtype), accumulate, s);
      if (st == CS_OK && late_dres) st = launch_add<TDX>(dx, late_dres, dx, rows * C, s);
      return st;
    }
  }
  using U = typename Acc<TX>::type;
  if (rows > 0x7fffffffLL) return CS_ERR_TOO_LARGE;
  if (dx) {
    ln_bwd_dx_general_kernel<TDY, TX, TDX, TP><<<dim3((unsigned)rows), dim3(kLnThreads), 0, s>>>(
        (const TDY *)dy, (const TX *)x, (const U *)mean, (const U *)rstd, (const TP *)gamma,
        (TDX *)dx, C, (const TDX *)late_dres);
    const int st = launch_status();
    if (st != CS_OK) return st;
  }
  if (want_dp) {
    ln_bwd_param_general_kernel<TDY, TX, TP>
        <<<dim3((unsigned)ceil_div(C, (int64_t)64)), dim3(64, 4), 0, s>>>(
            (const TDY *)dy, (const TX *)x, (const U *)mean, (const U *)rstd, (TP *)dgamma,
            (TP *)dbeta, rows, C, accumulate);
    return launch_status();
  }
  return CS_OK;
}

bool wide_ok(int narrow, int other) { return other == narrow || other == CS_F32; }

}  // namespace
}  // namespace cs_hip

using namespace cs_hip;

namespace {
int ln_forward(const void *x, const void *residual, void *sum_out, const void *gamma,
               const void *beta, void *y, void *mean, void *rstd, int64_t rows, int64_t C,
               double eps, int x_dtype, int y_dtype, int param_dtype, void *stream) {
  if (rows < 0 || C <= 0) return CS_ERR_INVALID_ARGUMENT;
  if (dtype_size(x_dtype) == 0 || dtype_size(y_dtype) == 0 || dtype_size(param_dtype) == 0)
    return CS_ERR_UNSUPPORTED;
  if (!wide_ok(x_dtype, y_dtype) || !wide_ok(x_dtype, param_dtype)) return CS_ERR_UNSUPPORTED;
  if (x_dtype == CS_F64 && (y_dtype != CS_F64 || param_dtype != CS_F64)) return CS_ERR_UNSUPPORTED;
  if (rows == 0) return CS_OK;
  if (!x || !gamma || !y || !mean || !rstd) return CS_ERR_INVALID_ARGUMENT;
  if ((residual == nullptr) != (sum_out == nullptr)) return CS_ERR_INVALID_ARGUMENT;
  if (residual && (!aligned_to(residual, dtype_size(x_dtype)) || !aligned_to(sum_out, dtype_size(x_dtype))))
    return CS_ERR_MISALIGNED;
  if (!aligned_to(x, dtype_size(x_dtype)) || !aligned_to(y, dtype_size(y_dtype)) ||
      !aligned_to(gamma, dtype_size(param_dtype)) ||
      (beta && !aligned_to(beta, dtype_size(param_dtype))) || !aligned_to(mean, 4) ||
      !aligned_to(rstd, 4))
    return CS_ERR_MISALIGNED;
  const bool aligned = is_aligned16(x) && (!residual || (is_aligned16(residual) && is_aligned16(sum_out))) &&
                       is_aligned16(y) && is_aligned16(gamma) && (!beta || is_aligned16(beta));
  hipStream_t s = as_stream(stream);
#define CS_CALL(TX, TY, TP)                                                                       \
  return fwd_typed<TX, TY, TP>(x, gamma, beta, y, mean, rstd, rows, C, eps, aligned, x_dtype, residual, \
                               sum_out, s)
  const bool y_wide = y_dtype != x_dtype, p_wide = param_dtype != x_dtype;
  switch (x_dtype) {
    case CS_F32: CS_CALL(float, float, float);
    case CS_F64: CS_CALL(double, double, double);
    case CS_F16:
      if (y_wide && p_wide) CS_CALL(f16_t, float, float);
      if (y_wide) CS_CALL(f16_t, float, f16_t);
      if (p_wide) CS_CALL(f16_t, f16_t, float);
      CS_CALL(f16_t, f16_t, f16_t);
    case CS_BF16:
      if (y_wide && p_wide) CS_CALL(bf16_t, float, float);
      if (y_wide) CS_CALL(bf16_t, float, bf16_t);
      if (p_wide) CS_CALL(bf16_t, bf16_t, float);
      CS_CALL(bf16_t, bf16_t, bf16_t);
  }
#undef CS_CALL
  return CS_ERR_UNSUPPORTED;
}
}  // namespace

extern "C" int cs_layernorm_forward(const void *x, const void *gamma, const void *beta, void *y,
                                    void *mean, void *rstd, int64_t rows, int64_t C, double eps,
                                    int x_dtype, int y_dtype, int param_dtype, void *stream) {
  return ln_forward(x, nullptr, nullptr, gamma, beta, y, mean, rstd, rows, C, eps, x_dtype, y_dtype,
                    param_dtype, stream);
}

extern "C" int cs_add_layernorm_forward(const void *x, const void *residual, void *sum_out,
                                        const void *gamma, const void *beta, void *y, void *mean,
                                        void *rstd, int64_t rows, int64_t C, double eps,
                                        int x_dtype, int y_dtype, int param_dtype, void *stream) {
  if (rows > 0 && (!residual || !sum_out)) return CS_ERR_INVALID_ARGUMENT;
  return ln_forward(x, residual, sum_out, gamma, beta, y, mean, rstd, rows, C, eps, x_dtype, y_dtype,
                    param_dtype, stream);
}

extern "C" size_t cs_layernorm_backward_workspace_bytes(int64_t rows, int64_t C) {
  if (rows <= 0 || C <= 0) return 0;
  // the most partial rows any plan leaves for this many rows, whatever the storage type
  int most = 0;
  for (int dt : {CS_F32, CS_F16}) {
    const BwdPlan b = bwd_plan(rows, C, dt, true);
    if (b.blocks > most) most = b.blocks;
  }
  return (size_t)most * 2 * (size_t)C * sizeof(float);
}

namespace {
int ln_backward(const void *dy, const void *x, const void *mean, const void *rstd,
                const void *gamma, const void *dres, void *dx, void *dgamma, void *dbeta,
                void *workspace, size_t workspace_bytes, int64_t rows, int64_t C, int dy_dtype,
                int x_dtype, int dx_dtype, int param_dtype, int accumulate, void *stream,
                BwdPhase phase = kBwdWhole, PendingSums pending = PendingSums{}) {
  if (rows < 0 || C <= 0) return CS_ERR_INVALID_ARGUMENT;
  if (dtype_size(x_dtype) == 0 || dtype_size(dy_dtype) == 0 || dtype_size(dx_dtype) == 0 ||
      dtype_size(param_dtype) == 0)
    return CS_ERR_UNSUPPORTED;
  if (!wide_ok(x_dtype, dy_dtype) || !wide_ok(x_dtype, dx_dtype) || !wide_ok(x_dtype, param_dtype))
    return CS_ERR_UNSUPPORTED;
  if (x_dtype == CS_F64 && (dy_dtype != CS_F64 || dx_dtype != CS_F64 || param_dtype != CS_F64))
    return CS_ERR_UNSUPPORTED;
  if (phase == kBwdWhole && !dx && !dgamma && !dbeta) return CS_OK;
  if (rows == 0) {
    // an empty batch still defines dgamma/dbeta: zero unless accumulating;
    // nothing to launch for that without rows, so leave it to the caller
    return CS_OK;
  }
  if (!dy || !x || !mean || !rstd || (dx && !gamma)) return CS_ERR_INVALID_ARGUMENT;
  if (dres && !dx) return CS_ERR_INVALID_ARGUMENT;
  if (dres && !aligned_to(dres, dtype_size(dx_dtype))) return CS_ERR_MISALIGNED;
  if (!aligned_to(dy, dtype_size(dy_dtype)) || !aligned_to(x, dtype_size(x_dtype)) ||
      (dx && !aligned_to(dx, dtype_size(dx_dtype))) ||
      (gamma && !aligned_to(gamma, dtype_size(param_dtype))) ||
      (dgamma && !aligned_to(dgamma, dtype_size(param_dtype))) ||
      (dbeta && !aligned_to(dbeta, dtype_size(param_dtype))) || !aligned_to(mean, 4) ||
      !aligned_to(rstd, 4))
    return CS_ERR_MISALIGNED;
  const bool aligned = is_aligned16(dy) && is_aligned16(x) && (!dx || is_aligned16(dx)) &&
                       (!dx || is_aligned16(gamma)) && (!workspace || is_aligned16(workspace)) &&
                       (!dres || is_aligned16(dres));
  hipStream_t s = as_stream(stream);
#define CS_CALL(TDY, TX, TDX, TP)                                                              \
  return bwd_typed<TDY, TX, TDX, TP>(dy, x, mean, rstd, gamma, dx, dgamma, dbeta, workspace,   \
                                     workspace_bytes, rows, C, aligned, x_dtype, accumulate, dres, s, phase, \
                                     pending)
  const bool dy_wide = dy_dtype != x_dtype, dx_wide = dx_dtype != x_dtype,
             p_wide = param_dtype != x_dtype;
  switch (x_dtype) {
    case CS_F32: CS_CALL(float, float, float, float);
    case CS_F64: CS_CALL(double, double, double, double);
    case CS_F16:
      // autocast runs: fp32 dy and dx with fp32 parameters; plain runs: all f16
      if (dy_wide && dx_wide && p_wide) CS_CALL(float, f16_t, float, float);
      if (!dy_wide && !dx_wide && p_wide) CS_CALL(f16_t, f16_t, f16_t, float);
      if (!dy_wide && !dx_wide && !p_wide) CS_CALL(f16_t, f16_t, f16_t, f16_t);
      return CS_ERR_UNSUPPORTED;
    case CS_BF16:
      if (dy_wide && dx_wide && p_wide) CS_CALL(float, bf16_t, float, float);
      if (!dy_wide && !dx_wide && p_wide) CS_CALL(bf16_t, bf16_t, bf16_t, float);
      if (!dy_wide && !dx_wide && !p_wide) CS_CALL(bf16_t, bf16_t, bf16_t, bf16_t);
      return CS_ERR_UNSUPPORTED;
  }
#undef CS_CALL
  return CS_ERR_UNSUPPORTED;
}
}  // namespace

extern "C" int cs_layernorm_backward(const void *dy, const void *x, const void *mean,
                                     const void *rstd, const void *gamma, void *dx, void *dgamma,
                                     void *dbeta, void *workspace, size_t workspace_bytes,
                                     int64_t rows, int64_t C, int dy_dtype, int x_dtype,
                                     int dx_dtype, int param_dtype, int accumulate, void *stream) {
  return ln_backward(dy, x, mean, rstd, gamma, nullptr, dx, dgamma, dbeta, workspace, workspace_bytes,
                     rows, C, dy_dtype, x_dtype, dx_dtype, param_dtype, accumulate, stream);
}

extern "C" int cs_layernorm_backward_add(const void *dy, const void *x, const void *mean,
                                         const void *rstd, const void *gamma,
                                         const void *dresidual, void *dx, void *dgamma,
                                         void *dbeta, void *workspace, size_t workspace_bytes,
                                         int64_t rows, int64_t C, int dy_dtype, int x_dtype,
                                         int dx_dtype, int param_dtype, int accumulate,
                                         void *stream) {
  if (rows > 0 && (!dresidual || !dx)) return CS_ERR_INVALID_ARGUMENT;
  return ln_backward(dy, x, mean, rstd, gamma, dresidual, dx, dgamma, dbeta, workspace,
                     workspace_bytes, rows, C, dy_dtype, x_dtype, dx_dtype, param_dtype, accumulate,
                     stream);
}

extern "C" int64_t cs_layernorm_backward_partial_rows(int64_t rows, int64_t C, int x_dtype) {
  if (rows <= 0 || C <= 0 || dtype_size(x_dtype) == 0) return 0;
  return bwd_plan(rows, C, x_dtype, true).blocks;
}

extern "C" int cs_layernorm_backward_rows(const void *dy, const void *x, const void *mean,
                                          const void *rstd, const void *gamma,
                                          const void *dresidual, void *dx, void *partials,
                                          size_t partials_bytes, int64_t rows, int64_t C,
                                          int dy_dtype, int x_dtype, int dx_dtype,
                                          int param_dtype, void *stream) {
  if (rows <= 0 || C <= 0 || !partials || !gamma) return CS_ERR_INVALID_ARGUMENT;
  if (dresidual && !dx) return CS_ERR_INVALID_ARGUMENT;
  return ln_backward(dy, x, mean, rstd, gamma, dresidual, dx, nullptr, nullptr, partials,
                     partials_bytes, rows, C, dy_dtype, x_dtype, dx_dtype, param_dtype, 0, stream,
                     kBwdRowsOnly);
}

extern "C" int cs_layernorm_backward_finalize(const void *partials, int64_t partial_rows,
                                              void *dgamma, void *dbeta, int64_t C, int x_dtype,
                                              int param_dtype, int accumulate, void *stream) {
  if (C <= 0 || partial_rows <= 0 || !partials) return CS_ERR_INVALID_ARGUMENT;
  if (dtype_size(x_dtype) == 0 || dtype_size(param_dtype) == 0 || x_dtype == CS_F64 ||
      !wide_ok(x_dtype, param_dtype))
    return CS_ERR_UNSUPPORTED;
  if (C % (16 / (int)dtype_size(x_dtype)) != 0 || partial_rows > kLnMaxPartialRows) return CS_ERR_INVALID_ARGUMENT;
  const int vn = partial_vn(x_dtype);
  if (!dgamma && !dbeta) return CS_OK;
  if (!is_aligned16(partials) || (dgamma && !aligned_to(dgamma, dtype_size(param_dtype))) ||
      (dbeta && !aligned_to(dbeta, dtype_size(param_dtype))))
    return CS_ERR_MISALIGNED;
  hipStream_t s = as_stream(stream);
  switch (param_dtype) {
    case CS_F32: return launch_finalize<float>(partials, partial_rows, dgamma, dbeta, C, vn, accumulate, s);
    case CS_F16: return launch_finalize<f16_t>(partials, partial_rows, dgamma, dbeta, C, vn, accumulate, s);
    case CS_BF16: return launch_finalize<bf16_t>(partials, partial_rows, dgamma, dbeta, C, vn, accumulate, s);
  }
  return CS_ERR_UNSUPPORTED;
}

extern "C" int cs_layernorm_backward_rows_pending(const void *dy, const void *x, const void *mean,
                                                  const void *rstd, const void *gamma,
                                                  const void *dresidual, void *dx, void *partials,
                                                  size_t partials_bytes, const void *pending_partials,
                                                  int64_t pending_partial_rows, void *pending_dgamma,
                                                  void *pending_dbeta, int pending_accumulate,
                                                  int64_t rows, int64_t C, int dy_dtype, int x_dtype,
                                                  int dx_dtype, int param_dtype, void *stream) {
  if (rows <= 0 || C <= 0 || !partials || !gamma) return CS_ERR_INVALID_ARGUMENT;
  if (dresidual && !dx) return CS_ERR_INVALID_ARGUMENT;
  PendingSums pending;
  if (pending_partials != nullptr) {
    if (pending_partial_rows <= 0 || pending_partial_rows > kLnMaxPartialRows) return CS_ERR_INVALID_ARGUMENT;
    // the sums are read while this call's partial rows are written: they cannot share memory
    const char *a = (const char *)pending_partials, *b = (const char *)partials;
    const size_t pend_bytes = (size_t)pending_partial_rows * 2 * (size_t)C * sizeof(float);
    if (a < b + partials_bytes && b < a + pend_bytes) return CS_ERR_INVALID_ARGUMENT;
    if (!is_aligned16(pending_partials) || (pending_dgamma && !aligned_to(pending_dgamma, dtype_size(param_dtype))) ||
        (pending_dbeta && !aligned_to(pending_dbeta, dtype_size(param_dtype))))
      return CS_ERR_MISALIGNED;
    pending.partial = pending_partials;
    pending.nparts = pending_partial_rows;
    pending.dgamma = pending_dgamma;
    pending.dbeta = pending_dbeta;
    pending.accumulate = pending_accumulate;
  }
  return ln_backward(dy, x, mean, rstd, gamma, dresidual, dx, nullptr, nullptr, partials,
                     partials_bytes, rows, C, dy_dtype, x_dtype, dx_dtype, param_dtype, 0, stream,
                     kBwdRowsOnly, pending);
}
