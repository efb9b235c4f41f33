// Embedding gather(-add) forward and deterministic scatter-add backward for
// gfx950.
//
// forward  : out[i,:] = weight[ids[i],:]                (src/compute/embedding.cpp:117-121)
// fwd-add  : out[b,t,:] = wte[ids[b,t],:] + wpe[t,:]    (example/gpt2/gpt2_single_device.cpp:541-545)
// backward : dweight[k,:] (+)= sum_{i: ids[i]==k} dout[i,:], dense, rows that
//            were never indexed are zero            (src/compute/embedding.cpp:147-157)
// positions: dwpe[t,:] (+)= sum_b dout[b,t,:]           (gpt2_single_device.cpp:565-566)
//
// The backward uses no floating point atomics.  It sorts (id, position) keys,
// so equal ids become one contiguous segment in ascending position order, and
// adds each segment's rows in a fixed order in fp32, which makes the result
// independent of scheduling.  Four launches:
//   1. tile sort  - each workgroup bitonic-sorts 1024 keys, one per lane:
//                   exchanges below 64 lanes are wave shuffles, the rest go
//                   through LDS.  Spare workgroups of the same launch sum the
//                   position-table gradient, which needs no order.
//   2. merge rank - every key finds its global rank by binary search in the
//                   other tiles (staged in LDS) and is scattered to its place.
//                   Launches 1 and 2 keep few CUs busy, so further workgroups
//                   of both zero the whole table meanwhile (`=` semantics).
//   3. reduce     - a segmented sum.  A workgroup owns 32 consecutive sorted
//                   entries, each of its 8 waves owns 4 of them and loads
//                   their rows at once.  Runs of equal ids inside a wave are
//                   added in registers; runs that cross waves are folded
//                   through LDS in wave order; a segment that crosses
//                   workgroups leaves one fp32 partial row per workgroup, so
//                   a hot row is read by as many CUs as it has windows.
//   4. finish     - the workgroup of a crossing segment's first window adds
//                   that segment's partial rows in window order.
// A list of at most 8192 entries skips 1 and 2: one launch ranks every key by
// comparing it with all others (see emb_bwd_rank_kernel), and does the zero
// fill and the position-table sum next to that.
// The traffic that matters is the dense write of dweight (V*C elements), one
// read of dout and a second write of the indexed rows.
#include "common.hpp"

#include <atomic>
#include <type_traits>

namespace cs_hip {
namespace {

constexpr int kThreads = 256;

// ------------------------------------------------------------------ forward
// One 16-byte vector per thread step, kFwdUnroll steps per thread; `nvec` vectors per row.
// The row and the vector of a thread's first step come from one 32-bit division, the later
// steps advance them by the constant 256 = step_rows * nvec + step_vecs.  Every load of a full
// workgroup is issued without a lane-dependent condition (an index out of range reads row 0 and
// the result is replaced by zeros): the position rows and the indices go first, the table rows
// as soon as the indices are there, so a thread makes two round trips however many steps it has.
#ifndef CS_EMB_FWD_UNROLL
#define CS_EMB_FWD_UNROLL 2
#endif
constexpr int kFwdUnroll = CS_EMB_FWD_UNROLL;

template <typename T, typename IdxT, bool ADD>
__global__ __launch_bounds__(kThreads) void emb_fwd_vec_kernel(
    const T *__restrict__ weight, const T *__restrict__ wpe, const IdxT *__restrict__ ids,
    T *__restrict__ out, int64_t n_rows, uint32_t nvec, int64_t num_weights, uint32_t T_len) {
  constexpr int VN = Vec16<T>::n;
  constexpr uint32_t kChunk = kThreads * kFwdUnroll;
  const int64_t total = n_rows * nvec;
  // the workgroup's first row: 32-bit divisions where the whole output has fewer than 2^32
  // vectors (a 64-bit division by a variable is a hundred instructions)
  const int64_t chunk_base = (int64_t)blockIdx.x * kChunk;
  int64_t row_base;
  uint32_t rem_base, t_base = 0u;
  if (total <= 0xFFFFFFFFll) {
    const uint32_t cb = (uint32_t)chunk_base;
    const uint32_t rb = cb / nvec;
    rem_base = cb - rb * nvec;
    if constexpr (ADD) t_base = rb % T_len;
    row_base = rb;
  } else {
    row_base = chunk_base / nvec;
    rem_base = (uint32_t)(chunk_base - row_base * nvec);
    if constexpr (ADD) t_base = (uint32_t)(row_base % T_len);
  }
  const uint32_t step_rows = kThreads / nvec, step_vecs = kThreads % nvec;
  const uint32_t local = rem_base + threadIdx.x;
  uint32_t drow = local / nvec;
  uint32_t vec = local - drow * nvec;
  const bool full = chunk_base + kChunk <= total;  // workgroup-uniform

  uint32_t drows[kFwdUnroll], vecs[kFwdUnroll];
#pragma unroll
  for (int u = 0; u < kFwdUnroll; ++u) {
    drows[u] = drow;
    vecs[u] = vec;
    drow += step_rows;
    vec += step_vecs;
    if (vec >= nvec) {
      vec -= nvec;
      ++drow;
    }
  }
  const int64_t row_stride = (int64_t)nvec * VN;
  if (full) {
    IdxT raw_id[kFwdUnroll];
    Vec16<T> w[kFwdUnroll], p[kFwdUnroll];
#pragma unroll
    for (int u = 0; u < kFwdUnroll; ++u) raw_id[u] = ids[row_base + drows[u]];
    if constexpr (ADD) {
#pragma unroll
      for (int u = 0; u < kFwdUnroll; ++u) {
        uint32_t t = t_base + drows[u];  // below 2 T_len + 256: the workgroup spans few rows
        t = t % T_len;
        p[u] = load16(wpe + (int64_t)t * row_stride + (int64_t)vecs[u] * VN);
      }
    }
    bool ok[kFwdUnroll];
#pragma unroll
    for (int u = 0; u < kFwdUnroll; ++u) {
      const int64_t id = (int64_t)raw_id[u];
      ok[u] = id >= 0 && id < num_weights;
      w[u] = load16(weight + (ok[u] ? id : 0) * row_stride + (int64_t)vecs[u] * VN);
    }
#pragma unroll
    for (int u = 0; u < kFwdUnroll; ++u) {
      Vec16<T> r;
#pragma unroll
      for (int k = 0; k < VN; ++k) {
        if constexpr (ADD) {
          // fp32 add, one rounding: equals the storage-type add bit for bit
          r.e[k] = ok[u] ? from_acc<T>(to_acc(w[u].e[k]) + to_acc(p[u].e[k])) : T{};
        } else {
          r.e[k] = ok[u] ? w[u].e[k] : T{};
        }
      }
      store16_stream(out + ((row_base + drows[u]) * nvec + vecs[u]) * VN, r);
    }
    return;
  }
  // the last, ragged workgroup
  for (int u = 0; u < kFwdUnroll; ++u) {
    const int64_t row = row_base + drows[u];
    if (row >= n_rows) break;
    const int64_t id = (int64_t)ids[row];
    const bool ok = id >= 0 && id < num_weights;
    Vec16<T> r;
#pragma unroll
    for (int k = 0; k < VN; ++k) r.e[k] = T{};
    if (ok) {
      r = load16(weight + id * row_stride + (int64_t)vecs[u] * VN);
      if constexpr (ADD) {
        const Vec16<T> pv = load16(wpe + (row % T_len) * row_stride + (int64_t)vecs[u] * VN);
#pragma unroll
        for (int k = 0; k < VN; ++k) r.e[k] = from_acc<T>(to_acc(r.e[k]) + to_acc(pv.e[k]));
      }
    }
    store16_stream(out + (row * nvec + vecs[u]) * VN, r);
  }
}

// any C, any alignment
template <typename T, typename IdxT, bool ADD>
__global__ __launch_bounds__(kThreads) void emb_fwd_scalar_kernel(
    const T *__restrict__ weight, const T *__restrict__ wpe, const IdxT *__restrict__ ids,
    T *__restrict__ out, int64_t n_rows, int64_t C, int64_t num_weights, int64_t T_len) {
  const int64_t total = n_rows * C;
  for (int64_t f = (int64_t)blockIdx.x * kThreads + threadIdx.x; f < total;
       f += (int64_t)gridDim.x * kThreads) {
    const int64_t row = f / C, c = f - row * C;
    const int64_t id = (int64_t)ids[row];
    const bool ok = id >= 0 && id < num_weights;
    if constexpr (ADD) {
      out[f] = ok ? from_acc<T>(to_acc(weight[id * C + c]) + to_acc(wpe[(row % T_len) * C + c]))
                  : T{};
    } else {
      out[f] = ok ? weight[id * C + c] : T{};
    }
  }
}

// ----------------------------------------------------------- backward: keys
// A key orders first by id, then by position.  32-bit keys are used when
// (num_weights << shift) fits, with shift = log2 of the padded entry count.
template <typename KeyT>
struct KeyCodec;
template <>
struct KeyCodec<uint32_t> {
  static constexpr uint32_t kSentinel = 0xFFFFFFFFu;
  __device__ static uint32_t make(uint32_t id, uint32_t pos, int shift) {
    return (id << shift) | pos;
  }
  __device__ static uint32_t id(uint32_t key, int shift) { return key >> shift; }
  __device__ static uint32_t pos(uint32_t key, int shift) { return key & ((1u << shift) - 1u); }
};
template <>
struct KeyCodec<uint64_t> {
  static constexpr uint64_t kSentinel = ~0ull;
  __device__ static uint64_t make(uint32_t id, uint32_t pos, int) {
    return ((uint64_t)id << 32) | pos;
  }
  __device__ static uint32_t id(uint64_t key, int) { return (uint32_t)(key >> 32); }
  __device__ static uint32_t pos(uint64_t key, int) { return (uint32_t)key; }
};

constexpr int kTile = 1024;  // keys per sorted tile = lanes of the sorting workgroup
constexpr uint32_t kNoId = 0xFFFFFFFFu;
#ifndef CS_EMB_WINDOW
#define CS_EMB_WINDOW 32
#endif
constexpr int kWindow = CS_EMB_WINDOW;  // sorted entries per reducing workgroup (at most 64)

// Position-table gradient for one 16-byte vector: dwpe[t, :] (+)= sum_b dout[b, t, :].
template <typename T>
__device__ __forceinline__ void positions_vector(const T *__restrict__ dout, T *__restrict__ dwpe,
                                                 int64_t f, int64_t B, int64_t TC,
                                                 int accumulate) {
  constexpr int VN = Vec16<T>::n;
  float a[VN];
#pragma unroll
  for (int k = 0; k < VN; ++k) a[k] = 0.f;
  // eight loads in flight, none under a condition (a batch row past the end re-reads the last
  // one and is not added)
  for (int64_t b0 = 0; b0 < B; b0 += 8) {
    Vec16<T> v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int64_t b = b0 + u < B ? b0 + u : B - 1;
      v[u] = load16_stream(dout + b * TC + f * VN);
    }
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (b0 + u < B)
#pragma unroll
        for (int k = 0; k < VN; ++k) a[k] += to_acc(v[u].e[k]);
  }
  Vec16<T> o;
  if (accumulate) {
    const Vec16<T> old = load16(dwpe + f * VN);
#pragma unroll
    for (int k = 0; k < VN; ++k) o.e[k] = from_acc<T>(to_acc(old.e[k]) + a[k]);
  } else {
#pragma unroll
    for (int k = 0; k < VN; ++k) o.e[k] = from_acc<T>(a[k]);
  }
  store16_stream(dwpe + f * VN, o);
}

// The same for a workgroup of kTile lanes, with the batch dimension split over S = 2^log2_s lanes
// per vector: a lane walks its rows with 8 loads in flight, so a long batch is a long chain of
// round trips unless it is cut up.  Lane (v, q) adds the rows of slice q for vector v of the
// workgroup's kTile / S; slices 1.. are left in LDS and slice 0 adds them in order, so the sum
// is a fixed tree.  lds: (S - 1) * (kTile / S) * VN floats.  With S = 1 this is positions_vector.
typedef float f32x4 __attribute__((ext_vector_type(4)));
constexpr int kPosMaxLog2Slices = 4;
constexpr size_t kPosLdsBytes = (size_t)kTile * 32;  // bound for every S and element type

template <typename T>
__device__ __forceinline__ void positions_block(const T *__restrict__ dout, T *__restrict__ dwpe,
                                                int64_t blk, int64_t B, int64_t TC, int accumulate,
                                                int log2_s, f32x4 *lds, int tid) {
  constexpr int VN = Vec16<T>::n;
  constexpr int kPieces = VN / 4;  // f32x4 pieces of one vector's sums
  if (log2_s == 0) {  // block-uniform
    const int64_t f = blk * kTile + tid;
    if (f < TC / VN) positions_vector<T>(dout, dwpe, f, B, TC, accumulate);
    return;
  }
  constexpr int kInFlight = 4;  // loads per lane: with the batch cut up there are lanes enough
  const int S = 1 << log2_s;
  const int V = kTile >> log2_s;
  const int v = tid & (V - 1);
  const int q = tid >> (10 - log2_s);
  static_assert(kTile == 1024, "q is tid / V with V = 1024 >> log2_s");
  const int64_t f = blk * V + v;
  const bool ok = f < TC / VN;
  const int64_t per = (B + S - 1) / S;
  const int64_t b_lo = q * per;
  const int64_t b_hi = b_lo + per < B ? b_lo + per : B;
  float a[VN];
#pragma unroll
  for (int k = 0; k < VN; ++k) a[k] = 0.f;
  if (ok) {
    for (int64_t b0 = b_lo; b0 < b_hi; b0 += kInFlight) {
      Vec16<T> r[kInFlight];
#pragma unroll
      for (int u = 0; u < kInFlight; ++u) {
        const int64_t b = b0 + u < b_hi ? b0 + u : b_hi - 1;
        r[u] = load16_stream(dout + b * TC + f * VN);
      }
#pragma unroll
      for (int u = 0; u < kInFlight; ++u)
        if (b0 + u < b_hi)
#pragma unroll
          for (int k = 0; k < VN; ++k) a[k] += to_acc(r[u].e[k]);
    }
  }
  if (q > 0 && ok) {
#pragma unroll
    for (int h = 0; h < kPieces; ++h) {
      const f32x4 piece = {a[4 * h], a[4 * h + 1], a[4 * h + 2], a[4 * h + 3]};
      lds[((q - 1) * kPieces + h) * V + v] = piece;
    }
  }
  __syncthreads();
  if (q != 0 || !ok) return;
  for (int qq = 1; qq < S; ++qq) {
#pragma unroll
    for (int h = 0; h < kPieces; ++h) {
      const f32x4 piece = lds[((qq - 1) * kPieces + h) * V + v];
      a[4 * h] += piece.x;
      a[4 * h + 1] += piece.y;
      a[4 * h + 2] += piece.z;
      a[4 * h + 3] += piece.w;
    }
  }
  Vec16<T> o;
  if (accumulate) {
    const Vec16<T> old = load16(dwpe + f * VN);
#pragma unroll
    for (int k = 0; k < VN; ++k) o.e[k] = from_acc<T>(to_acc(old.e[k]) + a[k]);
  } else {
#pragma unroll
    for (int k = 0; k < VN; ++k) o.e[k] = from_acc<T>(a[k]);
  }
  store16_stream(dwpe + f * VN, o);
}

// Zero fill of the table, spread over the sort and merge launches, whose own work leaves
// most CUs idle.  Every row is zeroed before the reduce launch writes the indexed ones.
// One fill workgroup clears a fixed number of 16-byte vectors, chosen per launch.
#ifndef CS_EMB_FILL_VECS_RANK
#define CS_EMB_FILL_VECS_RANK 2048
#endif
#ifndef CS_EMB_FILL_VECS_SORT
#define CS_EMB_FILL_VECS_SORT 1024
#endif
#ifndef CS_EMB_FILL_VECS_MERGE
#define CS_EMB_FILL_VECS_MERGE 256
#endif
// Two vectors per lane next to the ranking workgroups (27.9 us per call against 28.6 with one), one
// per lane next to the sort and merge workgroups (16384 tokens x 1600: 60.7 us per call against 65.5
// with 2048 vectors per workgroup in both, 62.7 with 2048 / 256, 62.1 with 1024 / 1024).
constexpr int kFillVecsRank = CS_EMB_FILL_VECS_RANK;
constexpr int kFillVecsSort = CS_EMB_FILL_VECS_SORT;
constexpr int kFillVecsMerge = CS_EMB_FILL_VECS_MERGE;
#ifndef CS_EMB_FILL_SORT_PCT
#define CS_EMB_FILL_SORT_PCT 50  // share of the table cleared in the sort launch
#endif

template <int THREADS, int kFillVecs>
__device__ __forceinline__ void zero_fill_block(u32x4 *__restrict__ dst, int64_t vecs, int64_t blk,
                                                int tid) {
  const u32x4 z = {0u, 0u, 0u, 0u};
  const int64_t v0 = blk * kFillVecs;
  static_assert(kFillVecs % THREADS == 0, "whole vectors per lane");
#pragma unroll 8
  for (int u = 0; u < kFillVecs / THREADS; ++u) {
    const int64_t i = v0 + (int64_t)u * THREADS + tid;
    if (i < vecs) store_stream(dst + i, z);
  }
}

// Launch layout, in block order:
//   [0, n_tiles)                sort one tile of 1024 keys
//   + 1                         preset sorted_id to "no id"
//   + pos_blocks                position-table gradient, 1024 vectors per block
//   + the rest                  zero fill of fill_dst[0, fill_vecs)
template <typename KeyT, typename IdxT, typename T>
__global__ __launch_bounds__(kTile) void emb_bwd_tile_sort_kernel(
    const IdxT *__restrict__ ids, KeyT *__restrict__ tiles, uint32_t *__restrict__ sorted_id,
    int64_t n, int n_tiles, int shift, int64_t num_weights, int64_t padding_idx,
    const T *__restrict__ dout, T *__restrict__ dwpe, int64_t B, int64_t TC, int accumulate,
    int64_t pos_blocks, int pos_log2_slices, u32x4 *__restrict__ fill_dst, int64_t fill_vecs) {
  // the sorting workgroups keep two key arrays here, the position workgroups their slice sums
  static_assert(2 * kTile * sizeof(KeyT) <= kPosLdsBytes, "the key arrays fit the shared buffer");
  __shared__ f32x4 shared_raw[kPosLdsBytes / sizeof(f32x4)];
  KeyT(*keys)[kTile] = reinterpret_cast<KeyT(*)[kTile]>(shared_raw);
  const int tid = threadIdx.x;
  const int64_t blk = blockIdx.x;
  if (blk > n_tiles + pos_blocks) {
    zero_fill_block<kTile, kFillVecsSort>(fill_dst, fill_vecs, blk - n_tiles - pos_blocks - 1, tid);
    return;
  }
  if (blk > n_tiles) {
    positions_block<T>(dout, dwpe, blk - n_tiles - 1, B, TC, accumulate, pos_log2_slices, shared_raw, tid);
    return;
  }
  if (blk == n_tiles) {
    for (int64_t i = tid; i < n; i += kTile) sorted_id[i] = kNoId;
    return;
  }
  const int64_t p = blk * kTile + tid;
  KeyT key = KeyCodec<KeyT>::kSentinel;
  if (p < n) {
    const int64_t id = (int64_t)ids[p];
    if (id >= 0 && id < num_weights && id != padding_idx)
      key = KeyCodec<KeyT>::make((uint32_t)id, (uint32_t)p, shift);
  }
  // bitonic network, ascending, one key per lane
  int buf = 0;
  for (int k = 2; k <= kTile; k <<= 1) {
    for (int j = k >> 1; j > 0; j >>= 1) {
      KeyT other;
      if (j >= kWave) {
        keys[buf][tid] = key;
        __syncthreads();
        other = keys[buf][tid ^ j];
        buf ^= 1;  // the next exchange writes the other array: one barrier per step
      } else {
        other = __shfl_xor(key, j, kWave);
      }
      const bool up = (tid & k) == 0;     // this 2k-block sorts ascending
      const bool lower = (tid & j) == 0;  // this lane is the lower index of its pair
      const KeyT lo = key < other ? key : other;
      const KeyT hi = key < other ? other : key;
      key = (lower == up) ? lo : hi;
    }
  }
  tiles[p] = key;
}

// One thread per key.  rank = own index in own tile + lower bounds in all
// other tiles.  The tiles are staged in LDS a chunk at a time and four of
// them are searched side by side, so the probes overlap.
constexpr int kMergeChunkBytes = 32768;

// Blocks past the keys zero fill_dst[0, fill_vecs).
template <typename KeyT>
__global__ __launch_bounds__(kThreads) void emb_bwd_merge_kernel(
    const KeyT *__restrict__ tiles, uint32_t *__restrict__ sorted_id,
    uint32_t *__restrict__ sorted_pos, int n_tiles, int shift, u32x4 *__restrict__ fill_dst,
    int64_t fill_vecs) {
  constexpr int kChunkTiles = kMergeChunkBytes / (kTile * (int)sizeof(KeyT));
  constexpr int kSide = 4;
  constexpr int kVecPerThread = kMergeChunkBytes / 16 / kThreads;  // 8
  __shared__ u32x4 staged_raw[kMergeChunkBytes / 16];
  const int64_t key_blocks = (int64_t)n_tiles * (kTile / kThreads);
  if ((int64_t)blockIdx.x >= key_blocks) {
    zero_fill_block<kThreads, kFillVecsMerge>(fill_dst, fill_vecs, (int64_t)blockIdx.x - key_blocks, threadIdx.x);
    return;
  }
  const KeyT *staged = reinterpret_cast<const KeyT *>(staged_raw);
  const int64_t g = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  const int own = (int)(g / kTile);  // block-uniform: 256 divides 1024
  const int local = (int)(g % kTile);
  const KeyT key = tiles[g];
  const bool real = key != KeyCodec<KeyT>::kSentinel;
  int64_t rank = local;
  for (int c0 = 0; c0 < n_tiles; c0 += kChunkTiles) {
    const int c_tiles = n_tiles - c0 < kChunkTiles ? n_tiles - c0 : kChunkTiles;
    const int c_vecs = c_tiles * kTile * (int)sizeof(KeyT) / 16;
    const u32x4 *src = reinterpret_cast<const u32x4 *>(tiles + (int64_t)c0 * kTile);
    u32x4 v[kVecPerThread];
#pragma unroll
    for (int u = 0; u < kVecPerThread; ++u) {
      const int i = u * kThreads + threadIdx.x;
      v[u] = src[i < c_vecs ? i : c_vecs - 1];  // all requested before the first is used
    }
    __syncthreads();  // the previous chunk is no longer being searched
#pragma unroll
    for (int u = 0; u < kVecPerThread; ++u) {
      const int i = u * kThreads + threadIdx.x;
      if (i < c_vecs) staged_raw[i] = v[u];
    }
    __syncthreads();
    for (int b0 = 0; b0 < c_tiles; b0 += kSide) {
      const KeyT *tile[kSide];
      int lb[kSide];
#pragma unroll
      for (int u = 0; u < kSide; ++u) {
        const int b = b0 + u < c_tiles ? b0 + u : c_tiles - 1;
        tile[u] = staged + b * kTile;
        lb[u] = 0;
      }
      // lower bound in a power-of-two tile: kTile/2, kTile/4, ... 1, then one last probe
      for (int step = kTile >> 1; step > 0; step >>= 1) {
        KeyT probe[kSide];
#pragma unroll
        for (int u = 0; u < kSide; ++u) probe[u] = tile[u][lb[u] + step - 1];
#pragma unroll
        for (int u = 0; u < kSide; ++u) lb[u] += probe[u] < key ? step : 0;
      }
#pragma unroll
      for (int u = 0; u < kSide; ++u) {
        const int b = c0 + b0 + u;
        if (b0 + u >= c_tiles || b == own) continue;
        // lb counts the keys < key so far; one last probe decides the element at the bound
        const KeyT at = tile[u][lb[u]];
        rank += lb[u] + (at < key ? 1 : 0);
      }
    }
  }
  if (!real) return;
  sorted_id[rank] = KeyCodec<KeyT>::id(key, shift);
  sorted_pos[rank] = KeyCodec<KeyT>::pos(key, shift);
}

// -------------------------------------------- backward: ranking a short list
// With few enough keys (they all fit in the LDS of one workgroup) sorting takes one launch
// instead of two: a key's place in the sorted order is the number of keys below it (keys are
// distinct: they contain the position), found by comparing it with every other key.  That is
// n^2 comparisons, 2 VALU operations each and nothing else, spread evenly over the chip, next
// to the zero fill that the same launch does.
//
// A workgroup of 1024 lanes ranks kRankOwn = 32 keys.  It first builds every key of the list
// in its LDS.  Lane l then owns key (l mod 32) of the workgroup's 32 and belongs to one of
// 32 groups; group g compares against the 16-byte key quads g, g + 32, g + 64, ...: the two
// groups of a wave read adjacent quads (no bank conflict, every lane of a group the same
// address).  The 32 partial counts of a key are added through the LDS.
// Launch layout, in block order (the ranking workgroups run longest, so they start first):
//   [0, rank_blocks)            rank 32 keys each; also preset the unused tail of sorted_id
//   + pos_blocks                position-table gradient, 1024 vectors per block
//   + the rest                  zero fill of fill_dst[0, fill_vecs)
constexpr int kRankThreads = 1024;
constexpr int kRankOwn = 32;
constexpr int kRankGroups = kRankThreads / kRankOwn;
#ifndef CS_EMB_RANK_MAX_KEY_BYTES
#define CS_EMB_RANK_MAX_KEY_BYTES 32768
#endif
constexpr size_t kRankMaxKeyBytes = CS_EMB_RANK_MAX_KEY_BYTES;  // longest key list that is ranked this way
constexpr size_t kRankPartBytes = (size_t)kRankGroups * kRankOwn * sizeof(int);

template <typename KeyT, typename IdxT, typename T>
__global__ __launch_bounds__(kRankThreads) void emb_bwd_rank_kernel(
    const IdxT *__restrict__ ids, uint32_t *__restrict__ sorted_id,
    uint32_t *__restrict__ sorted_pos, int64_t n, int n_quads, int shift, int64_t num_weights,
    int64_t padding_idx, const T *__restrict__ dout, T *__restrict__ dwpe, int64_t B, int64_t TC,
    int accumulate, int rank_blocks, int64_t pos_blocks, int pos_log2_slices,
    u32x4 *__restrict__ fill_dst, int64_t fill_vecs) {
  typedef KeyT Quad __attribute__((ext_vector_type(4)));
  extern __shared__ u32x4 rank_lds[];  // the key list and the partial counts; kPosLdsBytes at least when positions are sliced
  __shared__ int valid_of_wave[kRankThreads / kWave];
  const int tid = threadIdx.x;
  const int64_t blk = blockIdx.x;
  if (blk >= rank_blocks + pos_blocks) {
    zero_fill_block<kRankThreads, kFillVecsRank>(fill_dst, fill_vecs, blk - rank_blocks - pos_blocks, tid);
    return;
  }
  if (blk >= rank_blocks) {
    positions_block<T>(dout, dwpe, blk - rank_blocks, B, TC, accumulate, pos_log2_slices,
                       reinterpret_cast<f32x4 *>(rank_lds), tid);
    return;
  }
  KeyT *keys = reinterpret_cast<KeyT *>(rank_lds);  // [4 n_quads], padded with sentinels
  int *part = reinterpret_cast<int *>(keys + (size_t)n_quads * 4);  // [kRankGroups][kRankOwn]
  const int lane = tid & (kWave - 1);
  const int wave = tid >> 6;
  const int n_keys = n_quads * 4;

  // ---- every key of the list, and how many are real
  int mine = 0;
  constexpr int kIdsInFlight = 8;  // the whole list of 8192 in one round trip
  for (int i0 = tid; i0 < n_keys; i0 += kRankThreads * kIdsInFlight) {
    IdxT raw[kIdsInFlight];
#pragma unroll
    for (int u = 0; u < kIdsInFlight; ++u) {
      const int i = i0 + u * kRankThreads;
      raw[u] = ids[i < n ? i : n - 1];  // no load under a condition: they all go out at once
    }
#pragma unroll
    for (int u = 0; u < kIdsInFlight; ++u) {
      const int i = i0 + u * kRankThreads;
      if (i >= n_keys) break;
      KeyT key = KeyCodec<KeyT>::kSentinel;
      const int64_t id = (int64_t)raw[u];
      if (i < n && id >= 0 && id < num_weights && id != padding_idx)
        key = KeyCodec<KeyT>::make((uint32_t)id, (uint32_t)i, shift);
      keys[i] = key;
      mine += key != KeyCodec<KeyT>::kSentinel ? 1 : 0;
    }
  }
  const int in_wave = wave_reduce(mine, SumOp{});
  if (lane == 0) valid_of_wave[wave] = in_wave;
  __syncthreads();
  int n_valid = 0;
#pragma unroll
  for (int w = 0; w < kRankThreads / kWave; ++w) n_valid += valid_of_wave[w];

  // ---- entries past the real keys read "no id": each ranking workgroup presets a share
  {
    const int tail = (int)n - n_valid;
    const int share = (tail + rank_blocks - 1) / rank_blocks;
    for (int i = tid; i < share; i += kRankThreads) {
      const int64_t at = (int64_t)n_valid + blk * share + i;
      if (at < n) sorted_id[at] = kNoId;
    }
  }

  // ---- partial counts
  const int slot = lane & (kRankOwn - 1);
  const int group = wave * (kWave / kRankOwn) + lane / kRankOwn;
  const int own_at = (int)blk * kRankOwn + slot;
  const KeyT own = own_at < n_keys ? keys[own_at] : KeyCodec<KeyT>::kSentinel;
  const Quad *quads = reinterpret_cast<const Quad *>(keys);
  int below = 0;
#pragma unroll 4
  for (int q = group; q < n_quads; q += kRankGroups) {
    const Quad k = quads[q];
    below += (k.x < own ? 1 : 0) + (k.y < own ? 1 : 0) + (k.z < own ? 1 : 0) + (k.w < own ? 1 : 0);
  }
  part[group * kRankOwn + slot] = below;
  __syncthreads();
  if (tid < kRankOwn && own != KeyCodec<KeyT>::kSentinel) {
    int rank = 0;
#pragma unroll
    for (int g = 0; g < kRankGroups; ++g) rank += part[g * kRankOwn + tid];
    sorted_id[rank] = KeyCodec<KeyT>::id(own, shift);
    sorted_pos[rank] = KeyCodec<KeyT>::pos(own, shift);
  }
}

// ------------------------------------------------------ backward: reduction
constexpr int kOwn = 4;                         // sorted entries per wave
constexpr int kRedWaves = kWindow / kOwn;       // 8
constexpr int kRedThreads = kRedWaves * kWave;  // 512: two workgroups share a CU
constexpr int kFinThreads = 1024;               // finish kernel
constexpr int kFinWaves = kFinThreads / kWave;
#ifndef CS_EMB_FIN_DIRECT_ROWS
#define CS_EMB_FIN_DIRECT_ROWS 8
#endif
#ifndef CS_EMB_FIN_MAX_GROUPS
#define CS_EMB_FIN_MAX_GROUPS 8
#endif
#ifndef CS_EMB_FIN_IN_FLIGHT
#define CS_EMB_FIN_IN_FLIGHT 8
#endif
constexpr int kFinInFlight = CS_EMB_FIN_IN_FLIGHT;      // rows a lane of a group loads before it adds (a multiple of 8)
constexpr int kFinDirectRows = CS_EMB_FIN_DIRECT_ROWS;  // segments of up to this many partial rows: one column per lane
constexpr int kFinMaxGroups = CS_EMB_FIN_MAX_GROUPS;    // lane groups that share the rows of a longer segment
#ifndef CS_EMB_VPL
#define CS_EMB_VPL 2
#endif
constexpr int kVpl = CS_EMB_VPL;                // 16-byte column vectors per lane per column chunk

// Workgroup w reduces sorted entries [kWindow w, kWindow (w + 1)).  partial rows live at
// partial[(w*2 + slot) * C]: slot 0 for a run that came in over the window's
// left edge and ends inside, slot 1 for a run that leaves over its right edge.
template <typename T>
__global__ __launch_bounds__(kRedThreads, 2048 / kRedThreads) void emb_bwd_reduce_kernel(
    const T *__restrict__ dout, const uint32_t *__restrict__ sorted_id,
    const uint32_t *__restrict__ sorted_pos, T *__restrict__ dweight, float *__restrict__ partial,
    int64_t n, int64_t C, int accumulate, int by_freq) {
  constexpr int VN = Vec16<T>::n;
  constexpr int kChunkCols = kWave * kVpl * VN;
  extern __shared__ float lds[];  // [kRedWaves][2 slots][kChunkCols]
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid >> 6;
  const int nvec = (int)(C / VN);
  const int64_t w = blockIdx.x;
  const int64_t p0 = w * kWindow;

  // ---- ids of the window (lane l <-> entry p0 + l), the entry before and the entry after
  const int64_t p = p0 + lane;
  const bool in_window = lane < kWindow;
  // lanes 0..3: the positions of this wave's four entries, asked for together with the ids
  // (an entry past the real ones holds no position; it is never used)
  // The four index loads go out together: none sits under a lane-dependent condition (an entry
  // past the end re-reads the last one and is masked afterwards).
  const int64_t own_p = p0 + wave * kOwn + lane;
  const int64_t last = n - 1;
  const uint32_t raw_pos = sorted_pos[own_p < last ? own_p : last];
  const uint32_t raw_id = sorted_id[p < last ? p : last];
  const uint32_t raw_prev = sorted_id[p > 0 ? (p - 1 < last ? p - 1 : last) : 0];
  uint32_t raw_next = sorted_id[p0 + kWindow < last ? p0 + kWindow : last];  // uniform load
  // keeps the compiler from moving three of the loads below the early exit, where each would
  // wait for the one before it
  asm volatile("" : "+v"(raw_next) : "v"(raw_pos), "v"(raw_id), "v"(raw_prev));
  const uint32_t lane_pos = (lane < kOwn && own_p < n) ? raw_pos : 0u;
  const uint32_t my_id = (in_window && p < n) ? raw_id : kNoId;
  const uint32_t prev_id = (in_window && p > 0 && p <= n) ? raw_prev : kNoId;
  const uint64_t valid = __ballot(my_id != kNoId);
  if (valid == 0) return;  // nothing sorted into this window
  const int n_valid = __popcll(valid);  // valid entries are a prefix of the window
  // true segment heads, and run starts inside the window (a head, or entry 0)
  const uint64_t heads = __ballot(my_id != kNoId && (p == 0 || my_id != prev_id));
  const uint64_t starts = heads | 1ull;
  const uint32_t next_id = (p0 + kWindow < n) ? raw_next : kNoId;
  const uint32_t last_id = __shfl(my_id, n_valid - 1, kWave);
  const bool leaves = n_valid == kWindow && next_id == last_id;    // last run goes over the right edge

  // Of a run [a, b) inside the window: is it a whole segment?
  //   begins here  <=> a is a true head          ends here <=> b < n_valid, or b == n_valid and !leaves
  auto run_end = [&](int a) -> int {  // end of the run that starts at entry a
    const uint64_t later = a >= 63 ? 0ull : (starts >> (a + 1)) << (a + 1);
    const int b = later ? __ffsll((long long)later) - 1 : n_valid;
    return b < n_valid ? b : n_valid;
  };

  for (int cb = 0; cb < nvec; cb += kWave * kVpl) {
    // ---- level 1: this wave's four entries
    const int e0 = wave * kOwn;
    // all kOwn * kVpl row loads are in flight before the first is used: an entry past the valid
    // ones reads row 0, a vector past the row re-reads the row's last one; neither is added
    Vec16<T> r[kOwn][kVpl];
#pragma unroll
    for (int e = 0; e < kOwn; ++e) {
      const int64_t pos = e0 + e < n_valid ? (int64_t)__shfl(lane_pos, e, kWave) : 0;
#pragma unroll
      for (int j = 0; j < kVpl; ++j) {
        const int idx = cb + lane + kWave * j;
        r[e][j] = load16_stream(dout + pos * C + (int64_t)(idx < nvec ? idx : nvec - 1) * VN);
      }
    }
    float acc[kVpl][VN];
    int piece_start = e0;
#pragma unroll
    for (int e = 0; e < kOwn; ++e) {
      const int q = e0 + e;
      if (q >= n_valid) break;
      const bool starts_here = (starts >> q) & 1ull;
      if (e == 0 || starts_here) {
        piece_start = q;
#pragma unroll
        for (int j = 0; j < kVpl; ++j)
#pragma unroll
          for (int k = 0; k < VN; ++k) acc[j][k] = 0.f;
      }
#pragma unroll
      for (int j = 0; j < kVpl; ++j) {
        if (cb + lane + kWave * j < nvec) {
#pragma unroll
          for (int k = 0; k < VN; ++k) acc[j][k] += to_acc(r[e][j].e[k]);
        }
      }
      const bool piece_ends = e == kOwn - 1 || q + 1 >= n_valid || ((starts >> (q + 1)) & 1ull);
      if (!piece_ends) continue;
      // the run this piece belongs to
      const bool run_starts_in_piece = (starts >> piece_start) & 1ull;
      const bool run_ends_in_piece = q + 1 >= n_valid || ((starts >> (q + 1)) & 1ull);
      const uint32_t id = __shfl(my_id, q, kWave);
      if (run_starts_in_piece && run_ends_in_piece) {
        // a whole run of the window, inside one wave
        const bool seg_begins = (heads >> piece_start) & 1ull;
        const bool seg_ends = !(q + 1 >= n_valid && leaves);
        if (seg_begins && seg_ends) {
          T *dst = dweight + (int64_t)id * C;
          // scale_grad_by_freq: the sum over the id's entries divided by their number
          const float inv = by_freq ? 1.0f / (float)(q - piece_start + 1) : 1.0f;
#pragma unroll
          for (int j = 0; j < kVpl; ++j) {
            const int idx = cb + lane + kWave * j;
            if (idx < nvec) {
              Vec16<T> o;
              if (accumulate) {
                const Vec16<T> old = load16(dst + (int64_t)idx * VN);
#pragma unroll
                for (int k = 0; k < VN; ++k) o.e[k] = from_acc<T>(to_acc(old.e[k]) + acc[j][k] * inv);
              } else {
#pragma unroll
                for (int k = 0; k < VN; ++k) o.e[k] = from_acc<T>(acc[j][k] * inv);
              }
              store16_stream(dst + (int64_t)idx * VN, o);
            }
          }
        } else {
          float *dst = partial + (w * 2 + (seg_ends ? 0 : 1)) * C;
#pragma unroll
          for (int j = 0; j < kVpl; ++j) {
            const int idx = cb + lane + kWave * j;
            if (idx < nvec) {
#pragma unroll
              for (int k = 0; k < VN; ++k) dst[(int64_t)idx * VN + k] = acc[j][k];
            }
          }
        }
      } else {
        // part of a run that spans waves: slot 1 if it reaches this wave's last entry
        const int slot = e == kOwn - 1 ? 1 : 0;
        // four columns per 16-byte LDS word; word (j*H + h)*64 + lane holds columns
        // (lane + 64 j)*VN + 4h .. + 3, so the lanes of a wave write consecutive words
                constexpr int H = VN / 4;
        f32x4 *dst = reinterpret_cast<f32x4 *>(lds) + (wave * 2 + slot) * (kChunkCols / 4);
#pragma unroll
        for (int j = 0; j < kVpl; ++j)
#pragma unroll
          for (int h = 0; h < H; ++h)
            dst[(j * H + h) * kWave + lane] =
                f32x4{acc[j][4 * h], acc[j][4 * h + 1], acc[j][4 * h + 2], acc[j][4 * h + 3]};
      }
    }
    __syncthreads();
    // ---- level 2: runs of the window that span waves, folded in wave order.  A run that
    // spans waves is folded by the wave it starts in (wave 0 for the run that came in over the
    // left edge): that is at most one run per wave, so all folds proceed side by side.
    {
      const int first = wave * kOwn;
      const uint64_t mine = (starts >> first) & ((1ull << kOwn) - 1ull);  // run starts among my entries
      const int boundary = first + kOwn;  // the next wave's first entry
      const bool crosses = boundary < kWindow && ((valid >> boundary) & 1ull) &&
                           !((starts >> boundary) & 1ull);
      if (mine != 0 && crosses) {  // wave-uniform
        const int a = first + (63 - __clzll((long long)mine));  // my last run start: the run that crosses
        const int b = run_end(a);
        const int wb = (b - 1) / kOwn;
        const bool last_reaches_end = (b % kOwn) == 0;  // the run's piece in wave wb ends at its last entry
        const uint32_t id = __shfl(my_id, a, kWave);
        const bool seg_begins = (heads >> a) & 1ull;
        const bool seg_ends = !(b >= n_valid && leaves);
        const bool whole = seg_begins && seg_ends;
        T *drow = dweight + (int64_t)id * C;
        float *prow = partial + (w * 2 + (seg_ends ? 0 : 1)) * C;
        typedef float f32x4 __attribute__((ext_vector_type(4)));
        const f32x4 *lds4 = reinterpret_cast<const f32x4 *>(lds);
        constexpr int kSlices = kChunkCols / 4 / kWave;  // groups of four columns per lane (kVpl * VN / 4)
        f32x4 t[kSlices];
#pragma unroll
        for (int v = 0; v < kSlices; ++v) t[v] = f32x4{0.f, 0.f, 0.f, 0.f};
        for (int ww = wave; ww <= wb; ++ww) {
          // wave ww's piece of this run reaches its last entry unless the run ends inside it
          const int slot = (ww < wb || last_reaches_end) ? 1 : 0;
          const f32x4 *src = lds4 + (ww * 2 + slot) * (kChunkCols / 4) + lane;
          f32x4 x[kSlices];
#pragma unroll
          for (int v = 0; v < kSlices; ++v) x[v] = src[kWave * v];  // independent LDS reads
#pragma unroll
          for (int v = 0; v < kSlices; ++v) t[v] += x[v];
        }
#pragma unroll
        for (int v = 0; v < kSlices; ++v) {
          // slice v = j*H + h of the layout above
          constexpr int H = VN / 4;
          const int64_t col = ((int64_t)cb + lane + kWave * (v / H)) * VN + 4 * (v % H);
          if (col >= C) continue;  // C is a multiple of VN columns here
          if (whole) {
            const float inv = by_freq ? 1.0f / (float)(b - a) : 1.0f;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
              float o = t[v][k] * inv;
              if (accumulate) o += to_acc(drow[col + k]);
              drow[col + k] = from_acc<T>(o);
            }
          } else {
            *reinterpret_cast<f32x4 *>(prow + col) = t[v];
          }
        }
      }
    }
    __syncthreads();
  }

}

// The last level of the segmented sum.  Workgroup w looks at window w: if the
// run that leaves it over the right edge began in it (a true segment head),
// this is that segment's first window, and the workgroup adds the segment's
// partial rows in window order: slot 1 of every window the segment leaves,
// slot 0 of the one it ends in.
template <typename T>
__global__ __launch_bounds__(kFinThreads) void emb_bwd_finish_kernel(
    const uint32_t *__restrict__ sorted_id, const float *__restrict__ partial,
    T *__restrict__ dweight, int64_t n, int64_t C, int accumulate, int by_freq) {
  __shared__ int first_other[kFinWaves];
  __shared__ int first_tail[kFinWaves];
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid >> 6;
  const int64_t w = blockIdx.x;
  const int64_t last = w * kWindow + kWindow - 1;
  if (last + 1 >= n) return;  // nothing after this window
  // Everything the decisions below read, and the two partial rows of the usual case (a segment
  // that ends in the next window), is loaded here at once: taken one after another, each behind
  // the test of the one before, these were five trips to memory behind the kernel boundary.
  // Lane t probes window w + 1 + t: its last entry (does the segment leave it?) and its first
  // (does the segment reach it?).
  const int64_t pw = w + 1 + tid;
  const int64_t pq = pw * kWindow + kWindow - 1;
  uint32_t raw_last = sorted_id[last];
  uint32_t raw_next = sorted_id[last + 1];
  uint32_t raw_first = sorted_id[w * kWindow];
  uint32_t raw_before = sorted_id[w > 0 ? w * kWindow - 1 : 0];
  uint32_t raw_q = sorted_id[pq < n ? pq : n - 1];
  uint32_t raw_f = sorted_id[pw * kWindow < n ? pw * kWindow : n - 1];
  const int64_t col0 = tid < C ? tid : 0;
  float pre_leave = partial[(w * 2 + 1) * C + col0];        // window w, left over its right edge
  float pre_enter = partial[((w + 1) * 2 + 0) * C + col0];  // window w + 1, entered over its left edge
  asm volatile("" : "+v"(raw_last), "+v"(raw_next), "+v"(raw_first), "+v"(raw_before), "+v"(raw_q), "+v"(raw_f),
                    "+v"(pre_leave), "+v"(pre_enter));
  const uint32_t id = raw_last;
  if (id == kNoId || raw_next != id) return;  // no run leaves this window
  // its run began in this window unless the whole window (and the entry before it) has this id
  if (raw_first == id && w > 0 && raw_before == id) return;
  // windows after w whose last entry still has this id are left by the segment too; 1024 windows
  // per round.  w_hi: the first window whose last entry is not this id.  The segment ends inside
  // it when its first entry still has the id (`tail`), otherwise at the end of the window before.
  int64_t w_hi = -1;
  bool tail = false;
  for (int64_t base = w + 1; w_hi < 0; base += kFinThreads) {
    const int64_t ww = base + tid;
    const int64_t q = ww * kWindow + kWindow - 1;
    if (base != w + 1) {
      raw_q = sorted_id[q < n ? q : n - 1];
      raw_f = sorted_id[ww * kWindow < n ? ww * kWindow : n - 1];
    }
    const bool other = q >= n || raw_q != id;
    const uint64_t m = __ballot(other);
    const uint64_t reached = __ballot(ww * kWindow < n && raw_f == id);
    if (lane == 0) {
      const int at = m ? __ffsll((long long)m) - 1 : -1;
      first_other[wave] = at;
      first_tail[wave] = at >= 0 ? (int)((reached >> at) & 1) : 0;
    }
    __syncthreads();
    for (int k = 0; k < kFinWaves; ++k) {
      if (first_other[k] >= 0) {
        w_hi = base + k * kWave + first_other[k];
        tail = first_tail[k] != 0;
        break;
      }
    }
    __syncthreads();
  }
  const int64_t w_end = tail ? w_hi : w_hi - 1;  // the window the segment ends in (> w)
  // scale_grad_by_freq: the segment's length, from where it begins in window w to where it ends
  // in window w_end (it fills every window in between)
  float inv = 1.0f;
  if (by_freq) {
    const int64_t qa = w * kWindow + (lane < kWindow ? lane : kWindow - 1);
    const int64_t qb = w_end * kWindow + (lane < kWindow ? lane : kWindow - 1);
    const uint64_t in_first = __ballot(lane < kWindow && sorted_id[qa] == id);                        // a suffix of window w
    const uint64_t in_last = __ballot(lane < kWindow && qb < n && sorted_id[qb < n ? qb : n - 1] == id);  // a prefix of window w_end
    const int64_t count = __popcll(in_first) + (w_end - w - 1) * kWindow + __popcll(in_last);
    inv = 1.0f / (float)count;
  }
  T *dst = dweight + (int64_t)id * C;
  const bool usual = w_end == w + 1;
  // A hot id (many windows): the partial rows are dealt to groups of lanes, one 16-byte piece of a
  // row per lane, eight rows in flight per lane; the groups' sums meet in LDS and are added in
  // group order.  Taken one column per lane instead, the hottest row of a Zipf batch was a chain of
  // 9-18 trips to memory in a single workgroup while all others had finished.
  const int64_t rows_in = w_end - w + 1;  // partial rows of the segment
  const int vc = (int)(C >> 2);           // 16-byte pieces per row
  if (rows_in > kFinDirectRows && (C & 3) == 0 && vc <= kFinThreads) {
    __shared__ f32x4 group_sum[kFinThreads];
    int groups = kFinThreads / vc;
    if (groups > kFinMaxGroups) groups = kFinMaxGroups;
    const int g = tid / vc, v = tid - g * vc;
    if (g < groups) {
      f32x4 acc[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) acc[u] = f32x4{0.f, 0.f, 0.f, 0.f};
      for (int64_t r0 = g; r0 < rows_in; r0 += kFinInFlight * groups) {
        f32x4 x[kFinInFlight];
#pragma unroll
        for (int u = 0; u < kFinInFlight; ++u) {
          const int64_t r = r0 + (int64_t)u * groups;
          const int64_t rr = r < rows_in ? r : rows_in - 1;
          // rows before the last were left over the right edge (slot 1), the last was entered (slot 0)
          const int64_t slot = rr < rows_in - 1 ? (w + rr) * 2 + 1 : w_end * 2;
          x[u] = *reinterpret_cast<const f32x4 *>(partial + slot * C + 4 * v);
        }
#pragma unroll
        for (int u = 0; u < kFinInFlight; ++u) {
          const float keep = r0 + (int64_t)u * groups < rows_in ? 1.f : 0.f;
          acc[u & 7].x = fmaf(x[u].x, keep, acc[u & 7].x);
          acc[u & 7].y = fmaf(x[u].y, keep, acc[u & 7].y);
          acc[u & 7].z = fmaf(x[u].z, keep, acc[u & 7].z);
          acc[u & 7].w = fmaf(x[u].w, keep, acc[u & 7].w);
        }
      }
      f32x4 t;
      t.x = ((acc[0].x + acc[1].x) + (acc[2].x + acc[3].x)) + ((acc[4].x + acc[5].x) + (acc[6].x + acc[7].x));
      t.y = ((acc[0].y + acc[1].y) + (acc[2].y + acc[3].y)) + ((acc[4].y + acc[5].y) + (acc[6].y + acc[7].y));
      t.z = ((acc[0].z + acc[1].z) + (acc[2].z + acc[3].z)) + ((acc[4].z + acc[5].z) + (acc[6].z + acc[7].z));
      t.w = ((acc[0].w + acc[1].w) + (acc[2].w + acc[3].w)) + ((acc[4].w + acc[5].w) + (acc[6].w + acc[7].w));
      group_sum[tid] = t;
    }
    __syncthreads();
    if (g == 0) {
      f32x4 t = group_sum[v];
      for (int k = 1; k < groups; ++k) {
        const f32x4 o = group_sum[k * vc + v];
        t.x += o.x;
        t.y += o.y;
        t.z += o.z;
        t.w += o.w;
      }
      const float out[4] = {t.x * inv, t.y * inv, t.z * inv, t.w * inv};
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        float o = out[k];
        if (accumulate) o += to_acc(dst[4 * v + k]);
        dst[4 * v + k] = from_acc<T>(o);
      }
    }
    return;
  }
  for (int64_t col = tid; col < C; col += kFinThreads) {
    const bool have = col == tid;  // the first column of the lane came in with the loads above
    // eight interleaved sums keep eight loads in flight; the order is fixed all the same
    float t[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    int64_t ww = w;
    // every window before the last is left over its right edge (slot 1)
    for (; ww + 8 <= w_end; ww += 8) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = partial[((ww + u) * 2 + 1) * C + col];
#pragma unroll
      for (int u = 0; u < 8; ++u) t[u] += v[u];
    }
    if (usual && have) {
      t[0] += pre_leave;
      t[7] += pre_enter;
    } else {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = ww + u < w_end ? partial[((ww + u) * 2 + 1) * C + col] : 0.f;
#pragma unroll
      for (int u = 0; u < 7; ++u) t[u] += v[u];  // at most seven windows are left
      t[7] += partial[(w_end * 2 + 0) * C + col];  // the run that ends there came in over the left edge
    }
    float total = (((t[0] + t[1]) + (t[2] + t[3])) + ((t[4] + t[5]) + (t[6] + t[7]))) * inv;
    if (accumulate) total += to_acc(dst[col]);
    dst[col] = from_acc<T>(total);
  }
}

// Standalone position-table gradient.  The vector form is positions_block on its own (the
// fused call runs it inside its first launch); the scalar form takes any C and any alignment.
template <typename T>
__global__ __launch_bounds__(kTile) void emb_bwd_positions_vec_kernel(const T *__restrict__ dout,
                                                                      T *__restrict__ dwpe, int64_t B,
                                                                      int64_t TC, int accumulate,
                                                                      int log2_slices) {
  __shared__ f32x4 slices[kPosLdsBytes / sizeof(f32x4)];
  positions_block<T>(dout, dwpe, blockIdx.x, B, TC, accumulate, log2_slices, slices, threadIdx.x);
}

template <typename T>
__global__ __launch_bounds__(kThreads) void emb_bwd_positions_kernel(const T *__restrict__ dout,
                                                                     T *__restrict__ dwpe,
                                                                     int64_t B, int64_t TC,
                                                                     int accumulate) {
  using U = typename Acc<T>::type;
  for (int64_t f = (int64_t)blockIdx.x * kThreads + threadIdx.x; f < TC;
       f += (int64_t)gridDim.x * kThreads) {
    double a = 0;  // sequential over the batch, so in double like the general row kernel
    for (int64_t b = 0; b < B; ++b) a += (double)to_acc(dout[b * TC + f]);
    if (accumulate) a += (double)to_acc(dwpe[f]);
    dwpe[f] = from_acc<T>((U)a);
  }
}

// --------------------------------------------- backward: general (slow) path
// For fp64 and for rows that are not whole aligned 16-byte vectors.  Same
// sorted order, one workgroup per output row found by binary search.
template <typename T>
__global__ __launch_bounds__(kThreads) void emb_bwd_rows_general_kernel(
    const T *__restrict__ dout, const uint32_t *__restrict__ sorted_id,
    const uint32_t *__restrict__ sorted_pos, T *__restrict__ dweight, int64_t n, int64_t C,
    int accumulate, int by_freq) {
  using U = typename Acc<T>::type;
  const uint32_t row = blockIdx.x;
  // first sorted entry with id >= row (unused tail slots hold kNoId, the maximum)
  int64_t lo = 0, len = n;
  while (len > 0) {
    const int64_t half = len >> 1;
    const bool go = sorted_id[lo + half] < row;
    lo = go ? lo + half + 1 : lo;
    len = go ? len - half - 1 : half;
  }
  // One thread adds a whole segment in order: thousands of sequential fp32 additions for a hot
  // row drift by ~1e-4 of the terms' scale, so this path, which is not the fast one, adds in double.
  for (int64_t c = threadIdx.x; c < C; c += kThreads) {
    double a = 0;
    int64_t count = 0;
    for (int64_t p = lo; p < n && sorted_id[p] == row; ++p, ++count)
      a += (double)to_acc(dout[(int64_t)sorted_pos[p] * C + c]);
    if (by_freq && count > 0) a /= (double)count;  // scale_grad_by_freq
    if (accumulate) a += (double)to_acc(dweight[(int64_t)row * C + c]);
    dweight[(int64_t)row * C + c] = from_acc<T>((U)a);
  }
}

// ---------------------------------------------------------------- workspace
struct BwdLayout {
  int shift = 0;
  bool key64 = false;
  int64_t n_tiles = 0;
  int64_t n_windows = 0;
  size_t off_tiles = 0, off_sorted_id = 0, off_sorted_pos = 0, off_partial = 0;
  size_t bytes = 0;
};

size_t align256(size_t x) { return (x + 255) / 256 * 256; }

BwdLayout bwd_layout(int64_t n, int64_t C, int64_t num_weights) {
  BwdLayout L;
  L.n_tiles = ceil_div(n, (int64_t)kTile);
  const int64_t padded = L.n_tiles * kTile;
  while ((1ll << L.shift) < padded) ++L.shift;
  // ((V-1) << shift) | (2^shift - 1) must stay below the 32-bit sentinel
  L.key64 = L.shift >= 32 || ((uint64_t)num_weights << L.shift) > 0xFFFFFFFFull;
  L.n_windows = ceil_div(n, (int64_t)kWindow);
  size_t o = 0;
  L.off_tiles = o;
  o = align256(o + (size_t)padded * (L.key64 ? 8 : 4));
  L.off_sorted_id = o;
  o = align256(o + (size_t)n * 4);
  L.off_sorted_pos = o;
  o = align256(o + (size_t)n * 4);
  L.off_partial = o;
  o = align256(o + (size_t)L.n_windows * 2 * (size_t)C * sizeof(float));
  L.bytes = o;
  return L;
}

template <typename T, typename IdxT, bool ADD>
int fwd_launch(const void *weight, const void *wpe, const void *ids, void *out, int64_t n_rows,
               int64_t C, int64_t num_weights, int64_t T_len, hipStream_t s) {
  constexpr int VN = Vec16<T>::n;
  const bool vec_ok = C % VN == 0 && is_aligned16(weight) && is_aligned16(out) &&
                      (!ADD || is_aligned16(wpe)) && C / VN <= 0x7fffffff;
  if (vec_ok) {
    const int64_t total = n_rows * (C / VN);
    const int64_t blocks = ceil_div(total, (int64_t)kThreads * kFwdUnroll);
    if (blocks > 0x7fffffffLL) return CS_ERR_TOO_LARGE;
    emb_fwd_vec_kernel<T, IdxT, ADD><<<dim3((unsigned)blocks), dim3(kThreads), 0, s>>>(
        (const T *)weight, (const T *)wpe, (const IdxT *)ids, (T *)out, n_rows, (uint32_t)(C / VN),
        num_weights, (uint32_t)T_len);
  } else {
    int64_t blocks = ceil_div(n_rows * C, (int64_t)kThreads);
    if (blocks > 65536) blocks = 65536;
    emb_fwd_scalar_kernel<T, IdxT, ADD><<<dim3((unsigned)blocks), dim3(kThreads), 0, s>>>(
        (const T *)weight, (const T *)wpe, (const IdxT *)ids, (T *)out, n_rows, C, num_weights,
        T_len);
  }
  return launch_status();
}

template <typename T, bool ADD>
int fwd_idx(const void *weight, const void *wpe, const void *ids, void *out, int64_t n_rows,
            int64_t C, int64_t num_weights, int64_t T_len, int idx_dtype, hipStream_t s) {
  if (idx_dtype == CS_I32)
    return fwd_launch<T, int32_t, ADD>(weight, wpe, ids, out, n_rows, C, num_weights, T_len, s);
  if (idx_dtype == CS_I64)
    return fwd_launch<T, int64_t, ADD>(weight, wpe, ids, out, n_rows, C, num_weights, T_len, s);
  return CS_ERR_INVALID_ARGUMENT;
}

template <bool ADD>
int fwd_dispatch(const void *weight, const void *wpe, const void *ids, void *out, int64_t n_rows,
                 int64_t C, int64_t num_weights, int64_t T_len, int dtype, int idx_dtype,
                 void *stream) {
  if (n_rows < 0 || C <= 0 || num_weights < 0) return CS_ERR_INVALID_ARGUMENT;
  const size_t es = dtype_size(dtype);
  if (es == 0) return CS_ERR_UNSUPPORTED;
  if (idx_dtype != CS_I32 && idx_dtype != CS_I64) return CS_ERR_INVALID_ARGUMENT;
  if (n_rows == 0) return CS_OK;
  if (!weight || !ids || !out || (ADD && !wpe)) return CS_ERR_INVALID_ARGUMENT;
  // an empty table has no row 0 for the lanes that read it in place of an out-of-range id
  if (num_weights == 0) return CS_ERR_INVALID_ARGUMENT;
  // the vector kernel keeps the position-table length in 32 bits
  if (ADD && T_len > 0x7fffffffLL) return CS_ERR_TOO_LARGE;
  if (!aligned_to(weight, es) || !aligned_to(out, es) || (ADD && !aligned_to(wpe, es)) ||
      !aligned_to(ids, idx_dtype == CS_I64 ? 8 : 4))
    return CS_ERR_MISALIGNED;
  hipStream_t s = as_stream(stream);
  switch (dtype) {
    case CS_F32:
      return fwd_idx<float, ADD>(weight, wpe, ids, out, n_rows, C, num_weights, T_len, idx_dtype, s);
    case CS_F64:
      return fwd_idx<double, ADD>(weight, wpe, ids, out, n_rows, C, num_weights, T_len, idx_dtype, s);
    case CS_F16:
      return fwd_idx<f16_t, ADD>(weight, wpe, ids, out, n_rows, C, num_weights, T_len, idx_dtype, s);
    case CS_BF16:
      return fwd_idx<bf16_t, ADD>(weight, wpe, ids, out, n_rows, C, num_weights, T_len, idx_dtype, s);
  }
  return CS_ERR_UNSUPPORTED;
}

// Kernels whose dynamic LDS can exceed the 64 KB a launch gets by default ask for their maximum
// once per device.  `bytes` is one constant per kernel, so racing threads set the same value;
// `done` is that kernel's array of per-device flags.
int allow_dynamic_lds_once(const void *kernel, size_t bytes, std::atomic<bool> *done) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return (int)hipErrorInvalidDevice;
  if (!done[dev].load(std::memory_order_acquire)) {
    const hipError_t e =
        hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e != hipSuccess) return (int)e;
    done[dev].store(true, std::memory_order_release);
  }
  return CS_OK;
}
template <typename KeyT, typename IdxT, typename T>
int allow_rank_lds(size_t bytes) {
  static std::atomic<bool> done[64];
  return allow_dynamic_lds_once(
      reinterpret_cast<const void *>(&emb_bwd_rank_kernel<KeyT, IdxT, T>), bytes, done);
}

// lanes per vector of the position sum: enough that a lane walks at most ~16 rows of the batch
int position_slices(int64_t B) {
  int log2_slices = 0;
  while (log2_slices < kPosMaxLog2Slices && (B >> log2_slices) > 16) ++log2_slices;
  return log2_slices;
}

// Sort + merge.  The sort launch also sums dwpe (`fused_positions`), and both launches clear
// their share of fill_dst[0, fill_vecs), on the CUs the sorting leaves idle.
template <typename KeyT, typename IdxT, typename T>
int sort_launch(const void *ids, char *ws, const BwdLayout &L, int64_t n, int64_t num_weights,
                int64_t padding_idx, const T *dout, T *dwpe, bool fused_positions, int64_t B,
                int64_t TC, int accumulate, u32x4 *fill_dst, int64_t fill_vecs, hipStream_t s) {
  KeyT *tiles = reinterpret_cast<KeyT *>(ws + L.off_tiles);
  uint32_t *sorted_id = reinterpret_cast<uint32_t *>(ws + L.off_sorted_id);
  uint32_t *sorted_pos = reinterpret_cast<uint32_t *>(ws + L.off_sorted_pos);
  const int pos_log2_slices = position_slices(B);
  const int64_t pos_blocks =
      fused_positions ? ceil_div(TC / Vec16<T>::n, (int64_t)(kTile >> pos_log2_slices)) : 0;
  const int64_t n_quads = ceil_div(n, (int64_t)4);
  if ((size_t)n_quads * 4 * sizeof(KeyT) <= kRankMaxKeyBytes) {
    // a short list: one launch ranks every key against all others
    static_assert(kRankThreads == kTile, "positions_block assumes kTile lanes");
    const int64_t rank_blocks = ceil_div(n_quads * 4, (int64_t)kRankOwn);
    const int64_t fill_blocks = ceil_div(fill_vecs, (int64_t)kFillVecsRank);
    const int64_t blocks = rank_blocks + pos_blocks + fill_blocks;
    if (blocks == 0) return CS_OK;
    size_t lds = (size_t)n_quads * 4 * sizeof(KeyT) + kRankPartBytes;
    if (pos_blocks > 0 && pos_log2_slices > 0 && lds < kPosLdsBytes) lds = kPosLdsBytes;
    static_assert(kPosLdsBytes <= kRankMaxKeyBytes + kRankPartBytes, "within the limit asked for");
    const int st = allow_rank_lds<KeyT, IdxT, T>(kRankMaxKeyBytes + kRankPartBytes);
    if (st != CS_OK) return st;
    emb_bwd_rank_kernel<KeyT, IdxT, T><<<dim3((unsigned)blocks), dim3(kRankThreads), lds, s>>>(
        (const IdxT *)ids, sorted_id, sorted_pos, n, (int)n_quads, L.shift, num_weights, padding_idx,
        dout, dwpe, B, TC, accumulate, (int)rank_blocks, pos_blocks, pos_log2_slices, fill_dst, fill_vecs);
    return launch_status();
  }
  // whole fill workgroups to the sort launch, the remainder to the merge launch
  const int64_t sort_fill_blocks = ceil_div(fill_vecs, (int64_t)kFillVecsSort) * CS_EMB_FILL_SORT_PCT / 100;
  const int64_t sort_fill_vecs =
      sort_fill_blocks * kFillVecsSort < fill_vecs ? sort_fill_blocks * kFillVecsSort : fill_vecs;
  const int64_t merge_fill_blocks = ceil_div(fill_vecs - sort_fill_vecs, (int64_t)kFillVecsMerge);
  const int64_t blocks = L.n_tiles + 1 + pos_blocks + sort_fill_blocks;
  const int64_t mblocks = L.n_tiles * kTile / kThreads + merge_fill_blocks;
  if (blocks > 0x7fffffffLL || mblocks > 0x7fffffffLL) return CS_ERR_TOO_LARGE;
  emb_bwd_tile_sort_kernel<KeyT, IdxT, T><<<dim3((unsigned)blocks), dim3(kTile), 0, s>>>(
      (const IdxT *)ids, tiles, sorted_id, n, (int)L.n_tiles, L.shift, num_weights, padding_idx,
      dout, dwpe, B, TC, accumulate, pos_blocks, pos_log2_slices, fill_dst, sort_fill_vecs);
  int st = launch_status();
  if (st != CS_OK) return st;
  emb_bwd_merge_kernel<KeyT><<<dim3((unsigned)mblocks), dim3(kThreads), 0, s>>>(
      tiles, sorted_id, sorted_pos, (int)L.n_tiles, L.shift,
      fill_dst ? fill_dst + sort_fill_vecs : nullptr, fill_vecs - sort_fill_vecs);
  return launch_status();
}

template <typename T>
int allow_reduce_lds(size_t bytes) {
  static std::atomic<bool> done[64];
  return allow_dynamic_lds_once(reinterpret_cast<const void *>(&emb_bwd_reduce_kernel<T>), bytes, done);
}

template <typename T>
int bwd_typed(const void *dout, const void *ids, void *dweight, void *dwpe, char *ws,
              const BwdLayout &L, int64_t n, int64_t C, int64_t num_weights, int64_t padding_idx,
              int64_t B, int64_t T_len, int idx_dtype, int accumulate, int by_freq, hipStream_t s) {
  constexpr int VN = Vec16<T>::n;
  const bool vec_ok = !std::is_same_v<T, double> && C % VN == 0 && is_aligned16(dout) &&
                      is_aligned16(dweight) && (!dwpe || is_aligned16(dwpe));
  const bool fused_positions = vec_ok && dwpe != nullptr;
  const int64_t TC = T_len * C;
  // `=` semantics on the fast path: the whole table is zeroed, then indexed rows are written
  u32x4 *fill_dst = vec_ok && !accumulate ? reinterpret_cast<u32x4 *>(dweight) : nullptr;
  const int64_t fill_vecs = fill_dst ? num_weights * (C / VN) : 0;
  int st;
#define CS_SORT(KeyT, IdxT)                                                                      \
  sort_launch<KeyT, IdxT, T>(ids, ws, L, n, num_weights, padding_idx, (const T *)dout, (T *)dwpe, \
                             fused_positions, B, TC, accumulate, fill_dst, fill_vecs, s)
  if (L.key64) {
    st = idx_dtype == CS_I64 ? CS_SORT(uint64_t, int64_t) : CS_SORT(uint64_t, int32_t);
  } else {
    st = idx_dtype == CS_I64 ? CS_SORT(uint32_t, int64_t) : CS_SORT(uint32_t, int32_t);
  }
#undef CS_SORT
  if (st != CS_OK) return st;
  const uint32_t *sorted_id = reinterpret_cast<const uint32_t *>(ws + L.off_sorted_id);
  const uint32_t *sorted_pos = reinterpret_cast<const uint32_t *>(ws + L.off_sorted_pos);
  if (!vec_ok) {
    if (num_weights > 0x7fffffffLL) return CS_ERR_TOO_LARGE;
    emb_bwd_rows_general_kernel<T><<<dim3((unsigned)num_weights), dim3(kThreads), 0, s>>>(
        (const T *)dout, sorted_id, sorted_pos, (T *)dweight, n, C, accumulate, by_freq);
    st = launch_status();
    if (st != CS_OK || !dwpe) return st;
    int64_t blocks = ceil_div(TC, (int64_t)kThreads);
    if (blocks > 65536) blocks = 65536;
    emb_bwd_positions_kernel<T><<<dim3((unsigned)blocks), dim3(kThreads), 0, s>>>(
        (const T *)dout, (T *)dwpe, B, TC, accumulate);
    return launch_status();
  }
  if constexpr (!std::is_same_v<T, double>) {
    float *partial = reinterpret_cast<float *>(ws + L.off_partial);
    const int64_t windows = n > 0 ? L.n_windows : 0;
    if (windows > 0x7fffffffLL) return CS_ERR_TOO_LARGE;
    if (windows == 0) return CS_OK;
    const size_t lds = (size_t)kRedWaves * 2 * kWave * kVpl * VN * sizeof(float);
    st = allow_reduce_lds<T>(lds);
    if (st != CS_OK) return st;
    emb_bwd_reduce_kernel<T><<<dim3((unsigned)windows), dim3(kRedThreads), lds, s>>>(
        (const T *)dout, sorted_id, sorted_pos, (T *)dweight, partial, n, C, accumulate, by_freq);
    st = launch_status();
    if (st != CS_OK) return st;
    emb_bwd_finish_kernel<T><<<dim3((unsigned)windows), dim3(kFinThreads), 0, s>>>(
        sorted_id, partial, (T *)dweight, n, C, accumulate, by_freq);
    return launch_status();
  }
  return CS_ERR_UNSUPPORTED;
}

int bwd_dispatch(const void *dout, const void *ids, void *dweight, void *dwpe, void *workspace,
                 size_t workspace_bytes, int64_t n, int64_t C, int64_t num_weights,
                 int64_t padding_idx, int64_t B, int64_t T_len, int dtype, int idx_dtype,
                 int accumulate, void *stream, int by_freq = 0) {
  if (n < 0 || C <= 0 || num_weights <= 0) return CS_ERR_INVALID_ARGUMENT;
  const size_t es = dtype_size(dtype);
  if (es == 0) return CS_ERR_UNSUPPORTED;
  if (idx_dtype != CS_I32 && idx_dtype != CS_I64) return CS_ERR_INVALID_ARGUMENT;
  if (num_weights >= 0xFFFFFFFFll || n >= 0x7FFFFFFFll) return CS_ERR_TOO_LARGE;
  if (!dweight || (n > 0 && (!dout || !ids))) return CS_ERR_INVALID_ARGUMENT;
  if (!aligned_to(dweight, es) || (dout && !aligned_to(dout, es)) ||
      (dwpe && !aligned_to(dwpe, es)) || (ids && !aligned_to(ids, idx_dtype == CS_I64 ? 8 : 4)))
    return CS_ERR_MISALIGNED;
  const BwdLayout L = bwd_layout(n > 0 ? n : 1, C, num_weights);
  if (!workspace || workspace_bytes < L.bytes || !aligned_to(workspace, 256))
    return CS_ERR_WORKSPACE;
  char *ws = static_cast<char *>(workspace);
  hipStream_t s = as_stream(stream);
  switch (dtype) {
    case CS_F32:
      return bwd_typed<float>(dout, ids, dweight, dwpe, ws, L, n, C, num_weights, padding_idx, B,
                              T_len, idx_dtype, accumulate, by_freq, s);
    case CS_F64:
      return bwd_typed<double>(dout, ids, dweight, dwpe, ws, L, n, C, num_weights, padding_idx, B,
                               T_len, idx_dtype, accumulate, by_freq, s);
    case CS_F16:
      return bwd_typed<f16_t>(dout, ids, dweight, dwpe, ws, L, n, C, num_weights, padding_idx, B,
                              T_len, idx_dtype, accumulate, by_freq, s);
    case CS_BF16:
      return bwd_typed<bf16_t>(dout, ids, dweight, dwpe, ws, L, n, C, num_weights, padding_idx, B,
                               T_len, idx_dtype, accumulate, by_freq, s);
  }
  return CS_ERR_UNSUPPORTED;
}

}  // namespace
}  // namespace cs_hip

using namespace cs_hip;

extern "C" int cs_embedding_forward(const void *weight, const void *indices, void *out,
                                    int64_t n_indices, int64_t C, int64_t num_weights, int dtype,
                                    int idx_dtype, void *stream) {
  return fwd_dispatch<false>(weight, nullptr, indices, out, n_indices, C, num_weights, 1, dtype,
                             idx_dtype, stream);
}

extern "C" int cs_embedding_forward_add(const void *wte, const void *wpe, const void *indices,
                                        void *out, int64_t B, int64_t T, int64_t C,
                                        int64_t num_weights, int dtype, int idx_dtype,
                                        void *stream) {
  if (B < 0 || T <= 0) return CS_ERR_INVALID_ARGUMENT;
  return fwd_dispatch<true>(wte, wpe, indices, out, B * T, C, num_weights, T, dtype, idx_dtype,
                            stream);
}

extern "C" size_t cs_embedding_backward_workspace_bytes(int64_t n_indices, int64_t C,
                                                        int64_t num_weights) {
  if (n_indices < 0 || C <= 0 || num_weights <= 0) return 0;
  return bwd_layout(n_indices > 0 ? n_indices : 1, C, num_weights).bytes;
}

extern "C" int cs_embedding_backward(const void *dout, const void *indices, void *dweight,
                                     void *workspace, size_t workspace_bytes, int64_t n_indices,
                                     int64_t C, int64_t num_weights, int64_t padding_idx,
                                     int dtype, int idx_dtype, int accumulate, void *stream) {
  return bwd_dispatch(dout, indices, dweight, nullptr, workspace, workspace_bytes, n_indices, C,
                      num_weights, padding_idx, 0, 1, dtype, idx_dtype, accumulate, stream);
}

extern "C" int cs_embedding_backward_scaled(const void *dout, const void *indices, void *dweight,
                                            void *workspace, size_t workspace_bytes, int64_t n_indices,
                                            int64_t C, int64_t num_weights, int64_t padding_idx,
                                            int dtype, int idx_dtype, int accumulate, void *stream) {
  return bwd_dispatch(dout, indices, dweight, nullptr, workspace, workspace_bytes, n_indices, C,
                      num_weights, padding_idx, 0, 1, dtype, idx_dtype, accumulate, stream, 1);
}

extern "C" int cs_embedding_backward_fused(const void *dout, const void *indices, void *dwte,
                                           void *dwpe, void *workspace, size_t workspace_bytes,
                                           int64_t B, int64_t T, int64_t C, int64_t num_weights,
                                           int dtype, int idx_dtype, int accumulate,
                                           void *stream) {
  if (B < 0 || T <= 0 || !dwpe) return CS_ERR_INVALID_ARGUMENT;
  return bwd_dispatch(dout, indices, dwte, dwpe, workspace, workspace_bytes, B * T, C,
                      num_weights, -1, B, T, dtype, idx_dtype, accumulate, stream);
}

extern "C" int cs_embedding_backward_positions(const void *dout, void *dwpe, int64_t B, int64_t T,
                                               int64_t C, int dtype, int accumulate,
                                               void *stream) {
  if (B < 0 || T < 0 || C <= 0) return CS_ERR_INVALID_ARGUMENT;
  const size_t es = dtype_size(dtype);
  if (es == 0) return CS_ERR_UNSUPPORTED;
  if (T == 0) return CS_OK;
  if (!dwpe || (B > 0 && !dout)) return CS_ERR_INVALID_ARGUMENT;
  if (!aligned_to(dwpe, es) || (dout && !aligned_to(dout, es))) return CS_ERR_MISALIGNED;
  hipStream_t s = as_stream(stream);
  const int64_t TC = T * C;
#define CS_POS(T)                                                                                       \
  do {                                                                                                  \
    constexpr int VN = Vec16<T>::n;                                                                     \
    /* an empty batch goes to the scalar kernel, which then writes zeros */                            \
    if (!std::is_same_v<T, double> && B > 0 && C % VN == 0 && is_aligned16(dout) && is_aligned16(dwpe)) { \
      const int log2_slices = position_slices(B);                                                       \
      const int64_t vblocks = ceil_div(TC / VN, (int64_t)(kTile >> log2_slices));                       \
      if (vblocks > 0x7fffffffLL) return CS_ERR_TOO_LARGE;                                              \
      emb_bwd_positions_vec_kernel<T><<<dim3((unsigned)vblocks), dim3(kTile), 0, s>>>(                  \
          (const T *)dout, (T *)dwpe, B, TC, accumulate, log2_slices);                                  \
    } else {                                                                                            \
      int64_t blocks = ceil_div(TC, (int64_t)kThreads);                                                 \
      if (blocks > 65536) blocks = 65536;                                                               \
      emb_bwd_positions_kernel<T><<<dim3((unsigned)blocks), dim3(kThreads), 0, s>>>(                    \
          (const T *)dout, (T *)dwpe, B, TC, accumulate);                                               \
    }                                                                                                   \
  } while (0)
  switch (dtype) {
    case CS_F32: CS_POS(float); break;
    case CS_F64: CS_POS(double); break;
    case CS_F16: CS_POS(f16_t); break;
    case CS_BF16: CS_POS(bf16_t); break;
  }
#undef CS_POS
  return launch_status();
}
