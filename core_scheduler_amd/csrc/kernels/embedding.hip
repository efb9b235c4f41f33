// Embedding gather(-add) forward and deterministic scatter-add backward for
// gfx950.
//
// forward  : out[i,:] = weight[ids[i],:]                (src/compute/embedding.cpp:117-121)
// fwd-add  : out[b,t,:] = wte[ids[b,t],:] + wpe[t,:]    (example/gpt2/gpt2_single_device.cpp:541-545)
// backward : dweight[k,:] (+)= sum_{i: ids[i]==k} dout[i,:], dense, rows that
//            were never indexed are zero            (src/compute/embedding.cpp:147-157)
// positions: dwpe[t,:] (+)= sum_b dout[b,t,:]           (gpt2_single_device.cpp:565-566)
//
// The backward does not use floating point atomics.  It sorts (id, position)
// keys, so equal ids become one contiguous segment in ascending position
// order, and adds each segment's rows in that order in fp32, which makes the
// result independent of scheduling:
//   1. tile sort   - each workgroup bitonic-sorts a tile of keys in LDS
//   2. merge rank  - every key finds its global rank by binary search in the
//                    other tiles, is scattered to its place, and the first
//                    key of every id marks its row in a bitmap
//   3. window sums - one wavefront per 8 consecutive sorted entries adds the
//                    runs of equal ids it sees; a run that is a whole segment
//                    is written to its row, a run cut by the window edge is
//                    left as an fp32 partial row
//   4. finish      - segments longer than a window add their partial rows in
//                    window order; in the same launch the rows whose bit is
//                    clear are zero-filled and the position table gradient is
//                    summed
// The traffic that matters is step 4's dense write of dweight (V*C elements)
// and one read of dout.
#include "common.cuh"

#include <type_traits>

namespace cs_hip {
namespace {

constexpr int kThreads = 256;

template <typename IdxT>
__device__ __forceinline__ int64_t load_index(const void *ids, int64_t i) {
  return (int64_t) static_cast<const IdxT *>(ids)[i];
}

// ------------------------------------------------------------------ forward
// One 16-byte vector per thread step; `nvec` vectors per row.
template <typename T, typename IdxT, bool ADD>
__global__ __launch_bounds__(kThreads) void emb_fwd_vec_kernel(
    const T *__restrict__ weight, const T *__restrict__ wpe, const IdxT *__restrict__ ids,
    T *__restrict__ out, int64_t n_rows, int nvec, int64_t num_weights, int64_t T_len) {
  constexpr int VN = Vec16<T>::n;
  constexpr int kUnroll = 4;
  const int64_t total = n_rows * nvec;
  // one 64-bit division per workgroup, 32-bit ones per vector
  const int64_t chunk_base = (int64_t)blockIdx.x * (kThreads * kUnroll);
  const int64_t row_base = chunk_base / nvec;
  const uint32_t rem_base = (uint32_t)(chunk_base - row_base * nvec);
  const int64_t base = chunk_base + threadIdx.x;
  Vec16<T> w[kUnroll], p[kUnroll];
  bool ok[kUnroll];
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) {
    const int64_t f = base + (int64_t)u * kThreads;
    const uint32_t local = rem_base + (uint32_t)(u * kThreads) + threadIdx.x;
    const int64_t row = row_base + local / (uint32_t)nvec;
    const uint32_t vec = local % (uint32_t)nvec;
    ok[u] = false;
    if (f < total) {
      const int64_t id = (int64_t)ids[row];
      ok[u] = id >= 0 && id < num_weights;
      if (ok[u]) w[u] = load16(weight + id * ((int64_t)nvec * VN) + (int64_t)vec * VN);
      if constexpr (ADD) {
        const int64_t t = row % T_len;
        p[u] = load16(wpe + t * ((int64_t)nvec * VN) + (int64_t)vec * VN);
      }
    }
  }
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) {
    const int64_t f = base + (int64_t)u * kThreads;
    if (f < total) {
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
      store16_stream(out + f * VN, r);
    }
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

constexpr int kTile = 2048;         // keys per sorted tile
constexpr int kSortThreads = 1024;  // one compare-exchange pair per thread
constexpr uint32_t kNoId = 0xFFFFFFFFu;

// Blocks [0, n_tiles): sort one tile.  Blocks beyond: clear the row bitmap and
// preset sorted_id to "no id" so unused tail slots are recognisable.
template <typename KeyT, typename IdxT>
__global__ __launch_bounds__(kSortThreads) void emb_bwd_tile_sort_kernel(
    const IdxT *__restrict__ ids, KeyT *__restrict__ tiles, uint32_t *__restrict__ bitmap,
    int bitmap_words, uint32_t *__restrict__ sorted_id, int64_t n, int n_tiles, int shift,
    int64_t num_weights, int64_t padding_idx) {
  __shared__ KeyT keys[kTile];
  if ((int)blockIdx.x >= n_tiles) {
    const int64_t t = (int64_t)(blockIdx.x - n_tiles) * kSortThreads + threadIdx.x;
    const int64_t stride = (int64_t)(gridDim.x - n_tiles) * kSortThreads;
    for (int64_t i = t; i < bitmap_words; i += stride) bitmap[i] = 0u;
    for (int64_t i = t; i < n; i += stride) sorted_id[i] = kNoId;
    return;
  }
  const int64_t tile_base = (int64_t)blockIdx.x * kTile;
  for (int i = threadIdx.x; i < kTile; i += kSortThreads) {
    const int64_t p = tile_base + i;
    KeyT key = KeyCodec<KeyT>::kSentinel;
    if (p < n) {
      const int64_t id = (int64_t)ids[p];
      if (id >= 0 && id < num_weights && id != padding_idx)
        key = KeyCodec<KeyT>::make((uint32_t)id, (uint32_t)p, shift);
    }
    keys[i] = key;
  }
  __syncthreads();
  // bitonic network, ascending
  for (int k = 2; k <= kTile; k <<= 1) {
    for (int j = k >> 1; j > 0; j >>= 1) {
      const int t = threadIdx.x;
      const int i = ((t & ~(j - 1)) << 1) | (t & (j - 1));
      const int partner = i | j;
      const bool up = (i & k) == 0;
      const KeyT a = keys[i], b = keys[partner];
      if ((a > b) == up) {
        keys[i] = b;
        keys[partner] = a;
      }
      __syncthreads();
    }
  }
  for (int i = threadIdx.x; i < kTile; i += kSortThreads) tiles[tile_base + i] = keys[i];
}

// One thread per key.  rank = own index in own tile + lower bounds in all
// other tiles; four tiles are searched side by side so their loads overlap.
// The global predecessor is the largest of the per-tile predecessors; a key
// whose predecessor has another id starts a segment.
template <typename KeyT>
__global__ __launch_bounds__(kThreads) void emb_bwd_merge_kernel(
    const KeyT *__restrict__ tiles, uint32_t *__restrict__ bitmap,
    uint32_t *__restrict__ sorted_id, uint32_t *__restrict__ sorted_pos, int n_tiles, int shift) {
  constexpr int kSide = 4;
  const int64_t g = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  const int own = (int)(g / kTile);
  const int local = (int)(g % kTile);
  if (own >= n_tiles) return;
  const KeyT key = tiles[g];
  if (key == KeyCodec<KeyT>::kSentinel) return;
  int64_t rank = local;
  bool has_pred = local > 0;
  KeyT pred = has_pred ? tiles[g - 1] : (KeyT)0;
  for (int b0 = 0; b0 < n_tiles; b0 += kSide) {
    const KeyT *tile[kSide];
    int lb[kSide];
#pragma unroll
    for (int u = 0; u < kSide; ++u) {
      const int b = b0 + u < n_tiles ? b0 + u : n_tiles - 1;
      tile[u] = tiles + (int64_t)b * kTile;
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
    KeyT last[kSide], before[kSide];
#pragma unroll
    for (int u = 0; u < kSide; ++u) {
      last[u] = tile[u][lb[u]];
      before[u] = lb[u] > 0 ? tile[u][lb[u] - 1] : (KeyT)0;
    }
#pragma unroll
    for (int u = 0; u < kSide; ++u) {
      const int b = b0 + u;
      if (b >= n_tiles || b == own) continue;
      // lb is the count of keys < key; the key just below it is the tile's predecessor
      KeyT cand = before[u];
      int count = lb[u];
      if (last[u] < key) {
        cand = last[u];
        count += 1;
      }
      rank += count;
      if (count > 0 && (!has_pred || cand > pred)) {
        pred = cand;
        has_pred = true;
      }
    }
  }
  const uint32_t id = KeyCodec<KeyT>::id(key, shift);
  sorted_id[rank] = id;
  sorted_pos[rank] = KeyCodec<KeyT>::pos(key, shift);
  if (!has_pred || KeyCodec<KeyT>::id(pred, shift) != id) atomicOr(&bitmap[id >> 5], 1u << (id & 31));
}

// ------------------------------------------------------ backward: reduction
constexpr int kWin = 8;  // sorted entries per wavefront window
constexpr int kVpl = 2;  // 16-byte column vectors per lane per column chunk

template <typename T>
struct Row2 {
  Vec16<T> v[kVpl];
};

// Window w covers sorted entries [8w, 8w+8).  partial rows live at
// partial[(w*2 + slot) * C]: slot 1 for the run that contains the window's
// last entry, slot 0 for a cut run that contains only its first.
template <typename T>
__global__ __launch_bounds__(kThreads) void emb_bwd_window_kernel(
    const T *__restrict__ dout, const uint32_t *__restrict__ sorted_id,
    const uint32_t *__restrict__ sorted_pos, T *__restrict__ dweight, float *__restrict__ partial,
    int64_t n, int64_t C, int accumulate) {
  constexpr int VN = Vec16<T>::n;
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t w = (int64_t)blockIdx.x * (kThreads / kWave) + (threadIdx.x >> 6);
  const int64_t p0 = w * kWin;
  if (p0 >= n) return;  // wave-uniform
  // ids of entries p0-1 .. p0+8 (kNoId outside [0,n) and for unused slots)
  uint32_t id[kWin + 2], pos[kWin];
#pragma unroll
  for (int e = -1; e <= kWin; ++e) {
    const int64_t p = p0 + e;
    id[e + 1] = (p >= 0 && p < n) ? sorted_id[p] : kNoId;
  }
  if (id[1] == kNoId) return;  // nothing valid in this window
#pragma unroll
  for (int e = 0; e < kWin; ++e) pos[e] = id[e + 1] != kNoId ? sorted_pos[p0 + e] : 0u;

  const int nvec = (int)(C / VN);
  for (int cb = 0; cb < nvec; cb += kWave * kVpl) {
    Row2<T> r[kWin];
#pragma unroll
    for (int e = 0; e < kWin; ++e) {
#pragma unroll
      for (int j = 0; j < kVpl; ++j) {
        const int idx = cb + lane + kWave * j;
        if (id[e + 1] != kNoId && idx < nvec) {
          r[e].v[j] = load16_stream(dout + (int64_t)pos[e] * C + (int64_t)idx * VN);
        }
      }
    }
    float acc[kVpl][VN];
    int run_start = 0;
#pragma unroll
    for (int e = 0; e < kWin; ++e) {
      if (id[e + 1] == kNoId) break;
      if (e == 0 || id[e + 1] != id[e]) {
        run_start = e;
#pragma unroll
        for (int j = 0; j < kVpl; ++j)
#pragma unroll
          for (int k = 0; k < VN; ++k) acc[j][k] = 0.f;
      }
#pragma unroll
      for (int j = 0; j < kVpl; ++j) {
        if (cb + lane + kWave * j < nvec) {
#pragma unroll
          for (int k = 0; k < VN; ++k) acc[j][k] += to_acc(r[e].v[j].e[k]);
        }
      }
      const bool run_ends = e == kWin - 1 || id[e + 2] != id[e + 1];
      if (run_ends) {
        // does the segment start / end inside this window?
        const bool seg_begins = run_start > 0 || id[0] != id[e + 1];
        const bool seg_ends = id[e + 2] != id[e + 1];
        if (seg_begins && seg_ends) {
          T *dst = dweight + (int64_t)id[e + 1] * C;
#pragma unroll
          for (int j = 0; j < kVpl; ++j) {
            const int idx = cb + lane + kWave * j;
            if (idx < nvec) {
              Vec16<T> o;
              if (accumulate) {
                const Vec16<T> old = load16(dst + (int64_t)idx * VN);
#pragma unroll
                for (int k = 0; k < VN; ++k) o.e[k] = from_acc<T>(to_acc(old.e[k]) + acc[j][k]);
              } else {
#pragma unroll
                for (int k = 0; k < VN; ++k) o.e[k] = from_acc<T>(acc[j][k]);
              }
              store16_stream(dst + (int64_t)idx * VN, o);
            }
          }
        } else {
          const int slot = e == kWin - 1 ? 1 : 0;
          float *dst = partial + (w * 2 + slot) * C;
#pragma unroll
          for (int j = 0; j < kVpl; ++j) {
            const int idx = cb + lane + kWave * j;
            if (idx < nvec) {
#pragma unroll
              for (int q = 0; q < VN / 4; ++q) {
                Vec16<float> o;
#pragma unroll
                for (int k = 0; k < 4; ++k) o.e[k] = acc[j][q * 4 + k];
                store16(dst + (int64_t)idx * VN + q * 4, o);
              }
            }
          }
        }
      }
    }
  }
}

constexpr int kFinThreads = 1024;
constexpr int kFinGroups = 4;  // partial rows are dealt to 4 thread groups

// Launch layout of the finish kernel, in block order:
//   [0, n_windows)                       : long-segment fix-up, one block per window
//   [n_windows, n_windows + pos_blocks)  : position table gradient
//   the rest                             : zero fill of rows never indexed
template <typename T>
__global__ __launch_bounds__(kFinThreads) void emb_bwd_finish_kernel(
    const T *__restrict__ dout, const uint32_t *__restrict__ sorted_id,
    const uint32_t *__restrict__ bitmap, const float *__restrict__ partial,
    T *__restrict__ dweight, T *__restrict__ dwpe, int64_t n, int64_t C, int64_t num_weights,
    int64_t B, int64_t T_len, int64_t n_windows, int64_t pos_blocks, int accumulate,
    int do_fill) {
  constexpr int VN = Vec16<T>::n;
  extern __shared__ float lds[];  // [kFinGroups][256 * 4] column chunk
  const int64_t blk = blockIdx.x;
  if (blk < n_windows) {
    // ---- fix-up: only a window whose last run starts a segment that runs on
    const int64_t w = blk;
    const int64_t first = w * kWin;
    const int64_t last = first + kWin - 1;
    if (last + 1 >= n) return;
    const uint32_t id = sorted_id[last];
    if (id == kNoId || sorted_id[last + 1] != id) return;  // segment ends in this window
    // does the segment start in this window?  (entries are sorted, so "the
    // entry before the window has this id" means it started earlier)
    if (first > 0 && sorted_id[first - 1] == id) return;
    // first entry after `last` that has another id, found 1024 entries at a time
    __shared__ int64_t seg_end_sh;
    int64_t seg_end = n;
    for (int64_t base = last + 1; base < n; base += kFinThreads) {
      const int64_t p = base + threadIdx.x;
      const bool differs = p < n && sorted_id[p] != id;
      if (threadIdx.x == 0) seg_end_sh = n;
      __syncthreads();
      if (differs) atomicMin((unsigned long long *)&seg_end_sh, (unsigned long long)p);
      __syncthreads();
      seg_end = seg_end_sh;
      __syncthreads();
      if (seg_end < n) break;
    }
    const int64_t after = seg_end - (last + 1);  // entries of the segment past this window
    const int64_t full = after / kWin;           // windows it covers completely
    const bool head_cut = after % kWin != 0;     // then a cut run in the next one
    // partial rows to add, in window order: (w,1), (w+1,1) ... (w+full,1), then (w+full+1,0)
    const int64_t n_parts = 1 + full + (head_cut ? 1 : 0);
    const int group = threadIdx.x >> 8;   // 0..3
    const int lane256 = threadIdx.x & 255;
    const int64_t c4 = C / 4;             // float4 columns
    T *dst = dweight + (int64_t)id * C;
    for (int64_t cb = 0; cb < c4; cb += 256) {
      const int64_t col4 = cb + lane256;
      float a[4] = {0.f, 0.f, 0.f, 0.f};
      if (col4 < c4) {
        for (int64_t i = group; i < n_parts; i += kFinGroups) {
          const int64_t win = w + i;
          const int slot = (head_cut && i == n_parts - 1) ? 0 : 1;
          const Vec16<float> v = load16(partial + (win * 2 + slot) * C + col4 * 4);
#pragma unroll
          for (int k = 0; k < 4; ++k) a[k] += v.e[k];
        }
      }
#pragma unroll
      for (int k = 0; k < 4; ++k) lds[(group * 256 + lane256) * 4 + k] = a[k];
      __syncthreads();
      if (group == 0 && col4 < c4) {
        float t[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          t[k] = lds[(0 * 256 + lane256) * 4 + k];
#pragma unroll
          for (int g2 = 1; g2 < kFinGroups; ++g2) t[k] += lds[(g2 * 256 + lane256) * 4 + k];
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const int64_t c = col4 * 4 + k;
          const float old = accumulate ? to_acc(dst[c]) : 0.f;
          dst[c] = from_acc<T>(old + t[k]);
        }
      }
      __syncthreads();
    }
    return;
  }
  const int nvec = (int)(C / VN);
  if (blk < n_windows + pos_blocks) {
    // ---- dwpe[t, :] (+)= sum_b dout[b, t, :], ascending b
    const int64_t f = (blk - n_windows) * kFinThreads + threadIdx.x;
    if (f >= T_len * nvec) return;
    float a[VN];
#pragma unroll
    for (int k = 0; k < VN; ++k) a[k] = 0.f;
#pragma unroll 8
    for (int64_t b = 0; b < B; ++b) {
      const Vec16<T> v = load16(dout + b * T_len * C + f * VN);
#pragma unroll
      for (int k = 0; k < VN; ++k) a[k] += to_acc(v.e[k]);
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
    return;
  }
  if (!do_fill) return;
  // ---- zero fill: 4 vectors per thread
  const int64_t chunk_base = (blk - n_windows - pos_blocks) * (kFinThreads * 4);
  const int64_t row_base = chunk_base / nvec;
  const uint32_t rem_base = (uint32_t)(chunk_base - row_base * nvec);
  const int64_t total = num_weights * nvec;
  Vec16<T> z;
#pragma unroll
  for (int k = 0; k < VN; ++k) z.e[k] = T{};
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int64_t f = chunk_base + (int64_t)u * kFinThreads + threadIdx.x;
    if (f < total) {
      const uint32_t local = rem_base + (uint32_t)(u * kFinThreads) + threadIdx.x;
      const int64_t row = row_base + local / (uint32_t)nvec;
      if (((bitmap[row >> 5] >> (row & 31)) & 1u) == 0u) store16_stream(dweight + f * VN, z);
    }
  }
}

// Standalone position-table gradient (any C, any alignment).
template <typename T>
__global__ __launch_bounds__(kThreads) void emb_bwd_positions_kernel(const T *__restrict__ dout,
                                                                     T *__restrict__ dwpe,
                                                                     int64_t B, int64_t TC,
                                                                     int accumulate) {
  using U = typename Acc<T>::type;
  for (int64_t f = (int64_t)blockIdx.x * kThreads + threadIdx.x; f < TC;
       f += (int64_t)gridDim.x * kThreads) {
    U a = 0;
    for (int64_t b = 0; b < B; ++b) a += to_acc(dout[b * TC + f]);
    if (accumulate) a += to_acc(dwpe[f]);
    dwpe[f] = from_acc<T>(a);
  }
}

// --------------------------------------------- backward: general (slow) path
// For fp64 and for rows that are not whole aligned 16-byte vectors.  Same
// sorted order, one workgroup per output row found by binary search.
template <typename T>
__global__ __launch_bounds__(kThreads) void emb_bwd_rows_general_kernel(
    const T *__restrict__ dout, const uint32_t *__restrict__ sorted_id,
    const uint32_t *__restrict__ sorted_pos, T *__restrict__ dweight, int64_t n, int64_t C,
    int accumulate) {
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
  for (int64_t c = threadIdx.x; c < C; c += kThreads) {
    U a = 0;
    for (int64_t p = lo; p < n && sorted_id[p] == row; ++p)
      a += to_acc(dout[(int64_t)sorted_pos[p] * C + c]);
    if (accumulate) a += to_acc(dweight[(int64_t)row * C + c]);
    dweight[(int64_t)row * C + c] = from_acc<T>(a);
  }
}

// ---------------------------------------------------------------- workspace
struct BwdLayout {
  int shift = 0;
  bool key64 = false;
  int64_t n_tiles = 0;
  int64_t bitmap_words = 0;
  int64_t n_windows = 0;
  size_t off_bitmap = 0, off_tiles = 0, off_sorted_id = 0, off_sorted_pos = 0, off_partial = 0;
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
  L.bitmap_words = ceil_div(num_weights, (int64_t)32);
  L.n_windows = ceil_div(n, (int64_t)kWin);
  size_t o = 0;
  L.off_bitmap = o;
  o = align256(o + (size_t)L.bitmap_words * 4);
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
    const int64_t blocks = ceil_div(total, (int64_t)kThreads * 4);
    if (blocks > 0x7fffffffLL) return CS_ERR_TOO_LARGE;
    emb_fwd_vec_kernel<T, IdxT, ADD><<<dim3((unsigned)blocks), dim3(kThreads), 0, s>>>(
        (const T *)weight, (const T *)wpe, (const IdxT *)ids, (T *)out, n_rows, (int)(C / VN),
        num_weights, T_len);
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
  if (!aligned_to(weight, es) || !aligned_to(out, es) || (ADD && !aligned_to(wpe, es)) ||
      !aligned_to(ids, idx_dtype == CS_I64 ? 8 : 4))
    return CS_ERR_MISALIGNED;
  hipStream_t s = as_stream(stream);
  // a plain gather is a byte copy: 16-bit types share one kernel
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

template <typename KeyT, typename IdxT>
int sort_launch(const void *ids, char *ws, const BwdLayout &L, int64_t n, int64_t num_weights,
                int64_t padding_idx, hipStream_t s) {
  KeyT *tiles = reinterpret_cast<KeyT *>(ws + L.off_tiles);
  uint32_t *bitmap = reinterpret_cast<uint32_t *>(ws + L.off_bitmap);
  uint32_t *sorted_id = reinterpret_cast<uint32_t *>(ws + L.off_sorted_id);
  uint32_t *sorted_pos = reinterpret_cast<uint32_t *>(ws + L.off_sorted_pos);
  const int extra = 8;  // blocks that clear the bitmap and preset sorted_id
  emb_bwd_tile_sort_kernel<KeyT, IdxT>
      <<<dim3((unsigned)(L.n_tiles + extra)), dim3(kSortThreads), 0, s>>>(
          (const IdxT *)ids, tiles, bitmap, (int)L.bitmap_words, sorted_id, n, (int)L.n_tiles,
          L.shift, num_weights, padding_idx);
  int st = launch_status();
  if (st != CS_OK) return st;
  const int64_t blocks = ceil_div(L.n_tiles * kTile, (int64_t)kThreads);
  emb_bwd_merge_kernel<KeyT><<<dim3((unsigned)blocks), dim3(kThreads), 0, s>>>(
      tiles, bitmap, sorted_id, sorted_pos, (int)L.n_tiles, L.shift);
  return launch_status();
}

template <typename T>
int bwd_typed(const void *dout, const void *ids, void *dweight, void *dwpe, char *ws,
              const BwdLayout &L, int64_t n, int64_t C, int64_t num_weights, int64_t padding_idx,
              int64_t B, int64_t T_len, int idx_dtype, int accumulate, hipStream_t s) {
  int st;
  if (L.key64) {
    st = idx_dtype == CS_I64
             ? sort_launch<uint64_t, int64_t>(ids, ws, L, n, num_weights, padding_idx, s)
             : sort_launch<uint64_t, int32_t>(ids, ws, L, n, num_weights, padding_idx, s);
  } else {
    st = idx_dtype == CS_I64
             ? sort_launch<uint32_t, int64_t>(ids, ws, L, n, num_weights, padding_idx, s)
             : sort_launch<uint32_t, int32_t>(ids, ws, L, n, num_weights, padding_idx, s);
  }
  if (st != CS_OK) return st;
  const uint32_t *bitmap = reinterpret_cast<const uint32_t *>(ws + L.off_bitmap);
  const uint32_t *sorted_id = reinterpret_cast<const uint32_t *>(ws + L.off_sorted_id);
  const uint32_t *sorted_pos = reinterpret_cast<const uint32_t *>(ws + L.off_sorted_pos);
  float *partial = reinterpret_cast<float *>(ws + L.off_partial);
  constexpr int VN = Vec16<T>::n;
  const bool vec_ok = !std::is_same_v<T, double> && C % VN == 0 && C % 4 == 0 &&
                      is_aligned16(dout) && is_aligned16(dweight) && (!dwpe || is_aligned16(dwpe));
  if (!vec_ok) {
    if (num_weights > 0x7fffffffLL) return CS_ERR_TOO_LARGE;
    emb_bwd_rows_general_kernel<T><<<dim3((unsigned)num_weights), dim3(kThreads), 0, s>>>(
        (const T *)dout, sorted_id, sorted_pos, (T *)dweight, n, C, accumulate);
    st = launch_status();
    if (st != CS_OK || !dwpe) return st;
    int64_t blocks = ceil_div(T_len * C, (int64_t)kThreads);
    if (blocks > 65536) blocks = 65536;
    emb_bwd_positions_kernel<T><<<dim3((unsigned)blocks), dim3(kThreads), 0, s>>>(
        (const T *)dout, (T *)dwpe, B, T_len * C, accumulate);
    return launch_status();
  }
  if constexpr (!std::is_same_v<T, double>) {
    const int64_t win_blocks = ceil_div(L.n_windows, (int64_t)(kThreads / kWave));
    emb_bwd_window_kernel<T><<<dim3((unsigned)win_blocks), dim3(kThreads), 0, s>>>(
        (const T *)dout, sorted_id, sorted_pos, (T *)dweight, partial, n, C, accumulate);
    st = launch_status();
    if (st != CS_OK) return st;
    const int64_t nvec = C / VN;
    const int64_t pos_blocks = dwpe ? ceil_div(T_len * nvec, (int64_t)kFinThreads) : 0;
    const int64_t fill_blocks =
        accumulate ? 0 : ceil_div(num_weights * nvec, (int64_t)kFinThreads * 4);
    const int64_t blocks = L.n_windows + pos_blocks + fill_blocks;
    if (blocks > 0x7fffffffLL) return CS_ERR_TOO_LARGE;
    const size_t lds = (size_t)kFinGroups * 256 * 4 * sizeof(float);
    emb_bwd_finish_kernel<T><<<dim3((unsigned)blocks), dim3(kFinThreads), lds, s>>>(
        (const T *)dout, sorted_id, bitmap, partial, (T *)dweight, (T *)dwpe, n, C, num_weights, B,
        T_len, L.n_windows, pos_blocks, accumulate, accumulate ? 0 : 1);
    return launch_status();
  }
  return CS_ERR_UNSUPPORTED;
}

int bwd_dispatch(const void *dout, const void *ids, void *dweight, void *dwpe, void *workspace,
                 size_t workspace_bytes, int64_t n, int64_t C, int64_t num_weights,
                 int64_t padding_idx, int64_t B, int64_t T_len, int dtype, int idx_dtype,
                 int accumulate, void *stream) {
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
                              T_len, idx_dtype, accumulate, s);
    case CS_F64:
      return bwd_typed<double>(dout, ids, dweight, dwpe, ws, L, n, C, num_weights, padding_idx, B,
                               T_len, idx_dtype, accumulate, s);
    case CS_F16:
      return bwd_typed<f16_t>(dout, ids, dweight, dwpe, ws, L, n, C, num_weights, padding_idx, B,
                              T_len, idx_dtype, accumulate, s);
    case CS_BF16:
      return bwd_typed<bf16_t>(dout, ids, dweight, dwpe, ws, L, n, C, num_weights, padding_idx, B,
                               T_len, idx_dtype, accumulate, s);
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
  int64_t blocks = ceil_div(T * C, (int64_t)kThreads);
  if (blocks > 65536) blocks = 65536;
  hipStream_t s = as_stream(stream);
  const dim3 grid((unsigned)blocks), block(kThreads);
  switch (dtype) {
    case CS_F32:
      emb_bwd_positions_kernel<float><<<grid, block, 0, s>>>((const float *)dout, (float *)dwpe, B, T * C, accumulate);
      break;
    case CS_F64:
      emb_bwd_positions_kernel<double><<<grid, block, 0, s>>>((const double *)dout, (double *)dwpe, B, T * C, accumulate);
      break;
    case CS_F16:
      emb_bwd_positions_kernel<f16_t><<<grid, block, 0, s>>>((const f16_t *)dout, (f16_t *)dwpe, B, T * C, accumulate);
      break;
    case CS_BF16:
      emb_bwd_positions_kernel<bf16_t><<<grid, block, 0, s>>>((const bf16_t *)dout, (bf16_t *)dwpe, B, T * C, accumulate);
      break;
  }
  return launch_status();
}
