// Version and error reporting of the C ABI, and the plain copy kernel used to
// calibrate bandwidth measurements.
#include "common.hpp"

namespace cs_hip {
namespace {

constexpr int kCopyThreads = 256;

// dst[i] = src[i] over 16-byte vectors: the simplest HBM-bound kernel there is (one read and
// one write per byte).  What it reaches is the practical ceiling the other kernels are compared
// with, and what a hardware traffic counter reads for it is the counter's scale.  U vectors per
// lane; every load of a full chunk is issued unconditionally (a load under a lane-dependent
// condition makes the compiler wait for it before the next one).  Measured on MI355X: one vector
// per lane is fastest for large buffers (6.7 TB/s at 1.6 GB against 6.2 with four), two for small
// ones (4.9 us against 5.7 us for 25 MB).
template <int U>
__global__ __launch_bounds__(kCopyThreads) void stream_copy_kernel(const u32x4 *__restrict__ src,
                                                                   u32x4 *__restrict__ dst,
                                                                   int64_t nvec) {
  const int64_t base = (int64_t)blockIdx.x * (kCopyThreads * U) + threadIdx.x;
  if (base - threadIdx.x + kCopyThreads * U <= nvec) {  // block-uniform: a full chunk
    u32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = __builtin_nontemporal_load(src + base + (int64_t)u * kCopyThreads);
#pragma unroll
    for (int u = 0; u < U; ++u) store_stream(dst + base + (int64_t)u * kCopyThreads, v[u]);
    return;
  }
  for (int u = 0; u < U; ++u) {
    const int64_t i = base + (int64_t)u * kCopyThreads;
    if (i < nvec) dst[i] = src[i];
  }
}

// Read-only calibration: every workgroup reads its chunk and leaves one word (the xor of what it
// read) in out[blockIdx.x], so the loads cannot be dropped and the writes are negligible.
constexpr int kReadUnroll = 4;
__global__ __launch_bounds__(kCopyThreads) void stream_read_kernel(const u32x4 *__restrict__ src,
                                                                   uint32_t *__restrict__ out,
                                                                   int64_t nvec) {
  __shared__ uint32_t part[kCopyThreads / kWave];
  const int64_t base = (int64_t)blockIdx.x * (kCopyThreads * kReadUnroll) + threadIdx.x;
  uint32_t x = 0;
  if (base - threadIdx.x + kCopyThreads * kReadUnroll <= nvec) {
    u32x4 v[kReadUnroll];
#pragma unroll
    for (int u = 0; u < kReadUnroll; ++u) v[u] = __builtin_nontemporal_load(src + base + (int64_t)u * kCopyThreads);
#pragma unroll
    for (int u = 0; u < kReadUnroll; ++u) x ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  } else {
    for (int u = 0; u < kReadUnroll; ++u) {
      const int64_t i = base + (int64_t)u * kCopyThreads;
      if (i < nvec) {
        const u32x4 v = src[i];
        x ^= v.x ^ v.y ^ v.z ^ v.w;
      }
    }
  }
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) x ^= (uint32_t)__shfl_xor((int)x, off, kWave);
  if ((threadIdx.x & (kWave - 1)) == 0) part[threadIdx.x >> 6] = x;
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t t = 0;
#pragma unroll
    for (int w = 0; w < kCopyThreads / kWave; ++w) t ^= part[w];
    out[blockIdx.x] = t;
  }
}

// Write-only calibration: dst[i] = value.  One 16-byte vector per lane, one chunk per workgroup:
// the best of a sweep over 256 / 512 / 1024 lanes, 1 / 2 / 4 / 8 vectors per lane, lane-strided
// chunks against whole kilobytes per wave, one chunk per workgroup against 4 / 8 / 16 persistent
// workgroups per CU, nontemporal against plain stores (120 shapes, MI355X).  At 3.5 GB it writes
// 6.7 TB/s (plain stores 6.9), at 400 MB 6.7, at 100 MB 6.3, at 77 MB 6.1, at 25 MB 4.7-5.0
// (every shape within 10% there); four vectors per lane lose 11% at the large sizes, persistent
// grids up to 40%.
constexpr int kFillUnroll = 1;
__global__ __launch_bounds__(kCopyThreads) void stream_fill_kernel(u32x4 *__restrict__ dst, int64_t nvec,
                                                                   uint32_t value) {
  const int64_t base = (int64_t)blockIdx.x * (kCopyThreads * kFillUnroll) + threadIdx.x;
  const u32x4 v = {value, value, value, value};
  if (base - threadIdx.x + kCopyThreads * kFillUnroll <= nvec) {
#pragma unroll
    for (int u = 0; u < kFillUnroll; ++u) store_stream(dst + base + (int64_t)u * kCopyThreads, v);
    return;
  }
  for (int u = 0; u < kFillUnroll; ++u) {
    const int64_t i = base + (int64_t)u * kCopyThreads;
    if (i < nvec) dst[i] = v;
  }
}

// The traffic of an optimizer step without its arithmetic: four arrays read, three of them
// written back in place (AdamW reads g, w, m, v and writes w, m, v).  Same chunking as the
// multi-tensor AdamW kernel: four vectors per lane per array, every wave owning four consecutive
// kilobytes of each array, every load issued before the first use.
constexpr int kUpdateUnroll = 4;
__device__ __forceinline__ int64_t update_index(int64_t chunk_base, int u, int tid) {
  return chunk_base + (tid >> 6) * (kWave * kUpdateUnroll) + u * kWave + (tid & (kWave - 1));
}
__global__ __launch_bounds__(kCopyThreads) void stream_update4_kernel(const u32x4 *__restrict__ a0,
                                                                      u32x4 *__restrict__ a1,
                                                                      u32x4 *__restrict__ a2,
                                                                      u32x4 *__restrict__ a3, int64_t nvec) {
  const int64_t chunk_base = (int64_t)blockIdx.x * (kCopyThreads * kUpdateUnroll);
  const int tid = threadIdx.x;
  if (chunk_base + kCopyThreads * kUpdateUnroll <= nvec) {
    u32x4 v0[kUpdateUnroll], v1[kUpdateUnroll], v2[kUpdateUnroll], v3[kUpdateUnroll];
#pragma unroll
    for (int u = 0; u < kUpdateUnroll; ++u) {
      const int64_t i = update_index(chunk_base, u, tid);
      v0[u] = __builtin_nontemporal_load(a0 + i);
      v1[u] = __builtin_nontemporal_load(a1 + i);
      v2[u] = __builtin_nontemporal_load(a2 + i);
      v3[u] = __builtin_nontemporal_load(a3 + i);
    }
#pragma unroll
    for (int u = 0; u < kUpdateUnroll; ++u) {
      const int64_t i = update_index(chunk_base, u, tid);
      const u32x4 x = v0[u] ^ v1[u] ^ v2[u] ^ v3[u];
      store_stream(a1 + i, x + 1u);
      store_stream(a2 + i, x + 2u);
      store_stream(a3 + i, x + 3u);
    }
    return;
  }
  for (int u = 0; u < kUpdateUnroll; ++u) {
    const int64_t i = chunk_base + (int64_t)u * kCopyThreads + tid;
    if (i < nvec) {
      const u32x4 x = a0[i] ^ a1[i] ^ a2[i] ^ a3[i];
      a1[i] = x + 1u;
      a2[i] = x + 2u;
      a3[i] = x + 3u;
    }
  }
}

// The write-only kernel in the launch shapes cs_stream_fill's own was chosen from: THREADS lanes
// per workgroup, U vectors per lane, lane-strided chunks (LAYOUT 0: lane i writes vectors
// base + u*THREADS + i) or whole kilobytes per wave (1), nontemporal (STORE 0) or plain stores,
// and one chunk per workgroup or a fixed number of workgroups walking the chunks.
template <int THREADS, int U, int LAYOUT, int STORE>
__global__ __launch_bounds__(THREADS) void stream_fill_shape_kernel(u32x4 *__restrict__ dst, int64_t nvec,
                                                                    int64_t chunks_per_block, uint32_t value) {
  const u32x4 v = {value, value, value, value};
  const int tid = threadIdx.x;
  for (int64_t c = 0; c < chunks_per_block; ++c) {
    const int64_t base = ((int64_t)blockIdx.x + c * gridDim.x) * (THREADS * U);
    if (base + THREADS * U > nvec) {  // block-uniform: the ragged end
      for (int u = 0; u < U; ++u) {
        const int64_t i = base + (int64_t)u * THREADS + tid;
        if (i < nvec) dst[i] = v;
      }
      continue;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t i = LAYOUT == 0 ? base + (int64_t)u * THREADS + tid
                                    : base + (int64_t)(tid >> 6) * (kWave * U) + u * kWave + (tid & (kWave - 1));
      if constexpr (STORE == 0) {
        store_stream(dst + i, v);
      } else {
        dst[i] = v;
      }
    }
  }
}
template <int THREADS, int U, int LAYOUT, int STORE>
int launch_fill_shape(void *dst, int64_t nvec, int64_t workgroups_per_cu, uint32_t value, hipStream_t s) {
  const int64_t chunks = ceil_div(nvec, (int64_t)THREADS * U);
  int64_t blocks = chunks, per = 1;
  if (workgroups_per_cu > 0) {  // a persistent grid, sized for 256 CUs
    blocks = workgroups_per_cu * 256 < chunks ? workgroups_per_cu * 256 : chunks;
    per = ceil_div(chunks, blocks);
  }
  if (blocks > 0x7fffffffLL) return CS_ERR_TOO_LARGE;
  stream_fill_shape_kernel<THREADS, U, LAYOUT, STORE><<<dim3((unsigned)blocks), dim3(THREADS), 0, s>>>(
      static_cast<u32x4 *>(dst), nvec, per, value);
  return launch_status();
}

// bytes from which the copy uses one vector per lane instead of two
constexpr int64_t kCopyLargeBytes = 64ll << 20;

}  // namespace
}  // namespace cs_hip

using namespace cs_hip;

extern "C" int cs_hip_abi_version(void) { return CS_HIP_ABI_VERSION; }

extern "C" const char *cs_hip_error_string(int code) {
  switch (code) {
    case CS_OK: return "ok";
    case CS_ERR_INVALID_ARGUMENT: return "invalid argument (null pointer, negative size or bad enum)";
    case CS_ERR_UNSUPPORTED: return "unsupported dtype combination";
    case CS_ERR_MISALIGNED: return "pointer not aligned to its element size";
    case CS_ERR_WORKSPACE: return "workspace missing, misaligned or too small";
    case CS_ERR_TOO_LARGE: return "size beyond what one launch can address";
    case CS_ERR_STATIC_LIMIT:
      return "size beyond the library's built-in scratch buffer; use the entry point that takes a workspace";
    default: break;
  }
  if (code > 0) return hipGetErrorString(static_cast<hipError_t>(code));
  return "unknown error";
}

extern "C" int cs_stream_copy(void *dst, const void *src, int64_t bytes, void *stream) {
  if (bytes < 0 || bytes % 16 != 0) return CS_ERR_INVALID_ARGUMENT;
  if (bytes == 0) return CS_OK;
  if (!dst || !src) return CS_ERR_INVALID_ARGUMENT;
  if (!is_aligned16(dst) || !is_aligned16(src)) return CS_ERR_MISALIGNED;
  const int64_t nvec = bytes / 16;
  const int unroll = bytes >= kCopyLargeBytes ? 1 : 2;
  const int64_t blocks = ceil_div(nvec, (int64_t)kCopyThreads * unroll);
  if (blocks > 0x7fffffffLL) return CS_ERR_TOO_LARGE;
  const dim3 grid((unsigned)blocks), block(kCopyThreads);
  if (unroll == 1) {
    stream_copy_kernel<1><<<grid, block, 0, as_stream(stream)>>>(static_cast<const u32x4 *>(src),
                                                                 static_cast<u32x4 *>(dst), nvec);
  } else {
    stream_copy_kernel<2><<<grid, block, 0, as_stream(stream)>>>(static_cast<const u32x4 *>(src),
                                                                 static_cast<u32x4 *>(dst), nvec);
  }
  return launch_status();
}

extern "C" int64_t cs_stream_read_out_words(int64_t bytes) {
  return bytes <= 0 ? 0 : ceil_div(bytes / 16, (int64_t)kCopyThreads * kReadUnroll);
}

extern "C" int cs_stream_read(const void *src, void *out, int64_t bytes, void *stream) {
  if (bytes < 0 || bytes % 16 != 0) return CS_ERR_INVALID_ARGUMENT;
  if (bytes == 0) return CS_OK;
  if (!src || !out) return CS_ERR_INVALID_ARGUMENT;
  if (!is_aligned16(src) || !aligned_to(out, 4)) return CS_ERR_MISALIGNED;
  const int64_t nvec = bytes / 16;
  const int64_t blocks = cs_stream_read_out_words(bytes);
  if (blocks > 0x7fffffffLL) return CS_ERR_TOO_LARGE;
  stream_read_kernel<<<dim3((unsigned)blocks), dim3(kCopyThreads), 0, as_stream(stream)>>>(
      static_cast<const u32x4 *>(src), static_cast<uint32_t *>(out), nvec);
  return launch_status();
}

extern "C" int cs_stream_fill(void *dst, int64_t bytes, uint32_t value, void *stream) {
  if (bytes < 0 || bytes % 16 != 0) return CS_ERR_INVALID_ARGUMENT;
  if (bytes == 0) return CS_OK;
  if (!dst) return CS_ERR_INVALID_ARGUMENT;
  if (!is_aligned16(dst)) return CS_ERR_MISALIGNED;
  const int64_t nvec = bytes / 16;
  const int64_t blocks = ceil_div(nvec, (int64_t)kCopyThreads * kFillUnroll);
  if (blocks > 0x7fffffffLL) return CS_ERR_TOO_LARGE;
  stream_fill_kernel<<<dim3((unsigned)blocks), dim3(kCopyThreads), 0, as_stream(stream)>>>(
      static_cast<u32x4 *>(dst), nvec, value);
  return launch_status();
}

extern "C" int cs_stream_fill_shape(void *dst, int64_t bytes, uint32_t value, int lanes, int vectors_per_lane,
                                    int wave_kilobytes, int plain_stores, int workgroups_per_cu, void *stream) {
  if (bytes < 0 || bytes % 16 != 0 || workgroups_per_cu < 0) return CS_ERR_INVALID_ARGUMENT;
  if (bytes == 0) return CS_OK;
  if (!dst) return CS_ERR_INVALID_ARGUMENT;
  if (!is_aligned16(dst)) return CS_ERR_MISALIGNED;
  hipStream_t s = as_stream(stream);
  const int64_t nvec = bytes / 16;
#define CS_SHAPE(T, U, L, S)                                                                     \
  if (lanes == T && vectors_per_lane == U && (wave_kilobytes != 0) == (L != 0) && (plain_stores != 0) == (S != 0)) \
    return launch_fill_shape<T, U, L, S>(dst, nvec, workgroups_per_cu, value, s);
#define CS_SHAPES(T, U) CS_SHAPE(T, U, 0, 0) CS_SHAPE(T, U, 1, 0) CS_SHAPE(T, U, 0, 1) CS_SHAPE(T, U, 1, 1)
  CS_SHAPES(256, 1) CS_SHAPES(256, 2) CS_SHAPES(256, 4) CS_SHAPES(256, 8)
  CS_SHAPES(1024, 1) CS_SHAPES(1024, 2) CS_SHAPES(1024, 4) CS_SHAPES(1024, 8)
#undef CS_SHAPES
#undef CS_SHAPE
  return CS_ERR_UNSUPPORTED;
}

extern "C" int cs_stream_update4(const void *a0, void *a1, void *a2, void *a3, int64_t bytes, void *stream) {
  if (bytes < 0 || bytes % 16 != 0) return CS_ERR_INVALID_ARGUMENT;
  if (bytes == 0) return CS_OK;
  if (!a0 || !a1 || !a2 || !a3) return CS_ERR_INVALID_ARGUMENT;
  if (!is_aligned16(a0) || !is_aligned16(a1) || !is_aligned16(a2) || !is_aligned16(a3)) return CS_ERR_MISALIGNED;
  const int64_t nvec = bytes / 16;
  const int64_t blocks = ceil_div(nvec, (int64_t)kCopyThreads * kUpdateUnroll);
  if (blocks > 0x7fffffffLL) return CS_ERR_TOO_LARGE;
  stream_update4_kernel<<<dim3((unsigned)blocks), dim3(kCopyThreads), 0, as_stream(stream)>>>(
      static_cast<const u32x4 *>(a0), static_cast<u32x4 *>(a1), static_cast<u32x4 *>(a2),
      static_cast<u32x4 *>(a3), nvec);
  return launch_status();
}
