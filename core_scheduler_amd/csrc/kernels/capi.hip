// Version and error reporting of the C ABI, and the plain copy kernel used to
// calibrate bandwidth measurements.
#include "common.cuh"

namespace cs_hip {
namespace {

constexpr int kCopyThreads = 256;
constexpr int kCopyUnroll = 4;

// dst[i] = src[i] over 16-byte vectors: the simplest HBM-bound kernel there
// is (one read and one write per byte).  What it reaches is the practical
// ceiling the other kernels are compared with, and what a hardware traffic
// counter reads for it is the counter's scale.
__global__ __launch_bounds__(kCopyThreads) void stream_copy_kernel(const u32x4 *__restrict__ src,
                                                                   u32x4 *__restrict__ dst,
                                                                   int64_t nvec) {
  const int64_t base = (int64_t)blockIdx.x * (kCopyThreads * kCopyUnroll) + threadIdx.x;
  u32x4 v[kCopyUnroll];
#pragma unroll
  for (int u = 0; u < kCopyUnroll; ++u) {
    const int64_t i = base + (int64_t)u * kCopyThreads;
    if (i < nvec) v[u] = __builtin_nontemporal_load(src + i);
  }
#pragma unroll
  for (int u = 0; u < kCopyUnroll; ++u) {
    const int64_t i = base + (int64_t)u * kCopyThreads;
    if (i < nvec) __builtin_nontemporal_store(v[u], dst + i);
  }
}

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
  const int64_t blocks = ceil_div(nvec, (int64_t)kCopyThreads * kCopyUnroll);
  if (blocks > 0x7fffffffLL) return CS_ERR_TOO_LARGE;
  stream_copy_kernel<<<dim3((unsigned)blocks), dim3(kCopyThreads), 0, as_stream(stream)>>>(
      static_cast<const u32x4 *>(src), static_cast<u32x4 *>(dst), nvec);
  return launch_status();
}
