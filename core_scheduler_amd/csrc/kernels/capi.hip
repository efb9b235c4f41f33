// Version and error reporting of the C ABI.
#include "common.cuh"

extern "C" int cs_hip_abi_version(void) { return CS_HIP_ABI_VERSION; }

extern "C" const char *cs_hip_error_string(int code) {
  switch (code) {
    case CS_OK: return "ok";
    case CS_ERR_INVALID_ARGUMENT: return "invalid argument (null pointer, negative size or bad enum)";
    case CS_ERR_UNSUPPORTED: return "unsupported dtype combination";
    case CS_ERR_MISALIGNED: return "pointer not aligned to its element size";
    case CS_ERR_WORKSPACE: return "workspace missing, misaligned or too small";
    case CS_ERR_TOO_LARGE: return "size beyond what one launch can address";
    default: break;
  }
  if (code > 0) return hipGetErrorString(static_cast<hipError_t>(code));
  return "unknown error";
}
