// Version and status-string entry points of the C ABI.
#include "stof_common.h"

extern "C" int stof_abi_version(void) { return STOF_ABI_VERSION; }

extern "C" const char* stof_status_string(int status) {
  switch (status) {
    case STOF_OK: return "ok";
    case STOF_ERR_NULL_POINTER: return "a required pointer is NULL";
    case STOF_ERR_BAD_SHAPE: return "bad shape: a size is non-positive, not divisible as required, or too large";
    case STOF_ERR_UNSUPPORTED: return "unsupported head size, block size or mode";
    case STOF_ERR_MISALIGNED: return "pointer or stride is not aligned for 16-byte vector access";
    case STOF_ERR_LAUNCH: return "kernel launch failed";
    case STOF_ERR_BAD_LUT: return "inconsistent block LUT description";
    case STOF_ERR_TOO_LARGE: return "the problem exceeds the fixed scratch memory of this entry point (use the variant that takes a workspace)";
    default: return "unknown status";
  }
}
