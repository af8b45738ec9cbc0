// Version and status text of the C ABI.
#include "cce_common.h"

extern "C" int cce_version(void) { return 8; }

#ifndef CCE_SOURCE_HASH
#define CCE_SOURCE_HASH "unknown"
#endif
extern "C" const char* cce_source_hash(void) { return CCE_SOURCE_HASH; }

extern "C" const char* cce_error_string(int status) {
  switch (status) {
    case CCE_OK: return "success";
    case CCE_ERR_INVALID_ARGUMENT: return "cce: invalid argument";
    case CCE_ERR_UNSUPPORTED_DTYPE: return "cce: unsupported element type (bf16 and fp16 only)";
    case CCE_ERR_WORKSPACE_TOO_SMALL: return "cce: workspace missing or too small";
    case CCE_ERR_MISALIGNED: return "cce: pointer not aligned as required";
    case CCE_ERR_STATIC_SCRATCH_LIMIT:
      return "cce: shape needs more scratch than the static array holds (CCE_STATIC_SCRATCH_BYTES); "
             "use the entry point that takes a workspace";
    default: return hipGetErrorString(static_cast<hipError_t>(status));
  }
}
