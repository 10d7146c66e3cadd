// Version and status text of the C ABI declared in include/minivllm_amd.h.
#include "common.h"

extern "C" int mvllm_version(void) { return 1 * 1000 + 6; }

extern "C" const char* mvllm_status_string(int status) {
  switch (status) {
    case MVLLM_OK: return "ok";
    case MVLLM_ERR_NULL_POINTER: return "null pointer argument";
    case MVLLM_ERR_BAD_DTYPE: return "unknown dtype code";
    case MVLLM_ERR_BAD_SHAPE: return "invalid size argument";
    case MVLLM_ERR_UNSUPPORTED: return "shape not supported by any built kernel";
    case MVLLM_ERR_WORKSPACE: return "workspace missing, misaligned or too small";
    case MVLLM_ERR_MISALIGNED: return "pointer not 16-byte aligned";
    default: return status > 0 ? "hip runtime error" : "unknown status";
  }
}
