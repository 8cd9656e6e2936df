// Version and error-string entry points of libattorch_hip.
#include "at_common.h"

extern "C" {

int at_version(void) { return 100; }

const char* at_error_string(int code) {
  switch (code) {
    case AT_OK: return "success";
    case AT_ERR_NULL: return "a required pointer is null";
    case AT_ERR_DIM: return "a dimension or stride is out of range";
    case AT_ERR_DTYPE: return "unknown dtype or unsupported dtype combination";
    case AT_ERR_ACT: return "unknown activation id";
    case AT_ERR_WORKSPACE: return "workspace missing or too small";
    case AT_ERR_ALIGN: return "pointer or stride alignment the kernel cannot serve";
    case AT_ERR_UNSUPPORTED: return "configuration not implemented";
    default: return code > 0 ? "HIP runtime error (hipError_t)" : "unknown error code";
  }
}

}  // extern "C"
