// Small entry points of the C ABI that belong to no kernel file.
#include "pdllm_common.h"

extern "C" const char* pdllm_status_string(int status) {
  switch (status) {
    case PDLLM_OK: return "ok";
    case PDLLM_ERR_NULL: return "required pointer is NULL";
    case PDLLM_ERR_SHAPE: return "size is negative, inconsistent or out of range";
    case PDLLM_ERR_STRIDE: return "stride or alignment requirement not met";
    case PDLLM_ERR_DTYPE: return "unknown dtype or mode";
    case PDLLM_ERR_WORKSPACE: return "workspace missing, misaligned or too small";
    case PDLLM_ERR_LAUNCH: return "kernel launch failed";
    case PDLLM_ERR_UNSUPPORTED: return "request not covered by the kernels";
    case PDLLM_ERR_SCRATCH_LIMIT: return "input exceeds the static device scratch of this entry point";
    default: return "unknown status";
  }
}

extern "C" int pdllm_abi_version(void) { return 5; }
