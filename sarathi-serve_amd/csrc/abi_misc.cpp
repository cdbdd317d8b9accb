// Version and error-string entry points of the C ABI.
#include "../../include/sarathi_ops.h"

extern "C" int sarathi_ops_abi_version(void) { return SARATHI_OPS_ABI_VERSION; }

extern "C" const char* sarathi_ops_strerror(int code) {
  switch (code) {
    case SARATHI_OK: return "ok";
    case SARATHI_ERR_INVALID_ARG: return "invalid argument (null pointer, negative size or bad stride)";
    case SARATHI_ERR_UNSUPPORTED: return "unsupported dtype code or shape outside the library's limits";
    case SARATHI_ERR_LAUNCH: return "the HIP runtime rejected the kernel launch";
    case SARATHI_ERR_SCRATCH_LIMIT:
      return "the input needs more scratch than the fixed array of the non-allocating entry point holds";
    default: return "unknown sarathi_ops error code";
  }
}
