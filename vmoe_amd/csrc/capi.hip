// Version and error-string entry points of libvmoe_hip.so.
#include "vmoe_common.h"

extern "C" int vmoe_abi_version(void) { return VMOE_ABI_VERSION; }

extern "C" const char* vmoe_error_string(int code) {
  switch (code) {
    case VMOE_OK: return "ok";
    case VMOE_E_NULL: return "a required pointer is null";
    case VMOE_E_SHAPE: return "invalid sizes (size < 1, K > E, or sizes that disagree)";
    case VMOE_E_DTYPE: return "unknown dtype or enum value";
    case VMOE_E_ALIGN: return "row width or pointer not aligned to 16 bytes";
    case VMOE_E_OVERFLOW: return "an index would overflow int32";
    case VMOE_E_UNSUPPORTED: return "sizes outside what the kernels cover";
    case VMOE_E_WORKSPACE: return "workspace missing, misaligned or too small";
    default: return code > 0 ? hipGetErrorString((hipError_t)code) : "unknown vmoe error";
  }
}
