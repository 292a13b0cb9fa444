// Library-level entry points of the C ABI.
#include "common.h"

extern "C" int axon_amd_abi_version(void) { return AXON_AMD_ABI_VERSION; }

extern "C" const char* axon_amd_error_string(int code) {
  switch (code) {
    case AXON_OK: return "ok";
    case AXON_ERR_ARG: return "invalid argument (null pointer, bad enum or scalar)";
    case AXON_ERR_SHAPE: return "shape constraint violated";
    case AXON_ERR_WORKSPACE: return "workspace too small";
    case AXON_ERR_LAUNCH: return "kernel launch failed";
    case AXON_ERR_DEVICE: return "device is not gfx950";
    case AXON_ERR_TOO_LARGE: return "input larger than the fixed capacity of the no-allocation entry point";
    default: return "unknown error code";
  }
}
