// ABI bookkeeping: version and error strings.
#include "kx_common.h"

extern "C" int kx_abi_version(void) {
    return KX_ABI_VERSION;
}

extern "C" const char* kx_error_string(int code) {
    switch (code) {
        case KX_OK: return "ok";
        case KX_ERR_NULL_POINTER: return "a required pointer is null";
        case KX_ERR_BAD_SHAPE: return "shape or group size not accepted by the kernels";
        case KX_ERR_WORKSPACE: return "workspace missing or too small (see kx_gemv_workspace_bytes)";
        case KX_ERR_ALIGNMENT: return "pointer not aligned as the interface requires";
        case KX_ERR_ALIAS: return "an output overlaps an input that is still being read";
        default: break;
    }
    if (code > 0) return hipGetErrorString(static_cast<hipError_t>(code));
    return "unknown kx error code";
}
