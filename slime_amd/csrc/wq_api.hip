// ABI version and error strings of libslime_amd_wq.so.

#include "wq_common.h"

WQ_EXPORT int wq_abi_version(void) { return WQ_ABI_VERSION; }

WQ_EXPORT const char* wq_error_string(int code)
{
    switch (code) {
    case WQ_OK: return "success";
    case WQ_ERR_NULL: return "a required pointer is NULL";
    case WQ_ERR_SHAPE: return "invalid shape, block or group size";
    case WQ_ERR_MODE: return "unknown mode or dtype selector";
    case WQ_ERR_UNSUPPORTED: return "configuration not supported by this library";
    case WQ_ERR_ALIGN: return "pointer or stride alignment requirement violated";
    case WQ_ERR_TOO_LARGE: return "count exceeds the limits of this entry point";
    default: break;
    }
    if (code > 0) return hipGetErrorString((hipError_t)code);
    return "unknown error";
}
