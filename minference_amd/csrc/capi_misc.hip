// Version and status text of libminf_hip.so.
#include "minf_common.h"

extern "C" int minf_version(void) { return 300; }   // 0.3.0

extern "C" size_t minf_qkvo_size(void) { return sizeof(minf_qkvo); }

extern "C" const char *minf_status_string(int status) {
    switch (status) {
        case MINF_OK: return "ok";
        case MINF_ERR_INVALID_ARG: return "invalid argument";
        case MINF_ERR_UNSUPPORTED: return "unsupported shape, dtype or block size";
        case MINF_ERR_ALIGNMENT: return "pointer or stride not 16-byte aligned / last stride not 1";
        case MINF_ERR_WORKSPACE: return "workspace too small";
        default: break;
    }
    if (status <= MINF_ERR_HIP_BASE) return hipGetErrorString((hipError_t)(MINF_ERR_HIP_BASE - status));
    return "unknown status";
}
