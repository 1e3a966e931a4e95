// Internal helpers shared by the gfx950 kernels of libminf_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/minf_hip.h"

#define MINF_WAVE 64

static inline int minf_hip_status(hipError_t e) {
    return e == hipSuccess ? MINF_OK : MINF_ERR_HIP_BASE - (int)e;
}

// Status of the launch that was just enqueued on `stream` (does not synchronise).
static inline int minf_launch_status() { return minf_hip_status(hipGetLastError()); }

__device__ __forceinline__ int minf_lane() { return (int)(threadIdx.x & 63); }

__device__ __forceinline__ uint64_t minf_lanemask_lt() {
    return (1ull << minf_lane()) - 1ull;
}

// Value of `x` in lane `src` (src must be wave-uniform).
__device__ __forceinline__ int minf_readlane(int x, int src) {
    return __builtin_amdgcn_readlane(x, __builtin_amdgcn_readfirstlane(src));
}
