// Shared helpers of the gfx950 kernels.  Wave64 only.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "difflogic_hip.h"

#define DL_WAVE 64
#define DL_BLOCK 256  // four waves per workgroup everywhere

typedef uint32_t dl_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t dl_u32x2 __attribute__((ext_vector_type(2)));

// hipGetLastError() reports the last error of ANY earlier runtime call of this thread, including
// harmless ones of the caller (an event query that answered "not ready"), so the error state is
// cleared right before each launch and read right after it.
#define DL_LAUNCH(kernel, grid, block, lds, stream, ...)                      \
    do {                                                                      \
        (void) hipGetLastError();                                             \
        hipLaunchKernelGGL(kernel, grid, block, lds, stream, __VA_ARGS__);    \
    } while (0)

extern thread_local int dl_last_hip_error_code;    // hipError_t of this thread's last refused launch (packed.hip)

static inline int dl_launch_status() {
    const hipError_t e = hipGetLastError();
    if (e == hipSuccess) return DL_OK;
    dl_last_hip_error_code = (int) e;
    return DL_ERR_LAUNCH;
}

static inline int64_t dl_ceil_div(int64_t x, int64_t y) { return (x + y - 1) / y; }

static inline bool dl_aligned(const void *p, size_t n) { return (reinterpret_cast<uintptr_t>(p) % n) == 0; }

// Wave index inside the workgroup as a value the compiler knows to be wave-uniform, so that
// table lookups indexed by it become scalar loads.
__device__ __forceinline__ int dl_wave_in_block() { return __builtin_amdgcn_readfirstlane((int) (threadIdx.x >> 6)); }

__device__ __forceinline__ int dl_lane() { return (int) (threadIdx.x & 63u); }

__device__ __forceinline__ int64_t dl_uniform(int64_t v) {
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t) (uint64_t) v);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t) ((uint64_t) v >> 32));
    return (int64_t) (((uint64_t) hi << 32) | lo);
}
