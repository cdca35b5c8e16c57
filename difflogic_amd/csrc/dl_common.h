// Shared helpers of the gfx950 kernels.  Wave64 only.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <tuple>
#include <utility>

#include "difflogic_hip.h"

#define DL_WAVE 64
#define DL_BLOCK 256  // four waves per workgroup everywhere

typedef uint32_t dl_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t dl_u32x2 __attribute__((ext_vector_type(2)));

// Launches go through hipLaunchKernel, whose return value is the launch's own verdict; the
// runtime's per-thread "last error" (which also holds harmless results of the caller's earlier
// calls, such as an event query that answered "not ready") is neither read nor cleared.
extern thread_local int dl_last_hip_error_code;    // hipError_t of this thread's last refused launch (packed.hip)
extern thread_local int dl_launch_result;          // hipError_t of this thread's last DL_LAUNCH (packed.hip)

template <typename... P, size_t... I, typename... A>
inline hipError_t dl_launch_impl(void (*kernel)(P...), dim3 grid, dim3 block, size_t lds, hipStream_t stream,
                                 std::index_sequence<I...>, A &&... args) {
    std::tuple<P...> params{static_cast<P>(args)...};             // the kernel's own parameter types
    void *ptrs[] = {static_cast<void *>(&std::get<I>(params))...};
    return hipLaunchKernel(reinterpret_cast<const void *>(kernel), grid, block, ptrs, lds, stream);
}

template <typename... P, typename... A>
inline void dl_launch(void (*kernel)(P...), dim3 grid, dim3 block, size_t lds, hipStream_t stream, A &&... args) {
    static_assert(sizeof...(P) == sizeof...(A), "argument count differs from the kernel's parameter count");
    const hipError_t e = dl_launch_impl(kernel, grid, block, lds, stream, std::index_sequence_for<P...>(), args...);
    if (dl_launch_result == (int) hipSuccess) dl_launch_result = (int) e;   // the first failure is the one reported
}

#define DL_LAUNCH(kernel, grid, block, lds, stream, ...) dl_launch(kernel, grid, block, lds, stream, __VA_ARGS__)

// Status of the launch(es) since the last call: DL_OK, or DL_ERR_LAUNCH with the HIP error kept
// for dl_last_hip_error().
static inline int dl_launch_status() {
    const int e = dl_launch_result;
    dl_launch_result = (int) hipSuccess;
    if (e == (int) hipSuccess) return DL_OK;
    dl_last_hip_error_code = e;
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
