// Measurement helpers, not part of the kernel library: plain streaming and gather kernels whose
// achieved rates are the practical ceilings the LogicLayer kernels are compared with
// (`python bench.py --ceilings`).  Built as libdl_ceilings.so; nothing in the package loads it.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

namespace {

constexpr int BLOCK = 256;
constexpr int UNROLL = 8;

// Each workgroup streams a grid-strided sequence of 16-byte vectors, UNROLL requests in flight.
__global__ __launch_bounds__(BLOCK) void stream_read_kernel(const u32x4 *__restrict__ p, int64_t n,
                                                            u32x4 *__restrict__ sink) {
    const int64_t stride = (int64_t) gridDim.x * BLOCK;
    int64_t i = (int64_t) blockIdx.x * BLOCK + threadIdx.x;
    u32x4 acc = {0, 0, 0, 0};
    for (; i + (UNROLL - 1) * stride < n; i += UNROLL * stride) {
        u32x4 v[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) v[u] = __builtin_nontemporal_load(&p[i + u * stride]);
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) acc ^= v[u];
    }
    for (; i < n; i += stride) acc ^= p[i];
    if (acc.x == 0x12345678u && acc.y == 0x9abcdef0u) sink[0] = acc;      // keeps the loads alive
}

__global__ __launch_bounds__(BLOCK) void stream_write_kernel(u32x4 *__restrict__ p, int64_t n) {
    const int64_t stride = (int64_t) gridDim.x * BLOCK;
    int64_t i = (int64_t) blockIdx.x * BLOCK + threadIdx.x;
    const u32x4 v = {1u, 2u, 3u, (uint32_t) i};
    for (; i < n; i += stride) __builtin_nontemporal_store(v, &p[i]);
}

__global__ __launch_bounds__(BLOCK) void stream_copy_kernel(const u32x4 *__restrict__ s, u32x4 *__restrict__ d,
                                                            int64_t n) {
    const int64_t stride = (int64_t) gridDim.x * BLOCK;
    int64_t i = (int64_t) blockIdx.x * BLOCK + threadIdx.x;
    for (; i + (UNROLL - 1) * stride < n; i += UNROLL * stride) {
        u32x4 v[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) v[u] = __builtin_nontemporal_load(&s[i + u * stride]);
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) __builtin_nontemporal_store(v[u], &d[i + u * stride]);
    }
    for (; i < n; i += stride) d[i] = s[i];
}

// The access pattern of the gate kernels without their arithmetic: blockIdx.x walks tiles of
// output rows (fastest), blockIdx.y 1 KB column tiles; a wave gathers G rows of x [rows, ncols]
// (ids from `idx`, wave-uniform) at its column tile per output row, 64 lanes x 16 bytes each, and
// folds them with xor.  Nothing is written, so the rate is that of the gathers alone: from the L2
// caches when rows x 1 KB stays resident there, else from the fabric behind them.
template <int G>
__global__ __launch_bounds__(BLOCK) void gather_rows_kernel(const u32x4 *__restrict__ x, const int32_t *__restrict__ idx,
                                                            int64_t out_rows, int64_t ncols, u32x4 *__restrict__ sink) {
    const int wave = __builtin_amdgcn_readfirstlane((int) (threadIdx.x >> 6));
    const int lane = (int) (threadIdx.x & 63u);
    const int64_t col = (int64_t) blockIdx.y * 64 + lane;
    if (col >= ncols) return;
    const int64_t n0 = ((int64_t) blockIdx.x * 4 + wave) * 8;
    u32x4 acc = {0, 0, 0, 0};
#pragma unroll 1
    for (int j = 0; j < 8; j += 2) {
        if (n0 + j + 1 >= out_rows) break;
        u32x4 v[2 * G];
#pragma unroll
        for (int g = 0; g < 2 * G; ++g) v[g] = x[(int64_t) idx[(n0 + j) * G + g] * ncols + col];
#pragma unroll
        for (int g = 0; g < 2 * G; ++g) acc ^= v[g];
    }
    if (acc.x == 0x12345678u && acc.y == 0x9abcdef0u) sink[0] = acc;
}

}  // namespace

extern "C" int dlc_stream(int mode, const void *src, void *dst, int64_t bytes, int grid, void *stream) {
    const int64_t n = bytes / 16;
    hipStream_t s = (hipStream_t) stream;
    if (mode == 0)
        hipLaunchKernelGGL(stream_read_kernel, dim3(grid), dim3(BLOCK), 0, s, (const u32x4 *) src, n, (u32x4 *) dst);
    else if (mode == 1)
        hipLaunchKernelGGL(stream_write_kernel, dim3(grid), dim3(BLOCK), 0, s, (u32x4 *) dst, n);
    else
        hipLaunchKernelGGL(stream_copy_kernel, dim3(grid), dim3(BLOCK), 0, s, (const u32x4 *) src, (u32x4 *) dst, n);
    return (int) hipGetLastError();
}

// x [rows, row_bytes], idx int32 [out_rows * gathers] with values in [0, rows); gathers in {2, 4, 8}.
extern "C" int dlc_gather(const void *x, const int32_t *idx, int64_t out_rows, int64_t row_bytes, int gathers,
                          void *sink, void *stream) {
    const int64_t ncols = row_bytes / 16;
    const dim3 grid((unsigned) ((out_rows + 31) / 32), (unsigned) ((ncols + 63) / 64));
    hipStream_t s = (hipStream_t) stream;
    if (grid.y > 65535) return -1;
    switch (gathers) {
    case 2: hipLaunchKernelGGL(gather_rows_kernel<2>, grid, dim3(BLOCK), 0, s, (const u32x4 *) x, idx, out_rows, ncols, (u32x4 *) sink); break;
    case 4: hipLaunchKernelGGL(gather_rows_kernel<4>, grid, dim3(BLOCK), 0, s, (const u32x4 *) x, idx, out_rows, ncols, (u32x4 *) sink); break;
    case 8: hipLaunchKernelGGL(gather_rows_kernel<8>, grid, dim3(BLOCK), 0, s, (const u32x4 *) x, idx, out_rows, ncols, (u32x4 *) sink); break;
    default: return -1;
    }
    return (int) hipGetLastError();
}
