// Training-mode kernels for gfx950: relaxed forward, backward_w, backward_x.
//
// Layout: activations are feature-major [features, batch]; lanes run along the batch so that
// every gathered row segment is one coalesced access (16 bytes per lane where the batch length
// and the base addresses allow it).  Everything indexed by the neuron (connection indices, the
// 16 gate weights) is wave-uniform and read through the scalar cache.
//
// The mixture of the 16 relaxed gates is bilinear in (a, b).  With
//     P_st = sum_i w_i * [gate i is true at (s, t)]            (four sums of eight weights)
// it is  y = (1-a)(1-b) P00 + (1-a) b P01 + a (1-b) P10 + a b P11, evaluated as two
// interpolations along b followed by one along a.
#include <hip/hip_fp16.h>

#include "dl_common.h"

namespace {

template <typename T> struct Acc { typedef float type; };
template <> struct Acc<double> { typedef double type; };

template <typename T, int N> struct alignas(sizeof(T) * N) Pack { T v[N]; };

template <typename T> __device__ __forceinline__ typename Acc<T>::type up(T v) { return (typename Acc<T>::type) v; }
template <> __device__ __forceinline__ float up<__half>(__half v) { return __half2float(v); }
template <typename T, typename C> __device__ __forceinline__ T down(C v) { return (T) v; }
template <> __device__ __forceinline__ __half down<__half, float>(float v) { return __float2half(v); }

__device__ __forceinline__ float dl_fma(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ __forceinline__ double dl_fma(double a, double b, double c) { return __builtin_fma(a, b, c); }

// Gate weights (probabilities or logits) and their gradients sit next to activations of type T either in T as well
// or, `w32`, in fp32 whatever T is: what a layer with fp32 weights needs for half / double activations (the
// reference's --training-bit-count 16 / 64).  The pointers keep the type T* and are reinterpreted.
template <typename T> __device__ __forceinline__ typename Acc<T>::type wload(const T *__restrict__ w, int64_t at, bool w32) {
    typedef typename Acc<T>::type C;
    if constexpr (sizeof(T) == sizeof(float)) return w[at];
    else return w32 ? (C) reinterpret_cast<const float *>(w)[at] : up<T>(w[at]);
}
template <typename T> __device__ __forceinline__ void wstore(T *__restrict__ w, int64_t at, typename Acc<T>::type v, bool w32) {
    typedef typename Acc<T>::type C;
    if constexpr (sizeof(T) == sizeof(float)) w[at] = v;
    else if (w32) reinterpret_cast<float *>(w)[at] = (float) v;
    else w[at] = down<T, C>(v);
}

// y = lerp(lerp(P00, P01, b), lerp(P10, P11, b), a), three fused multiply-adds.
template <typename C> __device__ __forceinline__ C mix(C av, C bv, C p00, C p10, C d0, C d1) {
    const C lo = dl_fma(bv, d0, p00);
    const C hi = dl_fma(bv, d1, p10);
    return dl_fma(av, hi - lo, lo);
}

// The four corner values of neuron n's gate mixture.
template <typename C> struct Corners { C p00, p01, p10, p11; };

template <typename C> __device__ __forceinline__ Corners<C> corners_of(const C (&g)[16]) {
    Corners<C> c;
    c.p00 = ((g[8] + g[9]) + (g[10] + g[11])) + ((g[12] + g[13]) + (g[14] + g[15]));
    c.p01 = ((g[4] + g[5]) + (g[6] + g[7])) + ((g[12] + g[13]) + (g[14] + g[15]));
    c.p10 = ((g[2] + g[3]) + (g[6] + g[7])) + ((g[10] + g[11]) + (g[14] + g[15]));
    c.p11 = ((g[1] + g[3]) + (g[5] + g[7])) + ((g[9] + g[11]) + (g[13] + g[15]));
    return c;
}

template <typename T>
__device__ __forceinline__ Corners<typename Acc<T>::type> corners(const T *__restrict__ w, int64_t n, bool w32) {
    typedef typename Acc<T>::type C;
    C g[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) g[i] = wload<T>(w, n * 16 + i, w32);
    return corners_of<C>(g);
}

// ------------------------------------------------------------------------------------------
// Wave-wide sums with a fixed association order (deterministic).
// ------------------------------------------------------------------------------------------
template <int CTRL> __device__ __forceinline__ float dpp_f32(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}

__device__ __forceinline__ float lane_value(float v, int i) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), i));
}

__device__ __forceinline__ double lane_value(double v, int i) {
    const uint64_t u = __builtin_bit_cast(uint64_t, v);
    const uint32_t lo = (uint32_t) __builtin_amdgcn_readlane((int) (uint32_t) u, i);
    const uint32_t hi = (uint32_t) __builtin_amdgcn_readlane((int) (uint32_t) (u >> 32), i);
    return __builtin_bit_cast(double, ((uint64_t) hi << 32) | lo);
}

// Wave-wide sums of FOUR values at once, each replaced by its total (wave-uniform).  A butterfly
// that halves the number of live values at each of its first two steps: after exchanging with
// lane ^ 1 a lane keeps the first or the second value of each pair, after lane ^ 2 it keeps one
// value, index lane & 3, summed over its quad; the quads of a 16-lane row are then added with
// row rotations (which keep lane & 3), rows 0+1 and 2+3 with v_permlane16_swap and the two
// halves with v_permlane32_swap (gfx950).  19 vector instructions instead of 44 for four
// separate reductions; the order of the additions is fixed.
__device__ __forceinline__ float swap_add16(float v) {
    const unsigned u = __builtin_bit_cast(unsigned, v);
    const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);     // rows (0,0,2,2) and (1,1,3,3)
    return __builtin_bit_cast(float, (unsigned) r[0]) + __builtin_bit_cast(float, (unsigned) r[1]);
}

__device__ __forceinline__ float swap_add32(float v) {
    const unsigned u = __builtin_bit_cast(unsigned, v);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);     // lower half twice, upper half twice
    return __builtin_bit_cast(float, (unsigned) r[0]) + __builtin_bit_cast(float, (unsigned) r[1]);
}

__device__ __forceinline__ void wave_sum4(float &s0, float &s1, float &s2, float &s3, int lane) {
    const bool odd = lane & 1, high = lane & 2;
    const float x = (odd ? s1 : s0) + dpp_f32<0xB1>(odd ? s0 : s1);          // quad_perm [1,0,3,2]: lane ^ 1
    const float y = (odd ? s3 : s2) + dpp_f32<0xB1>(odd ? s2 : s3);
    float z = (high ? y : x) + dpp_f32<0x4E>(high ? x : y);                  // quad_perm [2,3,0,1]: lane ^ 2
    z += dpp_f32<0x124>(z);                                                  // row_ror:4
    z += dpp_f32<0x128>(z);                                                  // row_ror:8
    z = swap_add32(swap_add16(z));
    s0 = lane_value(z, 0);
    s1 = lane_value(z, 1);
    s2 = lane_value(z, 2);
    s3 = lane_value(z, 3);
}

__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
    for (int m = 1; m < DL_WAVE; m <<= 1) v += __shfl_xor(v, m, DL_WAVE);
    return v;
}

__device__ __forceinline__ void wave_sum4(double &s0, double &s1, double &s2, double &s3, int) {
    s0 = wave_sum(s0);
    s1 = wave_sum(s1);
    s2 = wave_sum(s2);
    s3 = wave_sum(s3);
}

// Sum over each aligned group of 16 lanes, result in every lane of the group.
__device__ __forceinline__ float row16_sum(float v) {
    v += dpp_f32<0xB1>(v);
    v += dpp_f32<0x4E>(v);
    v += dpp_f32<0x141>(v);
    v += dpp_f32<0x140>(v);
    return v;
}

__device__ __forceinline__ double row16_sum(double v) {
#pragma unroll
    for (int m = 1; m < 16; m <<= 1) v += __shfl_xor(v, m, DL_WAVE);
    return v;
}

__device__ __forceinline__ float dl_exp(float v) { return expf(v); }
__device__ __forceinline__ double dl_exp(double v) { return exp(v); }

__device__ __forceinline__ float row16_max(float v) {
    v = fmaxf(v, dpp_f32<0xB1>(v));
    v = fmaxf(v, dpp_f32<0x4E>(v));
    v = fmaxf(v, dpp_f32<0x141>(v));
    v = fmaxf(v, dpp_f32<0x140>(v));
    return v;
}

__device__ __forceinline__ double row16_max(double v) {
#pragma unroll
    for (int m = 1; m < 16; m <<= 1) v = fmax(v, __shfl_xor(v, m, DL_WAVE));
    return v;
}

// Row of the gradient matrix that belongs to neuron n.  gdiv == 0: grad_y is [out_dim, batch] and
// the row is n.  gdiv > 0: the layer feeds a GroupSum and grad_y is its [k, batch] gradient (already
// divided by tau): all gdiv = out_dim / k neurons of a class share one row, and the broadcast
// [out_dim, batch] matrix is never materialised.
__device__ __forceinline__ int64_t grad_row(int64_t n, int64_t gdiv) {
    return gdiv ? (int64_t) ((uint32_t) n / (uint32_t) gdiv) : n;
}

// Corner coefficients of FOUR neurons at once: the 16-lane row r of the wave works on neuron n[r]
// (n[r] < 0: none), lane i of the row on gate i.  LOGITS: `w` holds logits, the row computes their
// softmax (and stores it to `probs` if asked); otherwise `w` holds the probabilities.  The corner
// sums are masked row sums whose association order is that of corners_of(), so the results are
// bit-identical to it.  Returns, per neuron, the wave-uniform P00, P10, P01 - P00, P11 - P10.
template <typename T, bool LOGITS>
__device__ __forceinline__ void corners4(const T *__restrict__ w, const int32_t (&n)[4], int lane, bool store_probs,
                                         T *__restrict__ probs, typename Acc<T>::type (&p00)[4],
                                         typename Acc<T>::type (&p10)[4], typename Acc<T>::type (&d0)[4],
                                         typename Acc<T>::type (&d1)[4], bool w32 = false) {
    typedef typename Acc<T>::type C;
    const int row = lane >> 4, gate = lane & 15;
    const int32_t mine = row == 0 ? n[0] : row == 1 ? n[1] : row == 2 ? n[2] : n[3];
    const bool valid = mine >= 0;
    const int64_t at = (int64_t) (valid ? mine : 0) * 16 + gate;
    C p = wload<T>(w, at, w32);
    if (LOGITS) {
        const C e = dl_exp(p - row16_max(p));
        p = e / row16_sum(e);
        if (store_probs && valid) wstore<T>(probs, at, p, w32);
    }
    const C zero = (C) 0;
    const C q00 = row16_sum((gate & 8) ? p : zero), q01 = row16_sum((gate & 4) ? p : zero);
    const C q10 = row16_sum((gate & 2) ? p : zero), q11 = row16_sum((gate & 1) ? p : zero);
    const C e0 = q01 - q00, e1 = q11 - q10;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        p00[i] = lane_value(q00, 16 * i);
        p10[i] = lane_value(q10, 16 * i);
        d0[i] = lane_value(e0, 16 * i);
        d1[i] = lane_value(e1, 16 * i);
    }
}

// ------------------------------------------------------------------------------------------
// forward: one wave = NPW neurons x 64 vectors of the batch.
// ------------------------------------------------------------------------------------------
// LOGITS: `w` holds the raw gate logits; the kernel applies the softmax itself and (column tile 0
// only) stores the probabilities to `probs` for the backward pass.
template <typename T, int VEC, int NPW, bool LOGITS>
__global__ __launch_bounds__(DL_BLOCK) void forward_kernel(const T *__restrict__ x, const int64_t *__restrict__ a,
                                                           const int64_t *__restrict__ b, const T *__restrict__ w,
                                                           T *__restrict__ y, T *__restrict__ probs, int64_t out_dim,
                                                           int64_t ncols, bool w32) {
    typedef typename Acc<T>::type C;
    typedef Pack<T, VEC> P;
    const int wave = dl_wave_in_block();
    const int lane = dl_lane();
    const int64_t n0 = ((int64_t) blockIdx.x * 4 + wave) * NPW;
    if (n0 >= out_dim) return;

    static_assert(NPW == 4, "corners4 serves four neurons per wave");
    int64_t ia[NPW], ib[NPW];
    C p00[NPW], p10[NPW], d0[NPW], d1[NPW];
    int32_t ids[NPW];
#pragma unroll
    for (int j = 0; j < NPW; ++j) {
        const int64_t n = (n0 + j < out_dim) ? n0 + j : out_dim - 1;
        ia[j] = a[n];
        ib[j] = b[n];
        ids[j] = n0 + j < out_dim ? (int32_t) (n0 + j) : -1;
    }
    corners4<T, LOGITS>(w, ids, lane, blockIdx.y == 0, probs, p00, p10, d0, d1, w32);
    const P *xv = reinterpret_cast<const P *>(x);
    P *yv = reinterpret_cast<P *>(y);
    for (int64_t col = (int64_t) blockIdx.y * DL_WAVE + lane; col < ncols; col += (int64_t) gridDim.y * DL_WAVE) {
        P va[NPW], vb[NPW];
#pragma unroll
        for (int j = 0; j < NPW; ++j) {
            va[j] = xv[ia[j] * ncols + col];
            vb[j] = xv[ib[j] * ncols + col];
        }
#pragma unroll
        for (int j = 0; j < NPW; ++j) {
            if (n0 + j < out_dim) {
                P r;
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    r.v[e] = down<T, C>(mix<C>(up<T>(va[j].v[e]), up<T>(vb[j].v[e]), p00[j], p10[j], d0[j], d1[j]));
                }
                yv[(n0 + j) * ncols + col] = r;
            }
        }
    }
}

// Lane i < 16 holds gate i: its gradient is the sum of the corner sums at which gate i is true.
// probs != nullptr chains the softmax backward, p_i * (g_i - sum_j p_j g_j).  Called by whole
// waves (the 16-lane row sum needs every lane).
template <typename T>
__device__ __forceinline__ void store_grad_w(int lane, bool neuron_valid, int64_t n, typename Acc<T>::type s00,
                                             typename Acc<T>::type s01, typename Acc<T>::type s10,
                                             typename Acc<T>::type s11, const T *__restrict__ probs,
                                             T *__restrict__ gw, bool w32 = false) {
    typedef typename Acc<T>::type C;
    const bool valid = lane < 16 && neuron_valid;
    C r = (C) 0;
    if (lane & 8) r += s00;
    if (lane & 4) r += s01;
    if (lane & 2) r += s10;
    if (lane & 1) r += s11;
    if (probs != nullptr) {
        const C p = valid ? wload<T>(probs, n * 16 + lane, w32) : (C) 0;
        const C dot = row16_sum(p * r);
        r = p * (r - dot);
    }
    if (valid) wstore<T>(gw, n * 16 + lane, r, w32);
}

// ------------------------------------------------------------------------------------------
// backward_w: per neuron, the four corner-weighted batch sums
//     S_st = sum_r g[r] * a^s (1-a)^(1-s) * b^t (1-b)^(1-t)
// and grad_w[n, i] = sum of the S_st at which gate i is true.
// WPN = waves that share one neuron's batch (1: a wave owns NPW neurons; 4: the workgroup's
// four waves split the batch of NPW neurons and combine through LDS in wave order).
// ------------------------------------------------------------------------------------------
// probs != nullptr: chain the softmax backward, gw[n,i] = p_i * (g_i - sum_j p_j g_j), i.e. the
// gradient with respect to the logits that `probs` (forward_kernel's LOGITS output) came from.
template <typename T, int VEC, int NPW, int WPN>
__global__ __launch_bounds__(DL_BLOCK) void backward_w_kernel(const T *__restrict__ x, const int64_t *__restrict__ a,
                                                              const int64_t *__restrict__ b,
                                                              const T *__restrict__ gy, const T *__restrict__ probs,
                                                              T *__restrict__ gw, int64_t out_dim, int64_t ncols,
                                                              int64_t gdiv, bool w32) {
    typedef typename Acc<T>::type C;
    typedef Pack<T, VEC> P;
    __shared__ C partial[4][NPW][4];
    const int wave = dl_wave_in_block();
    const int lane = dl_lane();
    const int64_t n0 = (WPN == 1) ? ((int64_t) blockIdx.x * 4 + wave) * NPW : (int64_t) blockIdx.x * NPW;
    const int part = (WPN == 1) ? 0 : wave;

    C s00[NPW], s01[NPW], s10[NPW], s11[NPW];
#pragma unroll
    for (int j = 0; j < NPW; ++j) s00[j] = s01[j] = s10[j] = s11[j] = (C) 0;

    if (n0 < out_dim) {
        int64_t ia[NPW], ib[NPW], nn[NPW];
#pragma unroll
        for (int j = 0; j < NPW; ++j) {
            const int64_t n = (n0 + j < out_dim) ? n0 + j : out_dim - 1;
            ia[j] = a[n];
            ib[j] = b[n];
            nn[j] = grad_row(n, gdiv);
        }
        const P *xv = reinterpret_cast<const P *>(x);
        const P *gv = reinterpret_cast<const P *>(gy);
        for (int64_t base = (int64_t) part * DL_WAVE; base < ncols; base += (int64_t) WPN * DL_WAVE) {
            const int64_t col = base + lane;
            if (col < ncols) {
                P va[NPW], vb[NPW], vg[NPW];
#pragma unroll
                for (int j = 0; j < NPW; ++j) {
                    va[j] = xv[ia[j] * ncols + col];
                    vb[j] = xv[ib[j] * ncols + col];
                    vg[j] = gv[nn[j] * ncols + col];
                }
#pragma unroll
                for (int j = 0; j < NPW; ++j) {
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        const C av = up<T>(va[j].v[e]), bv = up<T>(vb[j].v[e]), g = up<T>(vg[j].v[e]);
                        const C ga = g * av, gna = g - ga;       // g*a, g*(1-a)
                        const C t11 = ga * bv, t01 = gna * bv;
                        s11[j] += t11;
                        s10[j] += ga - t11;
                        s01[j] += t01;
                        s00[j] += gna - t01;
                    }
                }
            }
        }
    }

#pragma unroll
    for (int j = 0; j < NPW; ++j) {
        wave_sum4(s00[j], s01[j], s10[j], s11[j], lane);
    }

    if (WPN != 1) {
        if (lane == 0) {
#pragma unroll
            for (int j = 0; j < NPW; ++j) {
                partial[wave][j][0] = s00[j];
                partial[wave][j][1] = s01[j];
                partial[wave][j][2] = s10[j];
                partial[wave][j][3] = s11[j];
            }
        }
        __syncthreads();
        if (wave != 0) return;
#pragma unroll
        for (int j = 0; j < NPW; ++j) {
            s00[j] = (partial[0][j][0] + partial[1][j][0]) + (partial[2][j][0] + partial[3][j][0]);
            s01[j] = (partial[0][j][1] + partial[1][j][1]) + (partial[2][j][1] + partial[3][j][1]);
            s10[j] = (partial[0][j][2] + partial[1][j][2]) + (partial[2][j][2] + partial[3][j][2]);
            s11[j] = (partial[0][j][3] + partial[1][j][3]) + (partial[2][j][3] + partial[3][j][3]);
        }
    }

#pragma unroll
    for (int j = 0; j < NPW; ++j)
        store_grad_w<T>(lane, n0 + j < out_dim, n0 + j, s00[j], s01[j], s10[j], s11[j], probs, gw, w32);
}

// ------------------------------------------------------------------------------------------
// backward_x: one wave = one input row x 64 vectors of the batch; it walks the row's fan-out
// list (reverse index) and gathers, so every grad_x element has a single writer.
//     dy/da = (P10 - P00) + b * ((P11 - P10) - (P01 - P00))
//     dy/db = (P01 - P00) + a * ((P11 - P10) - (P01 - P00))
// A neuron wired twice to this input appears twice in the list; each visit adds half of
// dy/da + dy/db.
// ------------------------------------------------------------------------------------------
template <typename T, int VEC>
__global__ __launch_bounds__(DL_BLOCK) void backward_x_kernel(const T *__restrict__ x, const int64_t *__restrict__ a,
                                                              const int64_t *__restrict__ b, const T *__restrict__ w,
                                                              const T *__restrict__ gy,
                                                              const int64_t *__restrict__ start,
                                                              const int64_t *__restrict__ idx, T *__restrict__ gx,
                                                              int64_t in_dim, int64_t ncols,
                                                              typename Acc<T>::type scale, int64_t gdiv, bool w32) {
    typedef typename Acc<T>::type C;
    typedef Pack<T, VEC> P;
    const int wave = dl_wave_in_block();
    const int lane = dl_lane();
    const int64_t c = (int64_t) blockIdx.x * 4 + wave;
    if (c >= in_dim) return;
    const int64_t e0 = start[c], e1 = start[c + 1];
    const P *xv = reinterpret_cast<const P *>(x);
    const P *gv = reinterpret_cast<const P *>(gy);
    P *ov = reinterpret_cast<P *>(gx);

    for (int64_t col = (int64_t) blockIdx.y * DL_WAVE + lane; col < ncols; col += (int64_t) gridDim.y * DL_WAVE) {
        C acc[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[e] = (C) 0;
        for (int64_t e = e0; e < e1; e += 2) {
            // two fan-out entries per trip so that their loads overlap
            const bool two = e + 1 < e1;
            const int64_t nA = idx[e], nB = two ? idx[e + 1] : nA;
            const int64_t iaA = a[nA], ibA = b[nA], iaB = a[nB], ibB = b[nB];
            const bool isaA = iaA == c, isaB = iaB == c;
            const P gA = gv[grad_row(nA, gdiv) * ncols + col], oA = xv[(isaA ? ibA : iaA) * ncols + col];
            const P gB = gv[grad_row(nB, gdiv) * ncols + col], oB = xv[(isaB ? ibB : iaB) * ncols + col];
            const Corners<C> kA = corners<T>(w, nA, w32), kB = corners<T>(w, nB, w32);
            {
                const C d0 = kA.p01 - kA.p00, d1 = kA.p11 - kA.p10, dd = d1 - d0, da = kA.p10 - kA.p00;
                const C k0 = (isaA && ibA == c) ? (C) 0.5 * (da + d0) : (isaA ? da : d0);
#pragma unroll
                for (int q = 0; q < VEC; ++q) acc[q] += up<T>(gA.v[q]) * (k0 + up<T>(oA.v[q]) * dd);
            }
            if (two) {
                const C d0 = kB.p01 - kB.p00, d1 = kB.p11 - kB.p10, dd = d1 - d0, da = kB.p10 - kB.p00;
                const C k0 = (isaB && ibB == c) ? (C) 0.5 * (da + d0) : (isaB ? da : d0);
#pragma unroll
                for (int q = 0; q < VEC; ++q) acc[q] += up<T>(gB.v[q]) * (k0 + up<T>(oB.v[q]) * dd);
            }
        }
        P r;
#pragma unroll
        for (int q = 0; q < VEC; ++q) r.v[q] = down<T, C>(acc[q] * scale);
        ov[c * ncols + col] = r;
    }
}

// ------------------------------------------------------------------------------------------
// Chained forward / backward_w.  The layer's neurons are walked along the trails of an
// evaluation schedule (schedule.cpp): step s brings in input row verts[s + 1] and evaluates
// neuron[s] from (verts[s], verts[s + 1]); flip[s] tells which of the two is the neuron's `a`
// input.  The shared row stays in registers, so a neuron costs one gathered row instead of two.
// Arithmetic and summation order per element are those of the unchained kernels: the fp32 and
// fp64 results are bit-identical (fp16 outputs can differ in the last bit, where the compiler
// folds the final conversion into a fused multiply-add in one kernel and not in the other).
// ------------------------------------------------------------------------------------------
template <typename T, int VEC, int CHUNK, bool LOGITS>
__global__ __launch_bounds__(DL_BLOCK) void forward_chain_kernel(const T *__restrict__ x,
                                                                 const int32_t *__restrict__ verts,
                                                                 const int32_t *__restrict__ neuron,
                                                                 const uint8_t *__restrict__ flip,
                                                                 const T *__restrict__ w, T *__restrict__ y,
                                                                 T *__restrict__ probs, int64_t nchunks, int64_t ncols,
                                                                 bool w32) {
    typedef typename Acc<T>::type C;
    typedef Pack<T, VEC> P;
    const int wave = dl_wave_in_block();
    const int lane = dl_lane();
    const int64_t c = (int64_t) blockIdx.x * 4 + wave;
    if (c >= nchunks) return;
    static_assert(CHUNK % 4 == 0, "neurons are served four at a time");
    const int64_t s0 = c * CHUNK;
    const P *xv = reinterpret_cast<const P *>(x);
    P *yv = reinterpret_cast<P *>(y);

    for (int64_t ct = blockIdx.y; ct * DL_WAVE < ncols; ct += gridDim.y) {
        const int64_t col = ct * DL_WAVE + lane;
        const bool live = col < ncols;
        const int64_t cl = live ? col : 0;
        // every row of the chunk is requested before the first one is used
        P rows[CHUNK + 1];
#pragma unroll
        for (int j = 0; j <= CHUNK; ++j) rows[j] = xv[(int64_t) verts[s0 + j] * ncols + cl];
#pragma unroll
        for (int j0 = 0; j0 < CHUNK; j0 += 4) {
            int32_t n[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) n[i] = neuron[s0 + j0 + i];
            C p00[4], p10[4], d0[4], d1[4];
            corners4<T, LOGITS>(w, n, lane, ct == 0, probs, p00, p10, d0, d1, w32);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int j = j0 + i;
                const bool f = flip[s0 + j] != 0;
                P r;
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    const C u0 = up<T>(rows[j].v[e]), u1 = up<T>(rows[j + 1].v[e]);
                    r.v[e] = down<T, C>(mix<C>(f ? u1 : u0, f ? u0 : u1, p00[i], p10[i], d0[i], d1[i]));
                }
                if (live && n[i] >= 0) yv[(int64_t) n[i] * ncols + col] = r;
            }
        }
    }
}

// forward_chain_kernel for a layer whose input is the output of the layer below, with that output
// recomputed instead of read: input row v = forward of neuron v of the lower layer, from lower input
// rows low_a[v], low_b[v] of `lx` (a small matrix that stays in the L2 caches) and its gate weights
// (LOGITS: logits, whose softmax goes to `lprobs`).  Values and rounding are those of forward_kernel
// on the lower layer, so the result equals running the two layers one after the other bit for bit,
// but the activation between them is neither written nor read.
template <typename T, int VEC, int CHUNK, bool LOGITS>
__global__ __launch_bounds__(DL_BLOCK) void forward_chain_lower_kernel(
    const T *__restrict__ lx, const int64_t *__restrict__ low_a, const int64_t *__restrict__ low_b,
    const T *__restrict__ lw, T *__restrict__ lprobs, const int32_t *__restrict__ verts,
    const int32_t *__restrict__ neuron, const uint8_t *__restrict__ flip, const T *__restrict__ w, T *__restrict__ y,
    T *__restrict__ probs, int64_t nchunks, int64_t ncols) {
    typedef typename Acc<T>::type C;
    typedef Pack<T, VEC> P;
    const int wave = dl_wave_in_block();
    const int lane = dl_lane();
    const int64_t c = (int64_t) blockIdx.x * 4 + wave;
    if (c >= nchunks) return;
    static_assert(CHUNK % 4 == 0, "neurons are served four at a time");
    const int64_t s0 = c * CHUNK;
    const P *xv = reinterpret_cast<const P *>(lx);
    P *yv = reinterpret_cast<P *>(y);

    // corner coefficients of the chunk's CHUNK + 1 lower neurons and CHUNK neurons, once for all column tiles
    constexpr int NV = CHUNK + 4;
    int32_t v[NV], n[CHUNK];
    C lp00[NV], lp10[NV], ld0[NV], ld1[NV], p00[CHUNK], p10[CHUNK], d0[CHUNK], d1[CHUNK];
#pragma unroll
    for (int j0 = 0; j0 <= CHUNK; j0 += 4) {
        int32_t v4[4];
        C q00[4], q10[4], e0[4], e1[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) v4[i] = j0 + i <= CHUNK ? verts[s0 + j0 + i] : -1;
        corners4<T, LOGITS>(lw, v4, lane, blockIdx.y == 0, lprobs, q00, q10, e0, e1);
#pragma unroll
        for (int i = 0; i < 4; ++i) v[j0 + i] = v4[i], lp00[j0 + i] = q00[i], lp10[j0 + i] = q10[i], ld0[j0 + i] = e0[i], ld1[j0 + i] = e1[i];
    }
#pragma unroll
    for (int j0 = 0; j0 < CHUNK; j0 += 4) {
        int32_t n4[4];
        C q00[4], q10[4], e0[4], e1[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) n4[i] = neuron[s0 + j0 + i];
        corners4<T, LOGITS>(w, n4, lane, blockIdx.y == 0, probs, q00, q10, e0, e1);
#pragma unroll
        for (int i = 0; i < 4; ++i) n[j0 + i] = n4[i], p00[j0 + i] = q00[i], p10[j0 + i] = q10[i], d0[j0 + i] = e0[i], d1[j0 + i] = e1[i];
    }
    int64_t ia[CHUNK + 1], ib[CHUNK + 1];
#pragma unroll
    for (int j = 0; j <= CHUNK; ++j) ia[j] = low_a[v[j]], ib[j] = low_b[v[j]];

    for (int64_t ct = blockIdx.y; ct * DL_WAVE < ncols; ct += gridDim.y) {
        const int64_t col = ct * DL_WAVE + lane;
        const bool live = col < ncols;
        const int64_t cl = live ? col : 0;
        // the chunk's CHUNK + 1 input rows, recomputed four at a time
        P rows[CHUNK + 1];
#pragma unroll
        for (int j0 = 0; j0 <= CHUNK; j0 += 4) {
            P va[4], vb[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (j0 + i <= CHUNK) {
                    va[i] = xv[ia[j0 + i] * ncols + cl];
                    vb[i] = xv[ib[j0 + i] * ncols + cl];
                }
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int j = j0 + i;
                if (j <= CHUNK) {
#pragma unroll
                    for (int e = 0; e < VEC; ++e)
                        rows[j].v[e] = down<T, C>(mix<C>(up<T>(va[i].v[e]), up<T>(vb[i].v[e]), lp00[j], lp10[j], ld0[j], ld1[j]));
                }
            }
        }
#pragma unroll
        for (int j = 0; j < CHUNK; ++j) {
            const bool f = flip[s0 + j] != 0;
            P r;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const C u0 = up<T>(rows[j].v[e]), u1 = up<T>(rows[j + 1].v[e]);
                r.v[e] = down<T, C>(mix<C>(f ? u1 : u0, f ? u0 : u1, p00[j], p10[j], d0[j], d1[j]));
            }
            if (live && n[j] >= 0) yv[(int64_t) n[j] * ncols + col] = r;
        }
    }
}

// Forward along the schedule for long rows: one wave owns `chunk` steps and a segment of
// CPL * 64 consecutive vectors of the row (blockIdx.y picks the segment; lane l holds its vectors
// l, l + 64, ...), so every gathered row is one contiguous request of up to 4 KB, and the next
// step's row is requested before this step's arithmetic.
template <typename T, int VEC, int CPL, bool LOGITS>
__global__ __launch_bounds__(DL_BLOCK) void forward_chain_rows_kernel(const T *__restrict__ x,
                                                                      const int32_t *__restrict__ verts,
                                                                      const int32_t *__restrict__ neuron,
                                                                      const uint8_t *__restrict__ flip,
                                                                      const T *__restrict__ w, T *__restrict__ y,
                                                                      T *__restrict__ probs, int64_t steps, int chunk,
                                                                      int64_t ncols, bool w32) {
    typedef typename Acc<T>::type C;
    typedef Pack<T, VEC> P;
    const int wave = dl_wave_in_block();
    const int lane = dl_lane();
    const int64_t s0 = ((int64_t) blockIdx.x * 4 + wave) * chunk;
    if (s0 >= steps) return;
    const int64_t s1 = s0 + chunk < steps ? s0 + chunk : steps;
    const P *xv = reinterpret_cast<const P *>(x);
    P *yv = reinterpret_cast<P *>(y);
    const int64_t col0 = (int64_t) blockIdx.y * (CPL * DL_WAVE);
    P zero;
#pragma unroll
    for (int e = 0; e < VEC; ++e) zero.v[e] = down<T, C>((C) 0);
    auto load_row = [&](int64_t row, P *out) {
#pragma unroll
        for (int q = 0; q < CPL; ++q) {
            const int64_t col = col0 + lane + q * DL_WAVE;
            out[q] = col < ncols ? xv[row * ncols + col] : zero;
        }
    };
    P prev[CPL], cur[CPL], next[CPL];
    load_row(verts[s0], prev);
    load_row(verts[s0 + 1], cur);
#pragma unroll 1
    for (int64_t g = s0; g < s1; g += 4) {           // four steps per trip: their corners are computed together
        int32_t n[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) n[i] = g + i < s1 ? neuron[g + i] : -1;
        C p00[4], p10[4], d0[4], d1[4];
        corners4<T, LOGITS>(w, n, lane, col0 == 0, probs, p00, p10, d0, d1, w32);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int64_t s = g + i;
            if (s < s1) {                            // wave-uniform
                if (s + 1 < s1) load_row(verts[s + 2], next);
                const bool f = flip[s] != 0;
#pragma unroll
                for (int q = 0; q < CPL; ++q) {
                    const int64_t col = col0 + lane + q * DL_WAVE;
                    P r;
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        const C u0 = up<T>(prev[q].v[e]), u1 = up<T>(cur[q].v[e]);
                        r.v[e] = down<T, C>(mix<C>(f ? u1 : u0, f ? u0 : u1, p00[i], p10[i], d0[i], d1[i]));
                    }
                    if (n[i] >= 0 && col < ncols) yv[(int64_t) n[i] * ncols + col] = r;
                }
#pragma unroll
                for (int q = 0; q < CPL; ++q) {
                    prev[q] = cur[q];
                    cur[q] = next[q];
                }
            }
        }
    }
}

// One wave owns CHUNK steps and the whole batch: lane l holds vectors l, l + 64, ... (CPL of them).
template <typename T, int VEC, int CPL, int CHUNK>
__global__ __launch_bounds__(DL_BLOCK) void backward_w_chain_kernel(const T *__restrict__ x,
                                                                    const int32_t *__restrict__ verts,
                                                                    const int32_t *__restrict__ neuron,
                                                                    const uint8_t *__restrict__ flip,
                                                                    const T *__restrict__ gy,
                                                                    const T *__restrict__ probs, T *__restrict__ gw,
                                                                    int64_t nchunks, int64_t ncols, int64_t gdiv, bool w32) {
    typedef typename Acc<T>::type C;
    typedef Pack<T, VEC> P;
    const int wave = dl_wave_in_block();
    const int lane = dl_lane();
    const int64_t c = (int64_t) blockIdx.x * 4 + wave;
    if (c >= nchunks) return;
    const int64_t s0 = c * CHUNK;
    const P *xv = reinterpret_cast<const P *>(x);
    const P *gv = reinterpret_cast<const P *>(gy);
    P zero;
#pragma unroll
    for (int e = 0; e < VEC; ++e) zero.v[e] = down<T, C>((C) 0);

    auto load_row = [&](const P *base, int64_t row, P *dst) {
#pragma unroll
        for (int q = 0; q < CPL; ++q) {
            const int64_t col = lane + q * DL_WAVE;
            dst[q] = col < ncols ? base[row * ncols + col] : zero;
        }
    };
    P prev[CPL];
    load_row(xv, verts[s0], prev);
#pragma unroll 1
    for (int j = 0; j < CHUNK; ++j) {
        const int32_t n = neuron[s0 + j];
        const bool f = flip[s0 + j] != 0;
        P cur[CPL], g[CPL];
        load_row(xv, verts[s0 + j + 1], cur);
        load_row(gv, grad_row(n >= 0 ? n : 0, gdiv), g);
        C s00 = (C) 0, s01 = (C) 0, s10 = (C) 0, s11 = (C) 0;
#pragma unroll
        for (int q = 0; q < CPL; ++q) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const C u0 = up<T>(prev[q].v[e]), u1 = up<T>(cur[q].v[e]), gg = up<T>(g[q].v[e]);
                const C av = f ? u1 : u0, bv = f ? u0 : u1;
                const C ga = gg * av, gna = gg - ga;
                const C t11 = ga * bv, t01 = gna * bv;
                s11 += t11;
                s10 += ga - t11;
                s01 += t01;
                s00 += gna - t01;
            }
        }
        wave_sum4(s00, s01, s10, s11, lane);
        store_grad_w<T>(lane, n >= 0, n >= 0 ? n : 0, s00, s01, s10, s11, probs, gw, w32);
#pragma unroll
        for (int q = 0; q < CPL; ++q) prev[q] = cur[q];
    }
}

// ------------------------------------------------------------------------------------------
// Chained backward: grad_w AND grad_x of a layer in one pass along the schedule.  Step s reads
// input row verts[s + 1] and grad_y row neuron[s] (the other input row is still in registers),
// which is all that backward_w and both directions of backward_x need for that neuron:
//     to a:  g * ((P10 - P00) + b * dd)      to b:  g * ((P01 - P00) + a * dd)
//     dd = (P11 - P10) - (P01 - P00)
// A vertex in the middle of a trail collects the share of the neuron before it (kept in
// `carry`) and of the neuron after it and is written once: position p of the schedule goes to
// row dst[p] (-1: nothing to write; >= in_dim: row dst[p] - in_dim of `overflow`, for vertices
// that occur at several positions and are summed afterwards by backward_fix_kernel).  Rows longer
// than CPL * 64 vectors are cut into segments (blockIdx.y); the corner sums of the segments then
// go to `partial` and backward_w_finish_kernel adds them.  A wave
// owns `chunk` positions [s0, s0 + chunk); it recomputes the last neuron of the chunk before it to get
// the carry into its first position, so chunks do not exchange partial rows.
// ------------------------------------------------------------------------------------------
// LOWER >= 1: the layer BELOW this one (whose output x is) needs no grad_x of its own and gets its
// grad_w here: a vertex's finished grad_x row is the grad_y row of neuron `vertex` of the layer below,
// so its four corner sums are taken on the spot from the row in registers and the two input rows of
// that neuron (`low.x`, gathered through `low.a`, `low.b`), and the row is not stored at all.  Only the
// vertices that finish in backward_fix_kernel still go through memory (backward_w_rows_kernel).
// LOWER == 2: x itself is not read either: row v of x is recomputed as the lower layer's forward pass
// computed it (same arithmetic, same rounding) from the two lower input rows that the vertex's
// backward_w needs anyway, so the activation between the two layers never exists in memory.
template <typename T> struct LowerLayer {
    const T *x;                 // [in_dim of the layer below, batch]
    const int64_t *a, *b;       // its wiring, [in_dim]
    const T *w;                 // its gate probabilities [in_dim, 16]
    const T *probs;             // == w: chain the softmax backward into gw; null: gw is the plain grad_w
    T *gw;                      // [in_dim, 16]
};

template <typename T, int VEC, int CPL, int LOWER>
__global__ __launch_bounds__(DL_BLOCK) void backward_chain_kernel(
    const T *__restrict__ x, const int32_t *__restrict__ verts, const int32_t *__restrict__ neuron,
    const uint8_t *__restrict__ flip, const int32_t *__restrict__ dst, const T *__restrict__ w,
    const T *__restrict__ gy, const T *__restrict__ probs, T *__restrict__ gw,
    typename Acc<T>::type *__restrict__ partial, T *__restrict__ gx, T *__restrict__ overflow, int64_t steps, int chunk,
    int64_t in_dim, int64_t out_dim, int64_t ncols, typename Acc<T>::type scale, int64_t gdiv, LowerLayer<T> low,
    bool w32) {
    typedef typename Acc<T>::type C;
    typedef Pack<T, VEC> P;
    constexpr bool RECOMPUTE = LOWER == 2;
    constexpr int LCPL = LOWER ? CPL : 1;                       // registers for lower rows only where they are used
    const int wave = dl_wave_in_block();
    const int lane = dl_lane();
    const int64_t s0 = ((int64_t) blockIdx.x * 4 + wave) * chunk;
    if (s0 >= steps) return;
    const int64_t s1 = s0 + chunk < steps ? s0 + chunk : steps;
    const P *xv = reinterpret_cast<const P *>(x);
    const P *gv = reinterpret_cast<const P *>(gy);
    const P *lx = reinterpret_cast<const P *>(low.x);
    const int64_t col0 = (int64_t) blockIdx.y * (CPL * DL_WAVE);   // this wave's segment of the rows
    const int gate = lane & 15;
    P zero;
#pragma unroll
    for (int e = 0; e < VEC; ++e) zero.v[e] = down<T, C>((C) 0);

    auto load_row = [&](const P *base, int64_t row, bool valid, P *out) {
#pragma unroll
        for (int q = 0; q < CPL; ++q) {
            const int64_t col = col0 + lane + q * DL_WAVE;
            out[q] = (valid && col < ncols) ? base[row * ncols + col] : zero;
        }
    };
    // the two input rows of neuron v of the layer below (v wave-uniform)
    auto lower_rows = [&](int64_t v, bool valid, P *la, P *lb) {
        if constexpr (LOWER != 0) {
            const int64_t r = valid ? v : 0;
            load_row(lx, low.a[r], valid, la);
            load_row(lx, low.b[r], valid, lb);
        }
    };
    // row v of x as the lower layer's forward kernel stored it: lane `gate` of every 16-lane row holds the
    // neuron's probability of that gate; corner sums and their order as corners4()
    auto lower_forward = [&](const P *la, const P *lb, C lp, P *out) {
        const C zc = (C) 0;
        const C q00 = row16_sum((gate & 8) ? lp : zc), q01 = row16_sum((gate & 4) ? lp : zc);
        const C q10 = row16_sum((gate & 2) ? lp : zc), q11 = row16_sum((gate & 1) ? lp : zc);
        const C p00 = lane_value(q00, 0), p10 = lane_value(q10, 0);
        const C d0 = lane_value(q01 - q00, 0), d1 = lane_value(q11 - q10, 0);
#pragma unroll
        for (int q = 0; q < CPL; ++q)
#pragma unroll
            for (int e = 0; e < VEC; ++e)
                out[q].v[e] = down<T, C>(mix<C>(up<T>(la[q].v[e]), up<T>(lb[q].v[e]), p00, p10, d0, d1));
    };
    // la, lb: with LOWER, the two input rows of neuron `row` of the layer below
    auto store_row = [&](int32_t row, const C (&val)[CPL][VEC], const P *la, const P *lb) {
        if (row < 0) return;
        if (LOWER != 0 && row < in_dim) {
            // as backward_w_kernel on the row this would have stored: same values, same order of additions
            C s00 = (C) 0, s01 = (C) 0, s10 = (C) 0, s11 = (C) 0;
#pragma unroll
            for (int q = 0; q < CPL; ++q) {
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    const C g = up<T>(down<T, C>(val[q][e] * scale));
                    const C av = up<T>(la[q].v[e]), bv = up<T>(lb[q].v[e]);
                    const C ga = g * av, gna = g - ga;
                    const C t11 = ga * bv, t01 = gna * bv;
                    s11 += t11;
                    s10 += ga - t11;
                    s01 += t01;
                    s00 += gna - t01;
                }
            }
            wave_sum4(s00, s01, s10, s11, lane);
            store_grad_w<T>(lane, true, row, s00, s01, s10, s11, low.probs, low.gw);
            return;
        }
        P *base = row < in_dim ? reinterpret_cast<P *>(gx) + (int64_t) row * ncols
                               : reinterpret_cast<P *>(overflow) + ((int64_t) row - in_dim) * ncols;
#pragma unroll
        for (int q = 0; q < CPL; ++q) {
            const int64_t col = col0 + lane + q * DL_WAVE;
            P r;
#pragma unroll
            for (int e = 0; e < VEC; ++e) r.v[e] = down<T, C>(val[q][e] * scale);
            if (col < ncols) base[col] = r;
        }
    };

    // prev: row of the vertex at the chunk's first position; pla, plb: (RECOMPUTE) the lower rows it came from,
    // which also serve that vertex's backward_w at step 0
    P prev[CPL], pla[LCPL], plb[LCPL];
    C carry[CPL][VEC];
    if constexpr (RECOMPUTE) {
        const int64_t v0 = verts[s0];
        lower_rows(v0, true, pla, plb);
        lower_forward(pla, plb, up<T>(low.w[v0 * 16 + gate]), prev);
    } else {
        load_row(xv, verts[s0], true, prev);
    }
#pragma unroll
    for (int q = 0; q < CPL; ++q)
#pragma unroll
        for (int e = 0; e < VEC; ++e) carry[q][e] = (C) 0;
    if (s0 > 0 && neuron[s0 - 1] >= 0) {             // share of the neuron that ends at this chunk's first vertex
        const int32_t n = neuron[s0 - 1];
        const bool f = flip[s0 - 1] != 0;
        P before[CPL], g[CPL];
        if constexpr (RECOMPUTE) {
            const int64_t vb = verts[s0 - 1];
            P ba[LCPL], bb[LCPL];
            lower_rows(vb, true, ba, bb);
            lower_forward(ba, bb, up<T>(low.w[vb * 16 + gate]), before);
        } else {
            load_row(xv, verts[s0 - 1], true, before);
        }
        load_row(gv, grad_row(n, gdiv), true, g);
        const Corners<C> k = corners<T>(w, n, w32);
        const C d0 = k.p01 - k.p00, dd = (k.p11 - k.p10) - d0, da = k.p10 - k.p00;
        const C kv = f ? da : d0;
#pragma unroll
        for (int q = 0; q < CPL; ++q)
#pragma unroll
            for (int e = 0; e < VEC; ++e) carry[q][e] = up<T>(g[q].v[e]) * dl_fma(up<T>(before[q].v[e]), dd, kv);
    }
    // The chunk's schedule entries are fetched once, one per lane (chunk <= 64), and handed out by
    // readlane, so the step loop waits for no scalar loads; the rows of step i + 1 are requested
    // before the arithmetic of step i.
    const int cnt = (int) (s1 - s0);
    const bool has = lane < cnt;
    const int32_t sch_n = has ? neuron[s0 + lane] : -1;
    const int32_t sch_v = has ? verts[s0 + 1 + lane] : 0;
    const int32_t sch_d = has ? dst[s0 + lane] : -1;
    const int32_t sch_f = has ? (int32_t) flip[s0 + lane] : 0;
    // Rows of step i: the new input row (RECOMPUTE: the two lower rows and the lower probabilities it is
    // recomputed from), the neuron's grad_y row (zero for a step without a neuron) and, in every 16-lane
    // row, the neuron's 16 gate probabilities.  LOWER == 1: la, lb are the lower rows of the vertex that
    // step i finishes (dst[i]); RECOMPUTE: of the vertex that step i brings in.
    auto fetch = [&](int i, P *row, P *grad, C &prob, P *la, P *lb, C &lprob) {
        const int32_t n = __builtin_amdgcn_readlane(sch_n, i);
        const bool valid = n >= 0;
        const int64_t nn = valid ? n : 0;
        const int32_t v = __builtin_amdgcn_readlane(sch_v, i);
        if constexpr (RECOMPUTE) {
            lower_rows(v, true, la, lb);
            lprob = up<T>(low.w[(int64_t) v * 16 + gate]);
        } else {
            load_row(xv, v, true, row);
            if constexpr (LOWER == 1) {
                const int32_t d = __builtin_amdgcn_readlane(sch_d, i);
                lower_rows(d, d >= 0 && d < in_dim, la, lb);
            }
        }
        load_row(gv, grad_row(nn, gdiv), valid, grad);
        prob = wload<T>(w, nn * 16 + gate, w32);
    };
    P cur[CPL], g[CPL], la[LCPL], lb[LCPL];
    C pw, lpw = (C) 0;
    fetch(0, cur, g, pw, la, lb, lpw);
#pragma unroll 1
    for (int i = 0; i < cnt; ++i) {
        P ncur[CPL], ng[CPL], nla[LCPL], nlb[LCPL];
        C npw = (C) 0, nlpw = (C) 0;
        if (i + 1 < cnt) fetch(i + 1, ncur, ng, npw, nla, nlb, nlpw);
        if constexpr (RECOMPUTE) lower_forward(la, lb, lpw, cur);
        const int32_t n = __builtin_amdgcn_readlane(sch_n, i);
        const bool valid = n >= 0;
        const int64_t nn = valid ? n : 0;
        const bool f = __builtin_amdgcn_readlane(sch_f, i) != 0;
        // corner sums of the probabilities, in the association order of corners_of()
        const C zc = (C) 0;
        const C p00 = lane_value(row16_sum((gate & 8) ? pw : zc), 0), p01 = lane_value(row16_sum((gate & 4) ? pw : zc), 0);
        const C p10 = lane_value(row16_sum((gate & 2) ? pw : zc), 0), p11 = lane_value(row16_sum((gate & 1) ? pw : zc), 0);
        const C d0 = p01 - p00, dd = (p11 - p10) - d0, da = p10 - p00;
        const C ku = f ? d0 : da, kv = f ? da : d0;
        C s00 = (C) 0, s01 = (C) 0, s10 = (C) 0, s11 = (C) 0;
        C out[CPL][VEC];
#pragma unroll
        for (int q = 0; q < CPL; ++q) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const C u0 = up<T>(prev[q].v[e]), u1 = up<T>(cur[q].v[e]), gg = up<T>(g[q].v[e]);
                const C av = f ? u1 : u0, bv = f ? u0 : u1;
                const C ga = gg * av, gna = gg - ga;
                const C t11 = ga * bv, t01 = gna * bv;
                s11 += t11;
                s10 += ga - t11;
                s01 += t01;
                s00 += gna - t01;
                out[q][e] = carry[q][e] + gg * dl_fma(u1, dd, ku);
                carry[q][e] = gg * dl_fma(u0, dd, kv);
            }
        }
        wave_sum4(s00, s01, s10, s11, lane);
        if (partial == nullptr) {
            // as store_grad_w, with the probabilities already at hand
            C r = (C) 0;
            if (lane & 8) r += s00;
            if (lane & 4) r += s01;
            if (lane & 2) r += s10;
            if (lane & 1) r += s11;
            if (probs != nullptr) {
                const C pr = (valid && lane < 16) ? pw : zc;
                const C dot = row16_sum(pr * r);
                r = pr * (r - dot);
            }
            if (valid && lane < 16) wstore<T>(gw, nn * 16 + lane, r, w32);
        } else if (valid && lane < 4) {              // several segments: backward_w_finish_kernel adds them
            const C mine = lane == 0 ? s00 : lane == 1 ? s01 : lane == 2 ? s10 : s11;
            partial[((int64_t) blockIdx.y * out_dim + nn) * 4 + lane] = mine;
        }
        // the vertex at position s0 + i is finished: RECOMPUTE keeps its lower rows from the step that brought it in
        store_row(__builtin_amdgcn_readlane(sch_d, i), out, RECOMPUTE ? pla : la, RECOMPUTE ? plb : lb);
#pragma unroll
        for (int q = 0; q < CPL; ++q) {
            prev[q] = cur[q];
            cur[q] = ncur[q];
            g[q] = ng[q];
        }
        if constexpr (LOWER != 0) {
#pragma unroll
            for (int q = 0; q < LCPL; ++q) {
                if constexpr (RECOMPUTE) pla[q] = la[q], plb[q] = lb[q];
                la[q] = nla[q], lb[q] = nlb[q];
            }
        }
        pw = npw;
        lpw = nlpw;
    }
    if (s1 == steps) {                                // the schedule's last position
        const int32_t last = dst[steps];
        if constexpr (LOWER == 1) lower_rows(last, last >= 0 && last < in_dim, la, lb);
        store_row(last, carry, RECOMPUTE ? pla : la, RECOMPUTE ? plb : lb);
    }
}

// grad_x rows of the vertices that backward_chain_kernel could not finish in one write: vertex
// fix_vertex[i] is the sum, in slot order, of overflow rows [fix_start[i], fix_start[i + 1])
// (no rows: the input feeds no neuron and its gradient is zero).
// compact: row i of gx instead of row fix_vertex[i] (gx then has n_fix rows only).
template <typename T, int VEC>
__global__ __launch_bounds__(DL_BLOCK) void backward_fix_kernel(const T *__restrict__ overflow,
                                                                const int32_t *__restrict__ fix_vertex,
                                                                const int32_t *__restrict__ fix_start,
                                                                T *__restrict__ gx, int64_t n_fix, int64_t ncols,
                                                                bool compact) {
    typedef typename Acc<T>::type C;
    typedef Pack<T, VEC> P;
    const int wave = dl_wave_in_block();
    const int lane = dl_lane();
    const int64_t i = (int64_t) blockIdx.x * 4 + wave;
    if (i >= n_fix) return;
    const int64_t v = compact ? i : (int64_t) fix_vertex[i];
    const int32_t r0 = fix_start[i], r1 = fix_start[i + 1];
    const P *ov = reinterpret_cast<const P *>(overflow);
    P *out = reinterpret_cast<P *>(gx);
    for (int64_t col = (int64_t) blockIdx.y * DL_WAVE + lane; col < ncols; col += (int64_t) gridDim.y * DL_WAVE) {
        C acc[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[e] = (C) 0;
        for (int32_t r = r0; r < r1; ++r) {
            const P part = ov[(int64_t) r * ncols + col];
#pragma unroll
            for (int e = 0; e < VEC; ++e) acc[e] += up<T>(part.v[e]);
        }
        P res;
#pragma unroll
        for (int e = 0; e < VEC; ++e) res.v[e] = down<T, C>(acc[e]);
        out[v * ncols + col] = res;
    }
}

// backward_w of the layer below for the few vertices whose grad_x row backward_fix_kernel finished:
// neuron list[i] of that layer, its grad_y row = row i of `rows`.  One wave per neuron, the sums in
// the order of backward_w_kernel.
template <typename T, int VEC>
__global__ __launch_bounds__(DL_BLOCK) void backward_w_rows_kernel(LowerLayer<T> low, const int32_t *__restrict__ list,
                                                                   const T *__restrict__ rows, int64_t n_list,
                                                                   int64_t ncols) {
    typedef typename Acc<T>::type C;
    typedef Pack<T, VEC> P;
    const int lane = dl_lane();
    const int64_t i = (int64_t) blockIdx.x * 4 + dl_wave_in_block();
    if (i >= n_list) return;
    const int64_t n = list[i];
    const P *xv = reinterpret_cast<const P *>(low.x);
    const P *gv = reinterpret_cast<const P *>(rows) + i * ncols;
    const int64_t ia = low.a[n], ib = low.b[n];
    C s00 = (C) 0, s01 = (C) 0, s10 = (C) 0, s11 = (C) 0;
    for (int64_t col = lane; col < ncols; col += DL_WAVE) {
        const P va = xv[ia * ncols + col], vb = xv[ib * ncols + col], vg = gv[col];
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            const C av = up<T>(va.v[e]), bv = up<T>(vb.v[e]), g = up<T>(vg.v[e]);
            const C ga = g * av, gna = g - ga;
            const C t11 = ga * bv, t01 = gna * bv;
            s11 += t11;
            s10 += ga - t11;
            s01 += t01;
            s00 += gna - t01;
        }
    }
    wave_sum4(s00, s01, s10, s11, lane);
    store_grad_w<T>(lane, true, n, s00, s01, s10, s11, low.probs, low.gw);
}

// grad_w from the per-segment corner sums of backward_chain_kernel, added in segment order.
// One 16-lane row per neuron (4 neurons per wave).
template <typename T>
__global__ __launch_bounds__(DL_BLOCK) void backward_w_finish_kernel(const typename Acc<T>::type *__restrict__ partial,
                                                                     const T *__restrict__ probs, T *__restrict__ gw,
                                                                     int64_t out_dim, int segments, bool w32) {
    typedef typename Acc<T>::type C;
    const int lane = dl_lane();
    const int64_t n = ((int64_t) blockIdx.x * 4 + dl_wave_in_block()) * 4 + (lane >> 4);
    const bool valid = n < out_dim;
    const int gate = lane & 15;
    C sum[4] = {(C) 0, (C) 0, (C) 0, (C) 0};
    if (valid)
        for (int g = 0; g < segments; ++g)
#pragma unroll
            for (int c = 0; c < 4; ++c) sum[c] += partial[((int64_t) g * out_dim + n) * 4 + c];
    C r = (C) 0;
    if (gate & 8) r += sum[0];
    if (gate & 4) r += sum[1];
    if (gate & 2) r += sum[2];
    if (gate & 1) r += sum[3];
    if (probs != nullptr) {
        const C p = valid ? wload<T>(probs, n * 16 + gate, w32) : (C) 0;
        const C dot = row16_sum(p * r);
        r = p * (r - dot);
    }
    if (valid) wstore<T>(gw, n * 16 + gate, r, w32);
}

template <typename T> struct Vec16 { static constexpr int n = 16 / (int) sizeof(T); };

unsigned col_tiles(int64_t ncols) {
    int64_t t = dl_ceil_div(ncols, DL_WAVE);
    return (unsigned) (t > 65535 ? 65535 : t);
}

template <typename T, bool LOGITS>
int forward_t(const void *x, const int64_t *a, const int64_t *b, const void *w, void *y, void *probs, int64_t out_dim,
              int64_t batch, hipStream_t s, bool w32 = false) {
    constexpr int NPW = 4;
    const int64_t blocks = dl_ceil_div(out_dim, 4 * NPW);
    if (out_dim > 0x7fffffffLL) return DL_ERR_TOO_LARGE;     // neuron ids travel as int32 inside the kernel
    constexpr int V = Vec16<T>::n;
    if (batch % V == 0 && dl_aligned(x, 16) && dl_aligned(y, 16)) {
        DL_LAUNCH((forward_kernel<T, V, NPW, LOGITS>), dim3((unsigned) blocks, col_tiles(batch / V)),
                           dim3(DL_BLOCK), 0, s, (const T *) x, a, b, (const T *) w, (T *) y, (T *) probs, out_dim,
                           batch / V, w32);
    } else {
        DL_LAUNCH((forward_kernel<T, 1, NPW, LOGITS>), dim3((unsigned) blocks, col_tiles(batch)), dim3(DL_BLOCK),
                           0, s, (const T *) x, a, b, (const T *) w, (T *) y, (T *) probs, out_dim, batch, w32);
    }
    return dl_launch_status();
}

template <typename T>
int backward_w_t(const void *x, const int64_t *a, const int64_t *b, const void *gy, const void *probs, void *gw,
                 int64_t out_dim, int64_t batch, hipStream_t s, int64_t gdiv = 0, bool w32 = false) {
    constexpr int NPW = 2;       // neurons per wave when the workgroup's waves split a neuron's batch
    constexpr int NPW1 = 2;      // ... when a wave owns whole rows: short rows, more neurons' loads in flight per wave
    constexpr int V = Vec16<T>::n;
    const bool vec = batch % V == 0 && dl_aligned(x, 16) && dl_aligned(gy, 16);
    const int64_t ncols = vec ? batch / V : batch;
    // Split one neuron's batch over the four waves once every wave still gets whole segments.
    const bool split = ncols >= 8 * DL_WAVE;
    const int64_t blocks = split ? dl_ceil_div(out_dim, NPW) : dl_ceil_div(out_dim, 4 * NPW1);
    if (blocks > 0x7fffffffLL) return DL_ERR_TOO_LARGE;
    const dim3 grid((unsigned) blocks), block(DL_BLOCK);
    const T *xp = (const T *) x, *gp = (const T *) gy, *pp = (const T *) probs;
    T *wp = (T *) gw;
    if (vec && split)
        DL_LAUNCH((backward_w_kernel<T, V, NPW, 4>), grid, block, 0, s, xp, a, b, gp, pp, wp, out_dim, ncols, gdiv, w32);
    else if (vec)
        DL_LAUNCH((backward_w_kernel<T, V, NPW1, 1>), grid, block, 0, s, xp, a, b, gp, pp, wp, out_dim, ncols, gdiv, w32);
    else if (split)
        DL_LAUNCH((backward_w_kernel<T, 1, NPW, 4>), grid, block, 0, s, xp, a, b, gp, pp, wp, out_dim, ncols, gdiv, w32);
    else
        DL_LAUNCH((backward_w_kernel<T, 1, NPW1, 1>), grid, block, 0, s, xp, a, b, gp, pp, wp, out_dim, ncols, gdiv, w32);
    return dl_launch_status();
}

template <typename T>
int backward_x_t(const void *x, const int64_t *a, const int64_t *b, const void *w, const void *gy,
                 const int64_t *start, const int64_t *idx, void *gx, int64_t in_dim, int64_t batch, double scale,
                 hipStream_t s, int64_t gdiv = 0, bool w32 = false) {
    typedef typename Acc<T>::type C;
    constexpr int V = Vec16<T>::n;
    const int64_t blocks = dl_ceil_div(in_dim, 4);
    if (blocks > 0x7fffffffLL) return DL_ERR_TOO_LARGE;
    if (batch % V == 0 && dl_aligned(x, 16) && dl_aligned(gy, 16) && dl_aligned(gx, 16)) {
        DL_LAUNCH((backward_x_kernel<T, V>), dim3((unsigned) blocks, col_tiles(batch / V)), dim3(DL_BLOCK), 0, s,
                           (const T *) x, a, b, (const T *) w, (const T *) gy, start, idx, (T *) gx, in_dim, batch / V,
                           (C) scale, gdiv, w32);
    } else {
        DL_LAUNCH((backward_x_kernel<T, 1>), dim3((unsigned) blocks, col_tiles(batch)), dim3(DL_BLOCK), 0, s,
                           (const T *) x, a, b, (const T *) w, (const T *) gy, start, idx, (T *) gx, in_dim, batch,
                           (C) scale, gdiv, w32);
    }
    return dl_launch_status();
}

// ------------------------------------------------------------------------------------------
// GroupSum on the feature-major layout.
//   forward : y[r, c] = (1/tau) * sum_{n in class c} x[n, r]       x [out, B] -> y [B, k]
//   backward: gx[n, r] = g[r, class(n)] / tau                      g [B, k]   -> gx [out, B]
// Forward is two passes with a fixed summation order: pass 1 sums SPLIT-th parts of every
// class block over the rows (lanes along the batch, the workgroup's four waves interleave
// rows and combine through LDS) into partial[s, c, r]; pass 2 adds the partials in order.
// ------------------------------------------------------------------------------------------
template <typename T, int VEC>
__global__ __launch_bounds__(DL_BLOCK) void group_sum_partial_kernel(const T *__restrict__ x,
                                                                     typename Acc<T>::type *__restrict__ partial,
                                                                     int64_t per_class, int64_t ncols, int64_t k,
                                                                     int64_t rows_per_split) {
    typedef typename Acc<T>::type C;
    typedef Pack<T, VEC> P;
    __shared__ C lds[4][DL_WAVE * VEC];
    const int wave = dl_wave_in_block();
    const int lane = dl_lane();
    const int64_t col = (int64_t) blockIdx.x * DL_WAVE + lane;
    const int64_t cls = blockIdx.y, split = blockIdx.z;
    int64_t r0 = split * rows_per_split, r1 = r0 + rows_per_split;
    if (r1 > per_class) r1 = per_class;
    C acc[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[e] = (C) 0;
    if (col < ncols) {
        const P *xv = reinterpret_cast<const P *>(x) + (cls * per_class) * ncols + col;
        int64_t r = r0 + wave;
        for (; r + 12 < r1; r += 16) {      // four independent row loads in flight per wave
            const P v0 = xv[r * ncols], v1 = xv[(r + 4) * ncols], v2 = xv[(r + 8) * ncols], v3 = xv[(r + 12) * ncols];
#pragma unroll
            for (int e = 0; e < VEC; ++e) acc[e] += (up<T>(v0.v[e]) + up<T>(v1.v[e])) + (up<T>(v2.v[e]) + up<T>(v3.v[e]));
        }
        for (; r < r1; r += 4) {
            const P v = xv[r * ncols];
#pragma unroll
            for (int e = 0; e < VEC; ++e) acc[e] += up<T>(v.v[e]);
        }
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) lds[wave][lane * VEC + e] = acc[e];
    __syncthreads();
    if (wave == 0 && col < ncols) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            const int i = lane * VEC + e;
            const C sum = (lds[0][i] + lds[1][i]) + (lds[2][i] + lds[3][i]);
            partial[((int64_t) split * k + cls) * (ncols * VEC) + col * VEC + e] = sum;
        }
    }
}

// The last LogicLayer and GroupSum in one pass: pass 1 of the sum above with the rows computed on
// the fly, y[n, r] = layer(x)[n, r] for the neurons of the class block, so the layer's output
// (and, in the backward pass, the broadcast gradient) never exists in memory.  Grid and partial
// layout as group_sum_partial_kernel; a wave takes four consecutive neurons at a time (their
// corner coefficients are computed together), the workgroup's waves interleave groups of four.
// LOGITS: `w` holds logits; the probabilities go to `probs` (column tile 0 only).
template <typename T, int VEC, bool LOGITS>
__global__ __launch_bounds__(DL_BLOCK) void forward_group_sum_kernel(const T *__restrict__ x, const int64_t *__restrict__ a,
                                                                     const int64_t *__restrict__ b, const T *__restrict__ w,
                                                                     T *__restrict__ probs,
                                                                     typename Acc<T>::type *__restrict__ partial,
                                                                     int64_t per_class, int64_t ncols, int64_t k,
                                                                     int64_t rows_per_split) {
    typedef typename Acc<T>::type C;
    typedef Pack<T, VEC> P;
    __shared__ C lds[4][DL_WAVE * VEC];
    const int wave = dl_wave_in_block();
    const int lane = dl_lane();
    const int64_t col = (int64_t) blockIdx.x * DL_WAVE + lane;
    const bool live = col < ncols;
    const int64_t cls = blockIdx.y, split = blockIdx.z;
    int64_t r0 = split * rows_per_split, r1 = r0 + rows_per_split;
    if (r1 > per_class) r1 = per_class;
    const P *xv = reinterpret_cast<const P *>(x) + (live ? col : 0);
    C acc[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[e] = (C) 0;
    for (int64_t r = r0 + 4 * wave; r < r1; r += 16) {           // uniform per wave
        int64_t ia[4], ib[4];
        int32_t ids[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const bool valid = r + j < r1;
            const int64_t n = cls * per_class + (valid ? r + j : r);
            ia[j] = a[n];
            ib[j] = b[n];
            ids[j] = valid ? (int32_t) n : -1;
        }
        C p00[4], p10[4], d0[4], d1[4];
        corners4<T, LOGITS>(w, ids, lane, blockIdx.x == 0, probs, p00, p10, d0, d1);
        P va[4], vb[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            va[j] = xv[ia[j] * ncols];
            vb[j] = xv[ib[j] * ncols];
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (ids[j] >= 0) {                                   // uniform
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    // rounded to T like the stored activation would have been
                    acc[e] += up<T>(down<T, C>(mix<C>(up<T>(va[j].v[e]), up<T>(vb[j].v[e]), p00[j], p10[j], d0[j], d1[j])));
                }
            }
        }
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) lds[wave][lane * VEC + e] = acc[e];
    __syncthreads();
    if (wave == 0 && live) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            const int i = lane * VEC + e;
            const C sum = (lds[0][i] + lds[1][i]) + (lds[2][i] + lds[3][i]);
            partial[((int64_t) split * k + cls) * (ncols * VEC) + col * VEC + e] = sum;
        }
    }
}

// One wave per 64 consecutive samples of one class; the four waves of a workgroup take
// interleaved splits and are added in wave order, so the summation order is fixed.
template <typename T>
__global__ __launch_bounds__(DL_BLOCK) void group_sum_finish_kernel(const typename Acc<T>::type *__restrict__ partial,
                                                                    T *__restrict__ y, int64_t batch, int64_t k,
                                                                    int splits, typename Acc<T>::type inv_tau) {
    typedef typename Acc<T>::type C;
    __shared__ C lds[4][DL_WAVE];
    const int wave = dl_wave_in_block();
    const int lane = dl_lane();
    const int64_t r = (int64_t) blockIdx.x * DL_WAVE + lane;
    const int64_t c = blockIdx.y;
    C sum = (C) 0;
    if (r < batch)
        for (int s = wave; s < splits; s += 4) sum += partial[((int64_t) s * k + c) * batch + r];
    lds[wave][lane] = sum;
    __syncthreads();
    if (wave == 0 && r < batch)
        y[r * k + c] = down<T, C>(((lds[0][lane] + lds[1][lane]) + (lds[2][lane] + lds[3][lane])) * inv_tau);
}

template <typename T, int VEC>
__global__ __launch_bounds__(DL_BLOCK) void group_sum_backward_kernel(const T *__restrict__ g, T *__restrict__ gx,
                                                                      int64_t out_dim, int64_t per_class,
                                                                      int64_t ncols, int64_t k,
                                                                      typename Acc<T>::type inv_tau) {
    typedef typename Acc<T>::type C;
    typedef Pack<T, VEC> P;
    const int wave = dl_wave_in_block();
    const int lane = dl_lane();
    const int64_t col = (int64_t) blockIdx.x * DL_WAVE + lane;
    if (col >= ncols) return;
    constexpr int ROWS = 16;                                              // rows per wave
    const int64_t n0 = ((int64_t) blockIdx.y * 4 + wave) * ROWS;
    P *ov = reinterpret_cast<P *>(gx);
    int64_t cached_cls = -1;
    P val;
    for (int64_t n = n0; n < n0 + ROWS && n < out_dim; ++n) {
        const int64_t cls = n / per_class;
        if (cls != cached_cls) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) val.v[e] = down<T, C>(up<T>(g[(col * VEC + e) * k + cls]) * inv_tau);
            cached_cls = cls;
        }
        ov[n * ncols + col] = val;
    }
}

template <typename T>
int group_sum_forward_t(const void *x, void *y, void *workspace, int64_t out_dim, int64_t batch, int64_t k, int splits,
                        double tau, hipStream_t s) {
    typedef typename Acc<T>::type C;
    constexpr int V = Vec16<T>::n;
    const int64_t per_class = out_dim / k;
    const int64_t rows_per_split = dl_ceil_div(per_class, splits);
    const bool vec = batch % V == 0 && dl_aligned(x, 16);
    const int64_t ncols = vec ? batch / V : batch;
    const int64_t gx = dl_ceil_div(ncols, DL_WAVE);
    if (gx > 0x7fffffffLL || k > 65535) return DL_ERR_TOO_LARGE;
    const dim3 grid((unsigned) gx, (unsigned) k, (unsigned) splits);
    if (vec)
        DL_LAUNCH((group_sum_partial_kernel<T, V>), grid, dim3(DL_BLOCK), 0, s, (const T *) x, (C *) workspace,
                           per_class, ncols, k, rows_per_split);
    else
        DL_LAUNCH((group_sum_partial_kernel<T, 1>), grid, dim3(DL_BLOCK), 0, s, (const T *) x, (C *) workspace,
                           per_class, ncols, k, rows_per_split);
    int st = dl_launch_status();
    if (st != DL_OK) return st;
    const int64_t blocks = dl_ceil_div(batch, DL_WAVE);
    if (blocks > 0x7fffffffLL) return DL_ERR_TOO_LARGE;
    DL_LAUNCH((group_sum_finish_kernel<T>), dim3((unsigned) blocks, (unsigned) k), dim3(DL_BLOCK), 0, s,
                       (const C *) workspace, (T *) y, batch, k, splits, (C) (1.0 / tau));
    return dl_launch_status();
}

template <typename T>
int group_sum_backward_t(const void *g, void *gx, int64_t out_dim, int64_t batch, int64_t k, double tau, hipStream_t s) {
    typedef typename Acc<T>::type C;
    constexpr int V = Vec16<T>::n;
    const bool vec = batch % V == 0 && dl_aligned(gx, 16);
    const int64_t ncols = vec ? batch / V : batch;
    const int64_t gxd = dl_ceil_div(ncols, DL_WAVE), gyd = dl_ceil_div(out_dim, 64);
    if (gxd > 0x7fffffffLL || gyd > 65535) return DL_ERR_TOO_LARGE;
    const dim3 grid((unsigned) gxd, (unsigned) gyd);
    if (vec)
        DL_LAUNCH((group_sum_backward_kernel<T, V>), grid, dim3(DL_BLOCK), 0, s, (const T *) g, (T *) gx, out_dim,
                           out_dim / k, ncols, k, (C) (1.0 / tau));
    else
        DL_LAUNCH((group_sum_backward_kernel<T, 1>), grid, dim3(DL_BLOCK), 0, s, (const T *) g, (T *) gx, out_dim,
                           out_dim / k, ncols, k, (C) (1.0 / tau));
    return dl_launch_status();
}

int group_sum_splits(int64_t out_dim, int64_t batch, int64_t k);

template <typename T>
int forward_group_sum_t(const void *x, const int64_t *a, const int64_t *b, const void *w, void *probs, void *y,
                        void *workspace, int64_t out_dim, int64_t batch, int64_t k, double tau, hipStream_t s) {
    typedef typename Acc<T>::type C;
    constexpr int V = Vec16<T>::n;
    const int splits = group_sum_splits(out_dim, batch, k);
    const int64_t per_class = out_dim / k;
    const int64_t rows_per_split = dl_ceil_div(dl_ceil_div(per_class, splits), 16) * 16;     // whole groups of four per wave
    const bool vec = batch % V == 0 && dl_aligned(x, 16);
    const int64_t ncols = vec ? batch / V : batch;
    const int64_t gx = dl_ceil_div(ncols, DL_WAVE);
    if (gx > 0x7fffffffLL || k > 65535 || out_dim > 0x7fffffffLL) return DL_ERR_TOO_LARGE;
    const dim3 grid((unsigned) gx, (unsigned) k, (unsigned) splits);
    const T *xp = (const T *) x, *wp = (const T *) w;
#define DL_LAUNCH_FGS(VV, LG)                                                                                               \
    DL_LAUNCH((forward_group_sum_kernel<T, VV, LG>), grid, dim3(DL_BLOCK), 0, s, xp, a, b, wp, (T *) probs, (C *) workspace, \
              per_class, ncols, k, rows_per_split)
    if (vec && probs) DL_LAUNCH_FGS(V, true);
    else if (vec) DL_LAUNCH_FGS(V, false);
    else if (probs) DL_LAUNCH_FGS(1, true);
    else DL_LAUNCH_FGS(1, false);
#undef DL_LAUNCH_FGS
    int st = dl_launch_status();
    if (st != DL_OK) return st;
    const int64_t blocks = dl_ceil_div(batch, DL_WAVE);
    if (blocks > 0x7fffffffLL) return DL_ERR_TOO_LARGE;
    DL_LAUNCH((group_sum_finish_kernel<T>), dim3((unsigned) blocks, (unsigned) k), dim3(DL_BLOCK), 0, s,
                       (const C *) workspace, (T *) y, batch, k, splits, (C) (1.0 / tau));
    return dl_launch_status();
}

// Number of row splits per class: enough workgroups to fill the chip, at least 64 rows each.
int group_sum_splits(int64_t out_dim, int64_t batch, int64_t k) {
    const int64_t per_class = out_dim / k;
    const int64_t col_tiles = dl_ceil_div(batch, 4 * DL_WAVE);
    int64_t want = dl_ceil_div(1024, col_tiles * k);
    const int64_t max_by_rows = per_class / 64 > 0 ? per_class / 64 : 1;
    if (want > max_by_rows) want = max_by_rows;
    if (want < 1) want = 1;
    if (want > 1024) want = 1024;
    return (int) want;
}

#define DL_TRAIN_CHUNK 8     // must equal the chunk the schedule was built with (dl_eval_schedule_chunk)
#define DL_FWD_ROWS_MIN 128  // vectors per row above which forward_chain_rows_kernel takes over

// Longest row (in 16-byte vectors) the whole-row kernels take: 16 segments of 256.
#define DL_ROWS_MAX_VECTORS (16 * 4 * DL_WAVE)

int row_segments(int64_t ncols) { return (int) dl_ceil_div(ncols, 4 * DL_WAVE); }

// Steps per wave of the kernels in which a wave owns whole rows: long chunks re-read fewer rows at
// their seams, short ones give more waves to hide latency with; keep about three waves per SIMD.
int chain_chunk(int64_t steps) {
    for (int chunk = 32; chunk > 8; chunk /= 2)
        if (steps / chunk >= 3000) return chunk;
    return 8;
}

template <typename T, bool LOGITS>
int forward_chain_t(const void *x, const int32_t *verts, const int32_t *neuron, const uint8_t *flip, int64_t steps,
                    const void *w, void *y, void *probs, int64_t batch, hipStream_t s, bool w32 = false) {
    constexpr int V = Vec16<T>::n;
    if (batch % V != 0 || !dl_aligned(x, 16) || !dl_aligned(y, 16)) return DL_ERR_TOO_LARGE;
    const int64_t nchunks = steps / DL_TRAIN_CHUNK, ncols = batch / V;
    const T *xp = (const T *) x, *wp = (const T *) w;
    if (ncols > DL_FWD_ROWS_MIN && ncols <= DL_ROWS_MAX_VECTORS) {
        // rows of 2 KB and more: a wave takes whole rows, or segments of 4 KB
        const int segments = row_segments(ncols);
        const int chunk = chain_chunk(steps * segments);
        const int64_t blocks = dl_ceil_div(dl_ceil_div(steps, chunk), 4);
        if (blocks > 0x7fffffffLL) return DL_ERR_TOO_LARGE;
        const dim3 grid((unsigned) blocks, (unsigned) segments), block(DL_BLOCK);
        if (ncols <= 2 * DL_WAVE)
            DL_LAUNCH((forward_chain_rows_kernel<T, V, 2, LOGITS>), grid, block, 0, s, xp, verts, neuron, flip, wp,
                               (T *) y, (T *) probs, steps, chunk, ncols, w32);
        else
            DL_LAUNCH((forward_chain_rows_kernel<T, V, 4, LOGITS>), grid, block, 0, s, xp, verts, neuron, flip, wp,
                               (T *) y, (T *) probs, steps, chunk, ncols, w32);
        return dl_launch_status();
    }
    const int64_t blocks = dl_ceil_div(nchunks, 4);
    if (blocks > 0x7fffffffLL) return DL_ERR_TOO_LARGE;
    if (V >= 2 && ncols <= DL_WAVE / 2) {
        // short rows: 8-byte vectors put a row on all 64 lanes instead of half of them
        constexpr int H = V >= 2 ? V / 2 : 1;
        DL_LAUNCH((forward_chain_kernel<T, H, DL_TRAIN_CHUNK, LOGITS>), dim3((unsigned) blocks, 1), dim3(DL_BLOCK), 0, s, xp,
                  verts, neuron, flip, wp, (T *) y, (T *) probs, nchunks, 2 * ncols, w32);
        return dl_launch_status();
    }
    DL_LAUNCH((forward_chain_kernel<T, V, DL_TRAIN_CHUNK, LOGITS>), dim3((unsigned) blocks, col_tiles(ncols)),
                       dim3(DL_BLOCK), 0, s, xp, verts, neuron, flip, wp, (T *) y, (T *) probs, nchunks, ncols, w32);
    return dl_launch_status();
}

template <typename T, bool LOGITS>
int forward_chain_lower_t(const void *lx, const int64_t *la, const int64_t *lb, const void *lw, void *lprobs,
                          const int32_t *verts, const int32_t *neuron, const uint8_t *flip, int64_t steps, const void *w,
                          void *y, void *probs, int64_t batch, hipStream_t s) {
    constexpr int V = Vec16<T>::n;
    if (batch % V != 0 || !dl_aligned(lx, 16) || !dl_aligned(y, 16)) return DL_ERR_TOO_LARGE;
    const int64_t nchunks = steps / DL_TRAIN_CHUNK, ncols = batch / V;
    if (ncols > DL_FWD_ROWS_MIN) return DL_ERR_TOO_LARGE;        // rows of at most 2 KB
    const int64_t blocks = dl_ceil_div(nchunks, 4);
    if (blocks > 0x7fffffffLL) return DL_ERR_TOO_LARGE;
    // one wave takes every column tile of its chunk (at most two): the corner coefficients are formed once
    DL_LAUNCH((forward_chain_lower_kernel<T, V, DL_TRAIN_CHUNK, LOGITS>), dim3((unsigned) blocks, 1),
              dim3(DL_BLOCK), 0, s, (const T *) lx, la, lb, (const T *) lw, (T *) lprobs, verts, neuron, flip, (const T *) w,
              (T *) y, (T *) probs, nchunks, ncols);
    return dl_launch_status();
}

template <typename T>
int backward_w_chain_t(const void *x, const int32_t *verts, const int32_t *neuron, const uint8_t *flip, int64_t steps,
                       const void *gy, const void *probs, void *gw, int64_t batch, hipStream_t s, int64_t gdiv = 0,
                       bool w32 = false) {
    constexpr int V = Vec16<T>::n;
    if (batch % V != 0 || !dl_aligned(x, 16) || !dl_aligned(gy, 16)) return DL_ERR_TOO_LARGE;
    const int64_t nchunks = steps / DL_TRAIN_CHUNK, ncols = batch / V;
    const int64_t blocks = dl_ceil_div(nchunks, 4);
    if (blocks > 0x7fffffffLL || ncols > 4 * DL_WAVE) return DL_ERR_TOO_LARGE;   // a lane holds at most 4 vectors of a row
    const dim3 grid((unsigned) blocks), block(DL_BLOCK);
    const T *xp = (const T *) x, *gp = (const T *) gy, *pp = (const T *) probs;
    if (ncols <= DL_WAVE)
        DL_LAUNCH((backward_w_chain_kernel<T, V, 1, DL_TRAIN_CHUNK>), grid, block, 0, s, xp, verts, neuron, flip,
                           gp, pp, (T *) gw, nchunks, ncols, gdiv, w32);
    else if (ncols <= 2 * DL_WAVE)
        DL_LAUNCH((backward_w_chain_kernel<T, V, 2, DL_TRAIN_CHUNK>), grid, block, 0, s, xp, verts, neuron, flip,
                           gp, pp, (T *) gw, nchunks, ncols, gdiv, w32);
    else
        DL_LAUNCH((backward_w_chain_kernel<T, V, 4, DL_TRAIN_CHUNK>), grid, block, 0, s, xp, verts, neuron, flip,
                           gp, pp, (T *) gw, nchunks, ncols, gdiv, w32);
    return dl_launch_status();
}

template <typename T> int64_t backward_partial_bytes(int64_t out_dim, int64_t batch) {
    constexpr int V = Vec16<T>::n;
    const int segments = batch % V == 0 ? row_segments(batch / V) : 1;
    return segments > 1 ? (int64_t) segments * out_dim * 4 * (int64_t) sizeof(typename Acc<T>::type) : 0;
}

template <typename T>
int backward_chain_t(const void *x, const int32_t *verts, const int32_t *neuron, const uint8_t *flip, const int32_t *dst,
                     int64_t steps, const void *w, const void *gy, bool softmax_backward, const int32_t *fix_vertex,
                     const int32_t *fix_start, int64_t n_fix, int64_t overflow_rows, void *gw, void *gx, void *workspace,
                     int64_t in_dim, int64_t out_dim, int64_t batch, double scale, hipStream_t s, int64_t gdiv = 0,
                     const LowerLayer<T> *lower = nullptr, bool w32 = false) {
    typedef typename Acc<T>::type C;
    constexpr int V = Vec16<T>::n;
    if (batch % V != 0 || !dl_aligned(x, 16) || !dl_aligned(gy, 16) || !dl_aligned(gx, 16) || !dl_aligned(workspace, 16))
        return DL_ERR_TOO_LARGE;
    if (!x && (!lower || !lower->w)) return DL_ERR_INVALID_ARGUMENT;     // x may only be left out for recomputation
    const int64_t ncols = batch / V;
    if (ncols > DL_ROWS_MAX_VECTORS) return DL_ERR_TOO_LARGE;
    const int segments = row_segments(ncols);
    // with `lower`: whole rows per wave only, and gx holds the n_fix rows that finish after the pass
    if (lower && (segments > 1 || !dl_aligned(lower->x, 16) || w32)) return DL_ERR_TOO_LARGE;
    const LowerLayer<T> none = {nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
    // workspace: [segments x out x 4 corner sums (only with several segments)] [overflow rows]
    const int64_t partial_bytes = backward_partial_bytes<T>(out_dim, batch);
    if ((partial_bytes > 0 || overflow_rows > 0) && workspace == nullptr) return DL_ERR_INVALID_ARGUMENT;
    C *partial = partial_bytes > 0 ? (C *) workspace : nullptr;
    T *overflow = (T *) ((char *) workspace + partial_bytes);
    const int chunk = chain_chunk(steps * segments);
    const int64_t blocks = dl_ceil_div(dl_ceil_div(steps, chunk), 4), fix_blocks = dl_ceil_div(n_fix, 4);
    if (blocks > 0x7fffffffLL || fix_blocks > 0x7fffffffLL) return DL_ERR_TOO_LARGE;
    const dim3 grid((unsigned) blocks, (unsigned) segments), block(DL_BLOCK);
    const T *xp = (const T *) x, *wp = (const T *) w, *gp = (const T *) gy, *pp = softmax_backward ? wp : nullptr;
    constexpr int H = V >= 2 ? V / 2 : 1;
#define DL_LAUNCH_BACKWARD_CHAIN(VV, CPL, NC)                                                                               \
    do {                                                                                                                    \
        if (lower && !x)                                                                                                    \
            DL_LAUNCH((backward_chain_kernel<T, VV, CPL, 2>), grid, block, 0, s, xp, verts, neuron, flip, dst, wp, gp,     \
                      pp, (T *) gw, partial, (T *) gx, overflow, steps, chunk, in_dim, out_dim, NC, (C) scale, gdiv, *lower, \
                      false);                                                                                               \
        else if (lower)                                                                                                     \
            DL_LAUNCH((backward_chain_kernel<T, VV, CPL, 1>), grid, block, 0, s, xp, verts, neuron, flip, dst, wp, gp,     \
                      pp, (T *) gw, partial, (T *) gx, overflow, steps, chunk, in_dim, out_dim, NC, (C) scale, gdiv, *lower, \
                      false);                                                                                               \
        else                                                                                                                \
            DL_LAUNCH((backward_chain_kernel<T, VV, CPL, 0>), grid, block, 0, s, xp, verts, neuron, flip, dst, wp, gp,     \
                      pp, (T *) gw, partial, (T *) gx, overflow, steps, chunk, in_dim, out_dim, NC, (C) scale, gdiv, none,   \
                      w32);                                                                                                 \
    } while (0)
    if (V >= 2 && ncols <= DL_WAVE / 2)
        DL_LAUNCH_BACKWARD_CHAIN(H, 1, 2 * ncols);   // short rows: 8-byte vectors use all 64 lanes
    else if (ncols <= DL_WAVE)
        DL_LAUNCH_BACKWARD_CHAIN(V, 1, ncols);
    else if (ncols <= 2 * DL_WAVE)
        DL_LAUNCH_BACKWARD_CHAIN(V, 2, ncols);
    else
        DL_LAUNCH_BACKWARD_CHAIN(V, 4, ncols);
#undef DL_LAUNCH_BACKWARD_CHAIN
    int st = dl_launch_status();
    if (st != DL_OK) return st;
    if (partial != nullptr) {
        const int64_t fin_blocks = dl_ceil_div(out_dim, 16);
        if (fin_blocks > 0x7fffffffLL) return DL_ERR_TOO_LARGE;
        DL_LAUNCH(backward_w_finish_kernel<T>, dim3((unsigned) fin_blocks), block, 0, s, (const C *) partial, pp, (T *) gw,
                  out_dim, segments, w32);
        st = dl_launch_status();
        if (st != DL_OK) return st;
    }
    if (n_fix == 0) return DL_OK;
    DL_LAUNCH((backward_fix_kernel<T, V>), dim3((unsigned) fix_blocks, col_tiles(ncols)), block, 0, s,
              (const T *) overflow, fix_vertex, fix_start, (T *) gx, n_fix, ncols, lower != nullptr);
    st = dl_launch_status();
    if (st != DL_OK || !lower) return st;
    DL_LAUNCH((backward_w_rows_kernel<T, V>), dim3((unsigned) fix_blocks), block, 0, s, *lower, fix_vertex, (const T *) gx,
              n_fix, ncols);
    return dl_launch_status();
}

// DL_F16_W32 / DL_F64_W32 (activations in half / double, gate weights and their gradients in fp32) -> the
// activations' dtype; returns whether the weights are fp32
bool weights_fp32(int &dtype) {
    if (dtype == DL_F16_W32) {
        dtype = DL_F16;
        return true;
    }
    if (dtype == DL_F64_W32) {
        dtype = DL_F64;
        return true;
    }
    return false;
}

}  // namespace

extern "C" int64_t dl_logic_backward_chained_workspace_bytes(int64_t overflow_rows, int64_t out_dim, int64_t batch,
                                                             int dtype) {
    if (overflow_rows < 0 || out_dim < 0 || batch < 0) return -DL_ERR_INVALID_ARGUMENT;
    weights_fp32(dtype);
    switch (dtype) {
    case DL_F16: return backward_partial_bytes<__half>(out_dim, batch) + overflow_rows * batch * 2;
    case DL_F32: return backward_partial_bytes<float>(out_dim, batch) + overflow_rows * batch * 4;
    case DL_F64: return backward_partial_bytes<double>(out_dim, batch) + overflow_rows * batch * 8;
    default: return -DL_ERR_DTYPE;
    }
}

extern "C" int dl_logic_backward_chained(const void *x, const int32_t *verts, const int32_t *neuron, const uint8_t *flip,
                                         const int32_t *dst, int64_t steps, const void *w, const void *grad_y,
                                         int softmax_backward, const int32_t *fix_vertex, const int32_t *fix_start,
                                         int64_t n_fix, int64_t overflow_rows, void *grad_w, void *grad_x,
                                         void *workspace, int64_t in_dim, int64_t out_dim, int64_t batch, double scale,
                                         int dtype, void *stream) {
    const bool w32 = weights_fp32(dtype);
    if (dtype != DL_F16 && dtype != DL_F32 && dtype != DL_F64) return DL_ERR_DTYPE;
    if (in_dim <= 0 || out_dim <= 0 || batch <= 0 || steps < out_dim || n_fix < 0 || n_fix > in_dim || overflow_rows < 0)
        return DL_ERR_INVALID_ARGUMENT;
    if (!x || !verts || !neuron || !flip || !dst || !w || !grad_y || !grad_w || !grad_x) return DL_ERR_INVALID_ARGUMENT;
    if (n_fix > 0 && (!fix_vertex || !fix_start)) return DL_ERR_INVALID_ARGUMENT;
    hipStream_t s = (hipStream_t) stream;
    const bool sb = softmax_backward != 0;
    switch (dtype) {
    case DL_F16:
        return backward_chain_t<__half>(x, verts, neuron, flip, dst, steps, w, grad_y, sb, fix_vertex, fix_start, n_fix,
                                        overflow_rows, grad_w, grad_x, workspace, in_dim, out_dim, batch, scale, s, 0, nullptr,
                                        w32);
    case DL_F32:
        return backward_chain_t<float>(x, verts, neuron, flip, dst, steps, w, grad_y, sb, fix_vertex, fix_start, n_fix,
                                       overflow_rows, grad_w, grad_x, workspace, in_dim, out_dim, batch, scale, s);
    default:
        return backward_chain_t<double>(x, verts, neuron, flip, dst, steps, w, grad_y, sb, fix_vertex, fix_start, n_fix,
                                        overflow_rows, grad_w, grad_x, workspace, in_dim, out_dim, batch, scale, s, 0, nullptr,
                                        w32);
    }
}

extern "C" int dl_logic_backward_chained_lower(const void *x, const int32_t *verts, const int32_t *neuron,
                                               const uint8_t *flip, const int32_t *dst, int64_t steps, const void *w,
                                               const void *grad_y, int softmax_backward, const int32_t *fix_vertex,
                                               const int32_t *fix_start, int64_t n_fix, int64_t overflow_rows,
                                               void *grad_w, void *fix_rows, void *workspace, const void *x_lower,
                                               const int64_t *a_lower, const int64_t *b_lower, const void *w_lower,
                                               int softmax_backward_lower, void *grad_w_lower, int64_t in_dim,
                                               int64_t out_dim, int64_t batch, double scale, int dtype, void *stream) {
    if (dtype != DL_F16 && dtype != DL_F32 && dtype != DL_F64) return DL_ERR_DTYPE;
    if (in_dim <= 0 || out_dim <= 0 || batch <= 0 || steps < out_dim || n_fix < 0 || n_fix > in_dim || overflow_rows < 0)
        return DL_ERR_INVALID_ARGUMENT;
    if (!verts || !neuron || !flip || !dst || !w || !grad_y || !grad_w || !x_lower || !a_lower || !b_lower || !grad_w_lower)
        return DL_ERR_INVALID_ARGUMENT;
    if ((softmax_backward_lower || !x) && !w_lower) return DL_ERR_INVALID_ARGUMENT;
    if (n_fix > 0 && (!fix_vertex || !fix_start || !fix_rows)) return DL_ERR_INVALID_ARGUMENT;
    // recomputing x needs the lower layer's probabilities exactly as its forward pass used them; the fp16 kernels
    // form them in fp32 and round only what they store
    if (!x && dtype == DL_F16) return DL_ERR_TOO_LARGE;
    hipStream_t s = (hipStream_t) stream;
    const bool sb = softmax_backward != 0;
    switch (dtype) {
    case DL_F16: {
        const LowerLayer<__half> low = {(const __half *) x_lower, a_lower, b_lower, (const __half *) w_lower,
                                        softmax_backward_lower ? (const __half *) w_lower : nullptr, (__half *) grad_w_lower};
        return backward_chain_t<__half>(x, verts, neuron, flip, dst, steps, w, grad_y, sb, fix_vertex, fix_start, n_fix,
                                        overflow_rows, grad_w, fix_rows, workspace, in_dim, out_dim, batch, scale, s, 0, &low);
    }
    case DL_F32: {
        const LowerLayer<float> low = {(const float *) x_lower, a_lower, b_lower, (const float *) w_lower,
                                       softmax_backward_lower ? (const float *) w_lower : nullptr, (float *) grad_w_lower};
        return backward_chain_t<float>(x, verts, neuron, flip, dst, steps, w, grad_y, sb, fix_vertex, fix_start, n_fix,
                                       overflow_rows, grad_w, fix_rows, workspace, in_dim, out_dim, batch, scale, s, 0, &low);
    }
    default: {
        const LowerLayer<double> low = {(const double *) x_lower, a_lower, b_lower, (const double *) w_lower,
                                        softmax_backward_lower ? (const double *) w_lower : nullptr, (double *) grad_w_lower};
        return backward_chain_t<double>(x, verts, neuron, flip, dst, steps, w, grad_y, sb, fix_vertex, fix_start, n_fix,
                                        overflow_rows, grad_w, fix_rows, workspace, in_dim, out_dim, batch, scale, s, 0, &low);
    }
    }
}

extern "C" int dl_logic_forward_chained(const void *x, const int32_t *verts, const int32_t *neuron, const uint8_t *flip,
                                        int64_t steps, const void *w, void *y, void *probs, int64_t in_dim,
                                        int64_t out_dim, int64_t batch, int dtype, void *stream) {
    const bool w32 = weights_fp32(dtype);
    if (dtype != DL_F16 && dtype != DL_F32 && dtype != DL_F64) return DL_ERR_DTYPE;
    if (in_dim < 0 || out_dim < 0 || batch <= 0 || steps < out_dim || steps % DL_TRAIN_CHUNK != 0)
        return DL_ERR_INVALID_ARGUMENT;
    if (out_dim == 0) return DL_OK;
    if (!x || !verts || !neuron || !flip || !w || !y || in_dim == 0) return DL_ERR_INVALID_ARGUMENT;
    hipStream_t s = (hipStream_t) stream;
    if (probs) {
        switch (dtype) {
        case DL_F16: return forward_chain_t<__half, true>(x, verts, neuron, flip, steps, w, y, probs, batch, s, w32);
        case DL_F32: return forward_chain_t<float, true>(x, verts, neuron, flip, steps, w, y, probs, batch, s);
        default: return forward_chain_t<double, true>(x, verts, neuron, flip, steps, w, y, probs, batch, s, w32);
        }
    }
    switch (dtype) {
    case DL_F16: return forward_chain_t<__half, false>(x, verts, neuron, flip, steps, w, y, nullptr, batch, s, w32);
    case DL_F32: return forward_chain_t<float, false>(x, verts, neuron, flip, steps, w, y, nullptr, batch, s);
    default: return forward_chain_t<double, false>(x, verts, neuron, flip, steps, w, y, nullptr, batch, s, w32);
    }
}

extern "C" int dl_logic_forward_chained_lower(const void *x_lower, const int64_t *a_lower, const int64_t *b_lower,
                                              const void *w_lower, void *probs_lower, const int32_t *verts,
                                              const int32_t *neuron, const uint8_t *flip, int64_t steps, const void *w,
                                              void *y, void *probs, int64_t in_dim_lower, int64_t in_dim, int64_t out_dim,
                                              int64_t batch, int dtype, void *stream) {
    if (dtype != DL_F16 && dtype != DL_F32 && dtype != DL_F64) return DL_ERR_DTYPE;
    if (in_dim_lower <= 0 || in_dim <= 0 || out_dim < 0 || batch <= 0 || steps < out_dim || steps % DL_TRAIN_CHUNK != 0)
        return DL_ERR_INVALID_ARGUMENT;
    if (out_dim == 0) return DL_OK;
    if (!x_lower || !a_lower || !b_lower || !w_lower || !verts || !neuron || !flip || !w || !y) return DL_ERR_INVALID_ARGUMENT;
    if ((probs == nullptr) != (probs_lower == nullptr)) return DL_ERR_INVALID_ARGUMENT;    // both layers on logits, or neither
    hipStream_t s = (hipStream_t) stream;
#define DL_FCL(TT, LG)                                                                                                  \
    forward_chain_lower_t<TT, LG>(x_lower, a_lower, b_lower, w_lower, probs_lower, verts, neuron, flip, steps, w, y, probs, \
                                  batch, s)
    if (probs) {
        switch (dtype) {
        case DL_F16: return DL_FCL(__half, true);
        case DL_F32: return DL_FCL(float, true);
        default: return DL_FCL(double, true);
        }
    }
    switch (dtype) {
    case DL_F16: return DL_FCL(__half, false);
    case DL_F32: return DL_FCL(float, false);
    default: return DL_FCL(double, false);
    }
#undef DL_FCL
}

extern "C" int dl_logic_backward_w_chained(const void *x, const int32_t *verts, const int32_t *neuron,
                                           const uint8_t *flip, int64_t steps, const void *grad_y, const void *probs,
                                           void *grad_w, int64_t in_dim, int64_t out_dim, int64_t batch, int dtype,
                                           void *stream) {
    const bool w32 = weights_fp32(dtype);
    if (dtype != DL_F16 && dtype != DL_F32 && dtype != DL_F64) return DL_ERR_DTYPE;
    if (in_dim < 0 || out_dim < 0 || batch <= 0 || steps < out_dim || steps % DL_TRAIN_CHUNK != 0)
        return DL_ERR_INVALID_ARGUMENT;
    if (out_dim == 0) return DL_OK;
    if (!x || !verts || !neuron || !flip || !grad_y || !grad_w || in_dim == 0) return DL_ERR_INVALID_ARGUMENT;
    hipStream_t s = (hipStream_t) stream;
    switch (dtype) {
    case DL_F16: return backward_w_chain_t<__half>(x, verts, neuron, flip, steps, grad_y, probs, grad_w, batch, s, 0, w32);
    case DL_F32: return backward_w_chain_t<float>(x, verts, neuron, flip, steps, grad_y, probs, grad_w, batch, s);
    default: return backward_w_chain_t<double>(x, verts, neuron, flip, steps, grad_y, probs, grad_w, batch, s, 0, w32);
    }
}

extern "C" int dl_logic_forward(const void *x, const int64_t *a, const int64_t *b, const void *w, void *y,
                                int64_t in_dim, int64_t out_dim, int64_t batch, int dtype, void *stream) {
    const bool w32 = weights_fp32(dtype);
    if (dtype != DL_F16 && dtype != DL_F32 && dtype != DL_F64) return DL_ERR_DTYPE;
    if (in_dim < 0 || out_dim < 0 || batch < 0) return DL_ERR_INVALID_ARGUMENT;
    if (out_dim == 0 || batch == 0) return DL_OK;
    if (!x || !a || !b || !w || !y || in_dim == 0) return DL_ERR_INVALID_ARGUMENT;
    hipStream_t s = (hipStream_t) stream;
    switch (dtype) {
    case DL_F16: return forward_t<__half, false>(x, a, b, w, y, nullptr, out_dim, batch, s, w32);
    case DL_F32: return forward_t<float, false>(x, a, b, w, y, nullptr, out_dim, batch, s);
    default: return forward_t<double, false>(x, a, b, w, y, nullptr, out_dim, batch, s, w32);
    }
}

extern "C" int dl_logic_forward_logits(const void *x, const int64_t *a, const int64_t *b, const void *logits, void *y,
                                       void *probs, int64_t in_dim, int64_t out_dim, int64_t batch, int dtype,
                                       void *stream) {
    const bool w32 = weights_fp32(dtype);
    if (dtype != DL_F16 && dtype != DL_F32 && dtype != DL_F64) return DL_ERR_DTYPE;
    if (in_dim < 0 || out_dim < 0 || batch <= 0) return DL_ERR_INVALID_ARGUMENT;   // probs are written by column tile 0
    if (out_dim == 0) return DL_OK;
    if (!x || !a || !b || !logits || !y || !probs || in_dim == 0) return DL_ERR_INVALID_ARGUMENT;
    hipStream_t s = (hipStream_t) stream;
    switch (dtype) {
    case DL_F16: return forward_t<__half, true>(x, a, b, logits, y, probs, out_dim, batch, s, w32);
    case DL_F32: return forward_t<float, true>(x, a, b, logits, y, probs, out_dim, batch, s);
    default: return forward_t<double, true>(x, a, b, logits, y, probs, out_dim, batch, s, w32);
    }
}

extern "C" int dl_logic_backward_w(const void *x, const int64_t *a, const int64_t *b, const void *grad_y,
                                   void *grad_w, int64_t in_dim, int64_t out_dim, int64_t batch, int dtype,
                                   void *stream) {
    const bool w32 = weights_fp32(dtype);
    if (dtype != DL_F16 && dtype != DL_F32 && dtype != DL_F64) return DL_ERR_DTYPE;
    if (in_dim < 0 || out_dim < 0 || batch < 0) return DL_ERR_INVALID_ARGUMENT;
    if (out_dim == 0) return DL_OK;
    if (!a || !b || !grad_w || in_dim == 0) return DL_ERR_INVALID_ARGUMENT;
    if (batch > 0 && (!x || !grad_y)) return DL_ERR_INVALID_ARGUMENT;
    hipStream_t s = (hipStream_t) stream;
    switch (dtype) {
    case DL_F16: return backward_w_t<__half>(x, a, b, grad_y, nullptr, grad_w, out_dim, batch, s, 0, w32);
    case DL_F32: return backward_w_t<float>(x, a, b, grad_y, nullptr, grad_w, out_dim, batch, s);
    default: return backward_w_t<double>(x, a, b, grad_y, nullptr, grad_w, out_dim, batch, s, 0, w32);
    }
}

extern "C" int dl_logic_backward_logits(const void *x, const int64_t *a, const int64_t *b, const void *grad_y,
                                        const void *probs, void *grad_logits, int64_t in_dim, int64_t out_dim,
                                        int64_t batch, int dtype, void *stream) {
    const bool w32 = weights_fp32(dtype);
    if (dtype != DL_F16 && dtype != DL_F32 && dtype != DL_F64) return DL_ERR_DTYPE;
    if (in_dim < 0 || out_dim < 0 || batch < 0) return DL_ERR_INVALID_ARGUMENT;
    if (out_dim == 0) return DL_OK;
    if (!a || !b || !probs || !grad_logits || in_dim == 0) return DL_ERR_INVALID_ARGUMENT;
    if (batch > 0 && (!x || !grad_y)) return DL_ERR_INVALID_ARGUMENT;
    hipStream_t s = (hipStream_t) stream;
    switch (dtype) {
    case DL_F16: return backward_w_t<__half>(x, a, b, grad_y, probs, grad_logits, out_dim, batch, s, 0, w32);
    case DL_F32: return backward_w_t<float>(x, a, b, grad_y, probs, grad_logits, out_dim, batch, s);
    default: return backward_w_t<double>(x, a, b, grad_y, probs, grad_logits, out_dim, batch, s, 0, w32);
    }
}

extern "C" int dl_logic_backward_x(const void *x, const int64_t *a, const int64_t *b, const void *w,
                                   const void *grad_y, const int64_t *start, const int64_t *idx, void *grad_x,
                                   int64_t in_dim, int64_t out_dim, int64_t batch, double scale, int dtype,
                                   void *stream) {
    const bool w32 = weights_fp32(dtype);
    if (dtype != DL_F16 && dtype != DL_F32 && dtype != DL_F64) return DL_ERR_DTYPE;
    if (in_dim < 0 || out_dim < 0 || batch < 0) return DL_ERR_INVALID_ARGUMENT;
    if (in_dim == 0 || batch == 0) return DL_OK;
    if (!x || !grad_x || !start) return DL_ERR_INVALID_ARGUMENT;
    if (out_dim > 0 && (!a || !b || !w || !grad_y || !idx)) return DL_ERR_INVALID_ARGUMENT;
    hipStream_t s = (hipStream_t) stream;
    switch (dtype) {
    case DL_F16: return backward_x_t<__half>(x, a, b, w, grad_y, start, idx, grad_x, in_dim, batch, scale, s, 0, w32);
    case DL_F32: return backward_x_t<float>(x, a, b, w, grad_y, start, idx, grad_x, in_dim, batch, scale, s);
    default: return backward_x_t<double>(x, a, b, w, grad_y, start, idx, grad_x, in_dim, batch, scale, s, 0, w32);
    }
}

extern "C" int64_t dl_group_sum_workspace_bytes(int64_t out_dim, int64_t batch, int64_t k, int dtype) {
    if (out_dim < 0 || batch < 0 || k <= 0 || out_dim % k != 0) return 0;
    const int64_t elem = dtype == DL_F64 ? 8 : 4;
    return (int64_t) group_sum_splits(out_dim, batch, k) * k * batch * elem;
}

extern "C" int dl_group_sum_forward(const void *x, void *y, void *workspace, int64_t out_dim, int64_t batch, int64_t k,
                                    double tau, int dtype, void *stream) {
    if (dtype != DL_F16 && dtype != DL_F32 && dtype != DL_F64) return DL_ERR_DTYPE;
    if (out_dim < 0 || batch < 0 || k <= 0 || tau == 0.0) return DL_ERR_INVALID_ARGUMENT;
    if (out_dim % k != 0) return DL_ERR_NOT_DIVISIBLE;
    if (batch == 0) return DL_OK;
    if (!y || !workspace || (out_dim > 0 && !x)) return DL_ERR_INVALID_ARGUMENT;
    hipStream_t s = (hipStream_t) stream;
    const int splits = group_sum_splits(out_dim, batch, k);
    switch (dtype) {
    case DL_F16: return group_sum_forward_t<__half>(x, y, workspace, out_dim, batch, k, splits, tau, s);
    case DL_F32: return group_sum_forward_t<float>(x, y, workspace, out_dim, batch, k, splits, tau, s);
    default: return group_sum_forward_t<double>(x, y, workspace, out_dim, batch, k, splits, tau, s);
    }
}

extern "C" int dl_group_sum_backward(const void *grad_y, void *grad_x, int64_t out_dim, int64_t batch, int64_t k,
                                     double tau, int dtype, void *stream) {
    if (dtype != DL_F16 && dtype != DL_F32 && dtype != DL_F64) return DL_ERR_DTYPE;
    if (out_dim < 0 || batch < 0 || k <= 0 || tau == 0.0) return DL_ERR_INVALID_ARGUMENT;
    if (out_dim % k != 0) return DL_ERR_NOT_DIVISIBLE;
    if (batch == 0 || out_dim == 0) return DL_OK;
    if (!grad_y || !grad_x) return DL_ERR_INVALID_ARGUMENT;
    hipStream_t s = (hipStream_t) stream;
    switch (dtype) {
    case DL_F16: return group_sum_backward_t<__half>(grad_y, grad_x, out_dim, batch, k, tau, s);
    case DL_F32: return group_sum_backward_t<float>(grad_y, grad_x, out_dim, batch, k, tau, s);
    default: return group_sum_backward_t<double>(grad_y, grad_x, out_dim, batch, k, tau, s);
    }
}

// ---- the last LogicLayer fused with GroupSum (training mode) --------------------------------

extern "C" int dl_logic_forward_group_sum(const void *x, const int64_t *a, const int64_t *b, const void *w, void *probs,
                                          void *y, void *workspace, int64_t in_dim, int64_t out_dim, int64_t batch,
                                          int64_t k, double tau, int dtype, void *stream) {
    if (dtype != DL_F16 && dtype != DL_F32 && dtype != DL_F64) return DL_ERR_DTYPE;
    if (in_dim <= 0 || out_dim <= 0 || batch <= 0 || k <= 0 || !(tau != 0.0)) return DL_ERR_INVALID_ARGUMENT;
    if (out_dim % k != 0) return DL_ERR_NOT_DIVISIBLE;
    if (!x || !a || !b || !w || !y || !workspace) return DL_ERR_INVALID_ARGUMENT;
    hipStream_t s = (hipStream_t) stream;
    switch (dtype) {
    case DL_F16: return forward_group_sum_t<__half>(x, a, b, w, probs, y, workspace, out_dim, batch, k, tau, s);
    case DL_F32: return forward_group_sum_t<float>(x, a, b, w, probs, y, workspace, out_dim, batch, k, tau, s);
    default: return forward_group_sum_t<double>(x, a, b, w, probs, y, workspace, out_dim, batch, k, tau, s);
    }
}

static int grouped_args(int64_t in_dim, int64_t out_dim, int64_t batch, int64_t k, int dtype) {
    if (dtype != DL_F16 && dtype != DL_F32 && dtype != DL_F64) return DL_ERR_DTYPE;
    if (in_dim <= 0 || out_dim <= 0 || batch <= 0 || k <= 0) return DL_ERR_INVALID_ARGUMENT;
    if (out_dim % k != 0) return DL_ERR_NOT_DIVISIBLE;
    if (out_dim > 0xffffffffLL) return DL_ERR_TOO_LARGE;          // class of a neuron by 32-bit division
    return DL_OK;
}

extern "C" int dl_logic_backward_logits_grouped(const void *x, const int64_t *a, const int64_t *b, const void *grad_cls,
                                                const void *probs, void *grad_w, int64_t in_dim, int64_t out_dim,
                                                int64_t batch, int64_t k, int dtype, void *stream) {
    const int st = grouped_args(in_dim, out_dim, batch, k, dtype);
    if (st != DL_OK) return st;
    if (!x || !a || !b || !grad_cls || !grad_w) return DL_ERR_INVALID_ARGUMENT;
    hipStream_t s = (hipStream_t) stream;
    const int64_t per_class = out_dim / k;
    switch (dtype) {
    case DL_F16: return backward_w_t<__half>(x, a, b, grad_cls, probs, grad_w, out_dim, batch, s, per_class);
    case DL_F32: return backward_w_t<float>(x, a, b, grad_cls, probs, grad_w, out_dim, batch, s, per_class);
    default: return backward_w_t<double>(x, a, b, grad_cls, probs, grad_w, out_dim, batch, s, per_class);
    }
}

extern "C" int dl_logic_backward_x_grouped(const void *x, const int64_t *a, const int64_t *b, const void *w,
                                           const void *grad_cls, const int64_t *start, const int64_t *idx, void *grad_x,
                                           int64_t in_dim, int64_t out_dim, int64_t batch, int64_t k, double scale,
                                           int dtype, void *stream) {
    const int st = grouped_args(in_dim, out_dim, batch, k, dtype);
    if (st != DL_OK) return st;
    if (!x || !a || !b || !w || !grad_cls || !start || !idx || !grad_x) return DL_ERR_INVALID_ARGUMENT;
    hipStream_t s = (hipStream_t) stream;
    const int64_t per_class = out_dim / k;
    switch (dtype) {
    case DL_F16: return backward_x_t<__half>(x, a, b, w, grad_cls, start, idx, grad_x, in_dim, batch, scale, s, per_class);
    case DL_F32: return backward_x_t<float>(x, a, b, w, grad_cls, start, idx, grad_x, in_dim, batch, scale, s, per_class);
    default: return backward_x_t<double>(x, a, b, w, grad_cls, start, idx, grad_x, in_dim, batch, scale, s, per_class);
    }
}

extern "C" int dl_logic_backward_chained_grouped(const void *x, const int32_t *verts, const int32_t *neuron,
                                                 const uint8_t *flip, const int32_t *dst, int64_t steps, const void *w,
                                                 const void *grad_cls, int softmax_backward, const int32_t *fix_vertex,
                                                 const int32_t *fix_start, int64_t n_fix, int64_t overflow_rows,
                                                 void *grad_w, void *grad_x, void *workspace, int64_t in_dim,
                                                 int64_t out_dim, int64_t batch, int64_t k, double scale, int dtype,
                                                 void *stream) {
    const int st = grouped_args(in_dim, out_dim, batch, k, dtype);
    if (st != DL_OK) return st;
    if (steps < out_dim || n_fix < 0 || n_fix > in_dim || overflow_rows < 0) return DL_ERR_INVALID_ARGUMENT;
    if (!x || !verts || !neuron || !flip || !dst || !w || !grad_cls || !grad_w || !grad_x) return DL_ERR_INVALID_ARGUMENT;
    if (n_fix > 0 && (!fix_vertex || !fix_start)) return DL_ERR_INVALID_ARGUMENT;
    hipStream_t s = (hipStream_t) stream;
    const bool sb = softmax_backward != 0;
    const int64_t per_class = out_dim / k;
    switch (dtype) {
    case DL_F16:
        return backward_chain_t<__half>(x, verts, neuron, flip, dst, steps, w, grad_cls, sb, fix_vertex, fix_start, n_fix,
                                        overflow_rows, grad_w, grad_x, workspace, in_dim, out_dim, batch, scale, s, per_class);
    case DL_F32:
        return backward_chain_t<float>(x, verts, neuron, flip, dst, steps, w, grad_cls, sb, fix_vertex, fix_start, n_fix,
                                       overflow_rows, grad_w, grad_x, workspace, in_dim, out_dim, batch, scale, s, per_class);
    default:
        return backward_chain_t<double>(x, verts, neuron, flip, dst, steps, w, grad_cls, sb, fix_vertex, fix_start, n_fix,
                                        overflow_rows, grad_w, grad_x, workspace, in_dim, out_dim, batch, scale, s, per_class);
    }
}

extern "C" int dl_version(void) { return 100; }

extern "C" const char *dl_status_string(int status) {
    switch (status) {
    case DL_OK: return "ok";
    case DL_ERR_INVALID_ARGUMENT: return "invalid argument (null pointer, negative size or misaligned buffer)";
    case DL_ERR_BIT_COUNT: return "`bit_count` has to be in { 8, 16, 32, 64 }";
    case DL_ERR_NOT_DIVISIBLE: return "in_dim has to be divisible by k";
    case DL_ERR_DTYPE: return "dtype has to be DL_F16, DL_F32 or DL_F64";
    case DL_ERR_LAUNCH: return "HIP refused the kernel launch";
    case DL_ERR_TOO_LARGE: return "size exceeds what this entry point supports";
    case DL_ERR_SCRATCH_LIMIT: return "the call needs more than the library's static scratch array (DL_STATIC_SCRATCH_BYTES)";
    case DL_ERR_CAPTURING: return "the first call on a device must be made outside a graph capture";
    default: return "unknown status";
    }
}

// ---- Adam over all of a model's weight tensors in one launch ---------------------------------
// Elementwise and bound by its 7 float streams (p, g, m, v read; p, m, v written).  The tensors'
// pointers and sizes travel in the kernel arguments; a block takes DL_ADAM_BLOCK_ELEMS consecutive
// elements of one tensor, found through the running block counts.  The step count lives on the
// device so that a captured launch advances it on every replay; a one-thread kernel advances it and
// derives the two bias-correction factors before the update runs.
#define DL_ADAM_MAX_TENSORS 48
#define DL_ADAM_BLOCK_ELEMS 4096

namespace {

struct AdamTensors {
    float *p[DL_ADAM_MAX_TENSORS];
    const float *g[DL_ADAM_MAX_TENSORS];
    float *m[DL_ADAM_MAX_TENSORS];
    float *v[DL_ADAM_MAX_TENSORS];
    int64_t numel[DL_ADAM_MAX_TENSORS];
    uint32_t first_block[DL_ADAM_MAX_TENSORS + 1];       // running sum of ceil(numel / DL_ADAM_BLOCK_ELEMS)
    int count;
};

// state[0]: updates done; state[1], state[2]: lr / (1 - beta1^step) and 1 / sqrt(1 - beta2^step) of the update
// under way, in double arithmetic (1 - 0.999^s cancels badly in float for small s)
__global__ void adam_advance_kernel(float *state, double lr, double beta1, double beta2) {
    const double s = (double) state[0] + 1.0;
    state[0] = (float) s;
    state[1] = (float) (lr / (1.0 - pow(beta1, s)));
    state[2] = (float) (1.0 / sqrt(1.0 - pow(beta2, s)));
}

__global__ __launch_bounds__(DL_BLOCK) void adam_kernel(AdamTensors t, const float *__restrict__ state, float beta2,
                                                        float one_minus_beta1, float one_minus_beta2, float eps,
                                                        float weight_decay) {
    // which tensor: scalar search over at most 48 entries
    int ti = 0;
    while (ti + 1 < t.count && blockIdx.x >= t.first_block[ti + 1]) ++ti;
    const int64_t base = (int64_t) (blockIdx.x - t.first_block[ti]) * DL_ADAM_BLOCK_ELEMS;
    const int64_t n = t.numel[ti];
    float *__restrict__ p = t.p[ti];
    const float *__restrict__ g = t.g[ti];
    float *__restrict__ m = t.m[ti];
    float *__restrict__ v = t.v[ti];

    const float step_size = state[1], inv_bc2_sqrt = state[2];

    auto update = [&](float &pi, float gi, float &mi, float &vi) {
        if (weight_decay != 0.0f) gi = fmaf(weight_decay, pi, gi);
        mi = fmaf(gi - mi, one_minus_beta1, mi);
        vi = fmaf(beta2, vi, one_minus_beta2 * gi * gi);
        pi -= step_size * mi / (sqrtf(vi) * inv_bc2_sqrt + eps);
    };
    const bool vec = ((reinterpret_cast<uintptr_t>(p) | reinterpret_cast<uintptr_t>(g) | reinterpret_cast<uintptr_t>(m) |
                       reinterpret_cast<uintptr_t>(v)) & 15) == 0;
#pragma unroll
    for (int r = 0; r < DL_ADAM_BLOCK_ELEMS / (4 * DL_BLOCK); ++r) {
        const int64_t i = base + ((int64_t) r * DL_BLOCK + threadIdx.x) * 4;
        if (i >= n) break;
        if (vec && i + 4 <= n) {
            float4 pv = *reinterpret_cast<const float4 *>(p + i), gv = *reinterpret_cast<const float4 *>(g + i);
            float4 mv = *reinterpret_cast<const float4 *>(m + i), vv = *reinterpret_cast<const float4 *>(v + i);
            update(pv.x, gv.x, mv.x, vv.x);
            update(pv.y, gv.y, mv.y, vv.y);
            update(pv.z, gv.z, mv.z, vv.z);
            update(pv.w, gv.w, mv.w, vv.w);
            *reinterpret_cast<float4 *>(p + i) = pv;
            *reinterpret_cast<float4 *>(m + i) = mv;
            *reinterpret_cast<float4 *>(v + i) = vv;
        } else {
            for (int64_t j = i; j < i + 4 && j < n; ++j) update(p[j], g[j], m[j], v[j]);
        }
    }
}

}  // namespace

extern "C" int dl_adam_max_tensors(void) { return DL_ADAM_MAX_TENSORS; }

extern "C" int dl_adam_step(int count, float *const *p, const float *const *g, float *const *m, float *const *v,
                            const int64_t *numel, float *state, double lr, double beta1, double beta2, double eps,
                            double weight_decay, void *stream) {
    if (count < 0 || !(lr >= 0.0) || !(beta1 >= 0.0 && beta1 < 1.0) || !(beta2 >= 0.0 && beta2 < 1.0) || !(eps >= 0.0) ||
        !(weight_decay >= 0.0))
        return DL_ERR_INVALID_ARGUMENT;
    if (count > DL_ADAM_MAX_TENSORS) return DL_ERR_TOO_LARGE;
    if (count == 0) return DL_OK;
    if (!p || !g || !m || !v || !numel || !state) return DL_ERR_INVALID_ARGUMENT;
    AdamTensors t;
    uint64_t blocks = 0;
    t.count = 0;
    for (int i = 0; i < count; ++i) {
        if (numel[i] < 0) return DL_ERR_INVALID_ARGUMENT;
        if (numel[i] == 0) continue;
        if (!p[i] || !g[i] || !m[i] || !v[i]) return DL_ERR_INVALID_ARGUMENT;
        const int k = t.count++;
        t.p[k] = p[i], t.g[k] = g[i], t.m[k] = m[i], t.v[k] = v[i], t.numel[k] = numel[i];
        t.first_block[k] = (uint32_t) blocks;
        blocks += (uint64_t) dl_ceil_div(numel[i], DL_ADAM_BLOCK_ELEMS);
        if (blocks > 0x7fffffffULL) return DL_ERR_TOO_LARGE;
    }
    hipStream_t s = (hipStream_t) stream;
    DL_LAUNCH(adam_advance_kernel, dim3(1), dim3(1), 0, s, state, lr, beta1, beta2);
    if (t.count > 0) {
        t.first_block[t.count] = (uint32_t) blocks;
        DL_LAUNCH(adam_kernel, dim3((unsigned) blocks), dim3(DL_BLOCK), 0, s, t, (const float *) state, (float) beta2,
                  (float) (1.0 - beta1), (float) (1.0 - beta2), (float) eps, (float) weight_decay);
    }
    return dl_launch_status();
}
