// Packed-bit inference kernels for gfx950: gate evaluation on bit-packed words, bool -> word
// packing, and the per-class vertical bit count.
//
// All three treat a packed matrix as rows of BYTES: with little-endian words, sample s of a
// row is bit (s % 8) of byte (s / 8) whatever the word width, so one code path serves the
// 8/16/32/64-bit word types and the widest vector access the row length allows is used.
#include <hip/hip_fp16.h>

#include "dl_common.h"

#include <mutex>

#include "count_chain.h"

namespace {

// ------------------------------------------------------------------------------------------
// Gate evaluation.  Gate id = 4-bit truth table (f(0,0) f(0,1) f(1,0) f(1,1)), MSB first.
// Branch-free: two levels of bitwise select driven by b then a, with the four table bits
// expanded to all-ones / all-zero masks (wave-uniform, they live in scalar registers).
// ------------------------------------------------------------------------------------------

struct GateMasks { uint32_t m00, m01, m10, m11; };

__device__ __forceinline__ GateMasks gate_masks(uint32_t op) {
    GateMasks m;
    m.m00 = 0u - ((op >> 3) & 1u);
    m.m01 = 0u - ((op >> 2) & 1u);
    m.m10 = 0u - ((op >> 1) & 1u);
    m.m11 = 0u - (op & 1u);
    return m;
}

// What stands in for an operand that no gate looks at: whatever the registers hold (an empty statement that the
// compiler takes to define them), so that nothing is executed to make a value up.  Not for a place where loads
// into the same registers may still be in flight: the compiler then waits for them before the statement.
// The language promises nothing about an output-only empty asm; what it relies on is that the value is never looked
// at by a gate (the records' liveness marks see to that) and that the compiler neither reads nor reorders around
// it in a way that changes results.  The guard is empirical: the bit-exact comparisons with the per-layer kernels
// and the CPU oracle at full size, for every gate mix (tests/test_gpu_fullsize.py, tests/test_gpu_gate_mixes.py),
// which a build with another compiler has to pass before its numbers mean anything.
template <typename V> __device__ __forceinline__ V any_value() {
    if constexpr (sizeof(V) < 4) {
        uint32_t v;
        asm volatile("" : "=v"(v));
        return (V) v;
    } else {
        V v;
        asm volatile("" : "=v"(v));
        return v;
    }
}

template <typename V> struct Splat;
template <> struct Splat<dl_u32x4> { static __device__ __forceinline__ dl_u32x4 of(uint32_t v) { return dl_u32x4{v, v, v, v}; } };
template <> struct Splat<dl_u32x2> { static __device__ __forceinline__ dl_u32x2 of(uint32_t v) { return dl_u32x2{v, v}; } };
template <> struct Splat<uint64_t> {
    static __device__ __forceinline__ uint64_t of(uint32_t v) { return ((uint64_t) v << 32) | v; }
};
template <> struct Splat<uint32_t> { static __device__ __forceinline__ uint32_t of(uint32_t v) { return v; } };
template <> struct Splat<uint16_t> { static __device__ __forceinline__ uint16_t of(uint32_t v) { return (uint16_t) v; } };
template <> struct Splat<uint8_t> { static __device__ __forceinline__ uint8_t of(uint32_t v) { return (uint8_t) v; } };

template <typename V> __device__ __forceinline__ V gate_apply(V a, V b, const GateMasks &m) {
    const V hi = (b & Splat<V>::of(m.m11)) | (~b & Splat<V>::of(m.m10));  // value if a = 1
    const V lo = (b & Splat<V>::of(m.m01)) | (~b & Splat<V>::of(m.m00));  // value if a = 0
    return (V) ((a & hi) | (~a & lo));
}

// Inputs a gate does not look at.  A gate id is the truth table (f(0,0) f(0,1) f(1,0) f(1,1)), MSB first; six of
// the sixteen ignore an input (constants, a, b, not a, not b).  Whatever feeds an ignored input cannot change the
// result, so the kernels that evaluate trees of gates per output do not fetch it: with uniformly drawn gates a
// leaf three gates below its root is needed with probability 0.75^3.
__host__ __device__ __forceinline__ bool gate_uses_a(uint32_t op) {
    return (((op >> 3) ^ (op >> 1)) & 1u) || (((op >> 2) ^ op) & 1u);
}
__host__ __device__ __forceinline__ bool gate_uses_b(uint32_t op) {
    return (((op >> 3) ^ (op >> 2)) & 1u) || (((op >> 1) ^ op) & 1u);
}

// Bit g set: leaf g of a depth-D subtree reaches its root (gates packed as TreeFold reads them).
template <int D> struct LiveLeaves {
    static __host__ __device__ __forceinline__ uint32_t of(uint64_t gates) {
        constexpr int half = 1 << (D - 1);
        const uint32_t top = (uint32_t) (gates >> (4 * (2 * half - 2))) & 15u;
        const uint32_t left = gate_uses_a(top) ? LiveLeaves<D - 1>::of(gates) : 0u;
        const uint32_t right = gate_uses_b(top) ? LiveLeaves<D - 1>::of(gates >> (4 * (half - 1))) : 0u;
        return left | (right << half);
    }
};
template <> struct LiveLeaves<0> {
    static __host__ __device__ __forceinline__ uint32_t of(uint64_t) { return 1u; }
};


// One wave owns NPW neurons x 64 consecutive vectors of the row; a workgroup owns
// 4 * NPW * ITERS consecutive neurons.  blockIdx.x walks neuron tiles, blockIdx.y column
// tiles: workgroups are dispatched x-fastest, so the chip sweeps all neurons of one column
// tile before the next and the input rows of that tile (in_dim * 64 * sizeof(V) bytes) are
// what has to stay cache-resident between a row's uses.
template <typename V, int NPW, int ITERS>
__global__ __launch_bounds__(DL_BLOCK) void eval_kernel(const V *__restrict__ x, const int64_t *__restrict__ a,
                                                        const int64_t *__restrict__ b,
                                                        const uint8_t *__restrict__ w, V *__restrict__ y,
                                                        int64_t out_dim, int64_t ncols) {
    const int wave = dl_wave_in_block();
    const int lane = dl_lane();
    const int64_t n_first = ((int64_t) blockIdx.x * 4 + wave) * (NPW * ITERS);

    for (int64_t ct = blockIdx.y; ct * DL_WAVE < ncols; ct += gridDim.y) {
        const int64_t col = ct * DL_WAVE + lane;
        const bool live = col < ncols;
#pragma unroll 1
        for (int it = 0; it < ITERS; ++it) {
            const int64_t n0 = n_first + (int64_t) it * NPW;
            if (n0 >= out_dim) break;
            int64_t ia[NPW], ib[NPW];
            uint32_t op[NPW];
#pragma unroll
            for (int j = 0; j < NPW; ++j) {
                const int64_t n = (n0 + j < out_dim) ? n0 + j : out_dim - 1;
                ia[j] = a[n];
                ib[j] = b[n];
                op[j] = w[n];
            }
            if (live) {
                V va[NPW], vb[NPW];
#pragma unroll
                for (int j = 0; j < NPW; ++j) {                  // (wave-uniform) a row the gate does not look at is not fetched
                    va[j] = gate_uses_a(op[j]) ? x[ia[j] * ncols + col] : V{};
                    vb[j] = gate_uses_b(op[j]) ? x[ib[j] * ncols + col] : V{};
                }
#pragma unroll
                for (int j = 0; j < NPW; ++j) {
                    if (n0 + j < out_dim) {
                        const V r = gate_apply<V>(va[j], vb[j], gate_masks(op[j]));
                        __builtin_nontemporal_store(r, &y[(n0 + j) * ncols + col]);
                    }
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
// Fused evaluation of D consecutive layers.  Output neuron n of the group's last layer is a
// depth-D binary tree of gates over 2^D rows of the group's input.  A small kernel flattens the
// D wiring tables into per-neuron composites (2^D int32 row ids + the 2^D - 1 gate ids packed
// 4 bits each), and the evaluation kernel gathers the leaves and folds the tree in registers:
// the D - 1 intermediate activations never exist in memory.  Bit-identical to D calls of the
// single-layer kernel.
//
// Packing of the gate ids follows the fold order: for a subtree of depth d at bit offset `off`
// the left child's subtree sits at off, the right child's at off + 4*(2^(d-1) - 1), and the
// subtree's own gate at off + 4*(2^d - 2).  Leaves are in left-to-right order (`a` before `b`).
// ------------------------------------------------------------------------------------------
#define DL_MAX_FUSE_DEPTH 4

struct TreeTables {
    const int64_t *a[DL_MAX_FUSE_DEPTH];   // [0] = first (lowest) layer of the group
    const int64_t *b[DL_MAX_FUSE_DEPTH];
    const uint8_t *w[DL_MAX_FUSE_DEPTH];
};

template <int D>
__global__ __launch_bounds__(DL_BLOCK) void compose_tree_kernel(TreeTables t, const int32_t *__restrict__ order,
                                                                int32_t *__restrict__ leaves,
                                                                uint64_t *__restrict__ gates, int64_t out_dim) {
    const int64_t n = (int64_t) blockIdx.x * DL_BLOCK + threadIdx.x;
    if (n >= out_dim) return;
    int64_t nodes[1 << D];
    nodes[0] = order ? (int64_t) order[n] : n;        // slot n of the composites describes this neuron
    uint64_t packed = 0;
#pragma unroll
    for (int r = 0; r < D; ++r) {                  // r = distance from the root; layer index D-1-r
        const int layer = D - 1 - r;
        int64_t next[1 << D];
#pragma unroll
        for (int i = 0; i < (1 << r); ++i) {
            const int64_t node = nodes[i];
            next[2 * i] = t.a[layer][node];
            next[2 * i + 1] = t.b[layer][node];
            int off = 0, d = D;                    // bit slot of node (r, i)
#pragma unroll
            for (int kbit = r - 1; kbit >= 0; --kbit) {
                off += ((i >> kbit) & 1) * ((1 << (d - 1)) - 1);
                d -= 1;
            }
            const int slot = off + 2 * ((1 << (d - 1)) - 1);
            packed |= (uint64_t) (t.w[layer][node] & 15u) << (4 * slot);
        }
#pragma unroll
        for (int i = 0; i < (2 << r); ++i) nodes[i] = next[i];
    }
    const uint32_t live = LiveLeaves<D>::of(packed);   // a row that no gate looks at is not fetched: id -1
#pragma unroll
    for (int i = 0; i < (1 << D); ++i) leaves[n * (1 << D) + i] = (live >> i) & 1u ? (int32_t) nodes[i] : -1;
    gates[n] = packed;
}

template <typename V, int D> struct TreeFold {
    static __device__ __forceinline__ V run(const V *leaf, uint64_t gates) {
        constexpr int half = 1 << (D - 1);
        const V l = TreeFold<V, D - 1>::run(leaf, gates);
        const V r = TreeFold<V, D - 1>::run(leaf + half, gates >> (4 * (half - 1)));
        return gate_apply<V>(l, r, gate_masks((uint32_t) (gates >> (4 * (2 * half - 2))) & 15u));
    }
};
template <typename V> struct TreeFold<V, 0> {
    static __device__ __forceinline__ V run(const V *leaf, uint64_t) { return leaf[0]; }
};

// Same tiling and dispatch order as eval_kernel; one wave = NPW output neurons x 64 vectors.
template <typename V, int D, int NPW, int ITERS>
__global__ __launch_bounds__(DL_BLOCK) void eval_tree_kernel(const V *__restrict__ x,
                                                             const int32_t *__restrict__ leaves,
                                                             const uint64_t *__restrict__ gates, V *__restrict__ y,
                                                             int64_t out_dim, int64_t ncols) {
    constexpr int G = 1 << D;
    const int wave = dl_wave_in_block();
    const int lane = dl_lane();
    const int64_t n_first = ((int64_t) blockIdx.x * 4 + wave) * (NPW * ITERS);

    for (int64_t ct = blockIdx.y; ct * DL_WAVE < ncols; ct += gridDim.y) {
        const int64_t col = ct * DL_WAVE + lane;
        const bool live = col < ncols;
#pragma unroll 1
        for (int it = 0; it < ITERS; ++it) {
            const int64_t n0 = n_first + (int64_t) it * NPW;
            if (n0 >= out_dim) break;
            int32_t id[NPW][G];
            uint64_t gt[NPW];
#pragma unroll
            for (int j = 0; j < NPW; ++j) {
                const int64_t n = (n0 + j < out_dim) ? n0 + j : out_dim - 1;
                gt[j] = gates[n];
#pragma unroll
                for (int g = 0; g < G; ++g) id[j][g] = leaves[n * G + g];
            }
            if (live) {
                V v[NPW][G];
#pragma unroll
                for (int j = 0; j < NPW; ++j) {
#pragma unroll
                    for (int g = 0; g < G; ++g) v[j][g] = id[j][g] < 0 ? V{} : x[(int64_t) id[j][g] * ncols + col];
                }
#pragma unroll
                for (int j = 0; j < NPW; ++j) {
                    if (n0 + j < out_dim)
                        __builtin_nontemporal_store(TreeFold<V, D>::run(v[j], gt[j]), &y[(n0 + j) * ncols + col]);
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
// Chained variant of eval_tree_kernel.  The group's top layer is walked along the trails of an
// evaluation schedule (schedule.cpp): consecutive top-layer neurons share one input, whose value
// (a depth-DS subtree over 2^DS gathered rows; DS = 0: the input row itself) stays in registers,
// so a neuron costs 2^DS gathers instead of 2^(DS+1).  One wave = CHUNK consecutive steps x 64
// vectors; the first vertex of a chunk is evaluated again (CHUNK + 1 subtrees per chunk).
// ------------------------------------------------------------------------------------------
__device__ __forceinline__ uint32_t swap_gate_inputs(uint32_t op) {   // f'(a, b) = f(b, a)
    return (op & 9u) | ((op & 4u) >> 1) | ((op & 2u) << 1);
}

template <typename V, int DS> struct Subtree {
    int32_t leaf[1 << DS];
    uint64_t gates;
    __device__ __forceinline__ void locate(int32_t vertex, const int32_t *__restrict__ sub_leaves,
                                           const uint64_t *__restrict__ sub_gates) {
        gates = sub_gates[vertex];
#pragma unroll
        for (int g = 0; g < (1 << DS); ++g) leaf[g] = sub_leaves[(int64_t) vertex * (1 << DS) + g];
    }
    __device__ __forceinline__ void gather(const V *__restrict__ xcol, int64_t ncols, V *v) const {
#pragma unroll
        for (int g = 0; g < (1 << DS); ++g) v[g] = leaf[g] < 0 ? V{} : xcol[(int64_t) leaf[g] * ncols];
    }
};
template <typename V> struct Subtree<V, 0> {
    int32_t leaf[1];
    uint64_t gates;
    __device__ __forceinline__ void locate(int32_t vertex, const int32_t *, const uint64_t *) {
        leaf[0] = vertex;
        gates = 0;
    }
    __device__ __forceinline__ void gather(const V *__restrict__ xcol, int64_t ncols, V *v) const {
        v[0] = xcol[(int64_t) leaf[0] * ncols];
    }
};

template <typename V, int DS, int CHUNK, int ITERS>
__global__ __launch_bounds__(DL_BLOCK) void eval_chain_kernel(const V *__restrict__ x,
                                                              const int32_t *__restrict__ sub_leaves,
                                                              const uint64_t *__restrict__ sub_gates,
                                                              const int32_t *__restrict__ verts,
                                                              const int32_t *__restrict__ neuron,
                                                              const uint8_t *__restrict__ flip,
                                                              const uint8_t *__restrict__ w_top, V *__restrict__ y,
                                                              int64_t nchunks, int64_t ncols) {
    constexpr int G = 1 << DS;
    static_assert(CHUNK % 2 == 0, "steps are processed in pairs");
    const int wave = dl_wave_in_block();
    const int lane = dl_lane();
    const int64_t c_first = ((int64_t) blockIdx.x * 4 + wave) * ITERS;

    for (int64_t ct = blockIdx.y; ct * DL_WAVE < ncols; ct += gridDim.y) {
        const int64_t col = ct * DL_WAVE + lane;
        if (col >= ncols) continue;
        const V *xcol = x + col;
        V *ycol = y + col;
        if (c_first >= nchunks) continue;
        // the wave's chunks follow each other in the schedule: only the first vertex of the first
        // one is evaluated on its own, after that every step's left input is the step before's right
        V prev;
        {
            Subtree<V, DS> first;
            first.locate(verts[c_first * CHUNK], sub_leaves, sub_gates);
            V leaves0[G];
            first.gather(xcol, ncols, leaves0);
            prev = TreeFold<V, DS>::run(leaves0, first.gates);
        }
#pragma unroll 1
        for (int it = 0; it < ITERS; ++it) {
            const int64_t c = c_first + it;
            if (c >= nchunks) break;
            const int64_t s0 = c * CHUNK;
#pragma unroll
            for (int j = 0; j < CHUNK; j += 2) {
                Subtree<V, DS> ta, tb;
                ta.locate(verts[s0 + j + 1], sub_leaves, sub_gates);
                tb.locate(verts[s0 + j + 2], sub_leaves, sub_gates);
                const int32_t na = neuron[s0 + j], nb = neuron[s0 + j + 1];
                uint32_t oa = w_top[na >= 0 ? na : 0], ob = w_top[nb >= 0 ? nb : 0];
                if (flip[s0 + j]) oa = swap_gate_inputs(oa);
                if (flip[s0 + j + 1]) ob = swap_gate_inputs(ob);
                V la[G], lb[G];
                ta.gather(xcol, ncols, la);
                tb.gather(xcol, ncols, lb);
                const V va = TreeFold<V, DS>::run(la, ta.gates);
                const V vb = TreeFold<V, DS>::run(lb, tb.gates);
                if (na >= 0) __builtin_nontemporal_store(gate_apply<V>(prev, va, gate_masks(oa)), ycol + (int64_t) na * ncols);
                if (nb >= 0) __builtin_nontemporal_store(gate_apply<V>(va, vb, gate_masks(ob)), ycol + (int64_t) nb * ncols);
                prev = vb;
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
// eval_chain_kernel with everything a step needs in ONE record, composed per call by a small
// kernel from the schedule, the flattened subtrees and the current gate ids:
//   rec[i + 1] for step i (rec[0]: the vertex before step 0, from which a wave starting at step 0
//   seeds its chain; a wave starting at step f seeds from rec[f]):
//     leaf[2^DS]  the subtree's rows, already multiplied by the row length in vectors
//     gates       the subtree's gate ids (4 bits each, fold order) | top gate << 28, the top gate
//                 with its inputs swapped where the schedule says so
//     out         the output row times the row length in vectors, 0xffffffff = no output
// so that a step costs one wide scalar load instead of a chain of dependent ones (vertex ->
// subtree tables, neuron -> gate id, flip), and every gather is a scalar row base plus the lane's
// constant 32-bit offset.  Applies when rows * row length and out_dim * row length fit 32 bits.
// ------------------------------------------------------------------------------------------
// Bit j set: the gate in nibble j of a depth-D subtree's packed gates feeds its root (`alive`: the root does).
template <int D> struct LiveGates {
    static __host__ __device__ __forceinline__ uint32_t of(uint64_t gates, bool alive) {
        if (!alive) return 0u;
        constexpr int half = 1 << (D - 1);
        const uint32_t top = (uint32_t) (gates >> (4 * (2 * half - 2))) & 15u;
        return (1u << (2 * half - 2)) | LiveGates<D - 1>::of(gates, gate_uses_a(top)) |
               (LiveGates<D - 1>::of(gates >> (4 * (half - 1)), gate_uses_b(top)) << (half - 1));
    }
};
template <> struct LiveGates<0> {
    static __host__ __device__ __forceinline__ uint32_t of(uint64_t, bool) { return 0u; }
};

#define DL_STEP_DEAD 0xffffffffu        // leaf of a step record that no gate looks at: not fetched

// records of subtrees with more than one gate also say which gates are worth evaluating (LiveGates)
template <int DS> struct StepLive {};
template <> struct StepLive<2> { uint32_t live; };
template <> struct StepLive<3> { uint32_t live; };

template <int DS> struct alignas(DS == 3 ? 64 : DS == 2 ? 32 : 16) StepRec : StepLive<DS> {
    uint32_t leaf[1 << DS];
    uint32_t gates;
    uint32_t out;
};

// TreeFold that leaves out the gates nobody looks at (`live` as LiveGates numbers them; wave-uniform branches)
template <typename V, int D> struct TreeFoldLive {
    static __device__ __forceinline__ V run(const V *leaf, uint32_t gates, uint32_t live) {
        constexpr int half = 1 << (D - 1);
        if (!((live >> (2 * half - 2)) & 1u)) return leaf[0];        // nobody looks at the result: any value does
        const V l = TreeFoldLive<V, D - 1>::run(leaf, gates, live);
        const V r = TreeFoldLive<V, D - 1>::run(leaf + half, gates >> (4 * (half - 1)), live >> (half - 1));
        return gate_apply<V>(l, r, gate_masks((gates >> (4 * (2 * half - 2))) & 15u));
    }
};
template <typename V> struct TreeFoldLive<V, 0> {
    static __device__ __forceinline__ V run(const V *leaf, uint32_t, uint32_t) { return leaf[0]; }
};

// the subtree value of a step record
template <typename V, int DS> __device__ __forceinline__ V fold_record(const V *leaf, const StepRec<DS> &r) {
    if constexpr (DS >= 2) return TreeFoldLive<V, DS>::run(leaf, r.gates, r.live);
    else return TreeFold<V, DS>::run(leaf, r.gates);
}
static_assert(sizeof(StepRec<3>) == 64 && sizeof(StepRec<2>) == 32 && sizeof(StepRec<1>) == 16 && sizeof(StepRec<0>) == 16,
              "records are whole scalar-load units");

template <int DS>
__global__ __launch_bounds__(DL_BLOCK) void compose_steps_kernel(const int32_t *__restrict__ sub_leaves,
                                                                 const uint64_t *__restrict__ sub_gates,
                                                                 const int32_t *__restrict__ verts,
                                                                 const int32_t *__restrict__ neuron,
                                                                 const uint8_t *__restrict__ flip,
                                                                 const uint8_t *__restrict__ w_top,
                                                                 const uint8_t *__restrict__ out_live, int64_t steps,
                                                                 uint32_t ncols, StepRec<DS> *__restrict__ rec) {
    const int64_t i = (int64_t) blockIdx.x * DL_BLOCK + threadIdx.x;      // record index: step i - 1
    if (i > steps) return;
    const int64_t v = verts[i];
    StepRec<DS> r;
    uint32_t gates = 0;
    r.out = 0xffffffffu;
    // the vertex is the second input of step i - 1's neuron and the first input of step i's
    // (out_live: output rows nobody will read are neither computed nor written)
    bool needed = false;
    if (i >= 1 && neuron[i - 1] >= 0 && (!out_live || out_live[neuron[i - 1]])) {
        const int32_t n = neuron[i - 1];
        uint32_t top = w_top[n] & 15u;
        if (flip[i - 1]) top = swap_gate_inputs(top);
        gates |= top << 28;
        r.out = (uint32_t) n * ncols;
        needed = gate_uses_b(top);
    }
    if (i < steps && neuron[i] >= 0 && (!out_live || out_live[neuron[i]])) {
        uint32_t next = w_top[neuron[i]] & 15u;
        if (flip[i]) next = swap_gate_inputs(next);
        needed = needed || gate_uses_a(next);
    }
    if (DS == 0) {
        r.leaf[0] = needed ? (uint32_t) v * ncols : DL_STEP_DEAD;
    } else {
        const uint64_t sub = sub_gates[v];
        gates |= (uint32_t) sub;
        const uint32_t live = needed ? LiveLeaves<DS>::of(sub) : 0u;
        if constexpr (DS >= 2) r.live = LiveGates<DS>::of(sub, needed);
#pragma unroll
        for (int g = 0; g < (1 << DS); ++g)
            r.leaf[g] = (live >> g) & 1u ? (uint32_t) sub_leaves[v * (1 << DS) + g] * ncols : DL_STEP_DEAD;
    }
    r.gates = gates;
    rec[i] = r;
}

// One wave = STEPS consecutive steps x 64 vectors; dispatch order as eval_kernel.  BUF: x is at
// most 4 GiB and is read through a buffer resource, whose loads take the row's byte offset as a
// scalar operand next to the lane's constant offset: no vector instruction per gather.
#ifndef DL_CC_REQUEST_PARTS
#define DL_CC_REQUEST_PARTS 2          // count_chain_kernel: a block's rows are requested in this many parts along the walk before
#endif
#ifndef DL_PACK_SHARE
#define DL_PACK_SHARE 16               // pack kernel: neighbouring workgroups (64 output bytes per row each) that share an XCD
#endif
#ifndef DL_CC_XCD_TILE_BYTES
#define DL_CC_XCD_TILE_BYTES (64 << 20)    // count_chain_kernel: input column tiles up to this size get an XCD of their own
#endif
#ifndef DL_XCD_TILE_BYTES
#define DL_XCD_TILE_BYTES (2 << 20)    // eval_steps_kernel: input column tiles up to this size get an XCD (an L2) of their own
#endif
#ifndef DL_STEPS_PER_WAVE
#define DL_STEPS_PER_WAVE 32           // steps a wave of eval_steps_kernel walks (its first vertex is evaluated on top)
#endif
template <typename V, int DS, int STEPS, bool BUF>
__global__ __launch_bounds__(DL_BLOCK) void eval_steps_kernel(const V *__restrict__ x, const StepRec<DS> *__restrict__ rec,
                                                              V *__restrict__ y, int64_t nsteps, int64_t ncols,
                                                              uint32_t x_bytes, uint32_t xcd_owns_tiles) {
    constexpr int G = 1 << DS;
    static_assert(STEPS % 2 == 0, "steps are processed in pairs");
    const int wave = dl_wave_in_block();
    const int lane = dl_lane();
    // Workgroups are dealt round-robin to the 8 XCDs, each with an L2 of its own.  xcd_owns_tiles (the grid's
    // second dimension is then a multiple of 8): XCD j takes the column tiles j, j + 8, ... one after the other, so
    // that a tile of the input is fetched into one L2 instead of eight and stays there while the tile is swept
    // (headline prefix: fetched 2.08 -> 0.97 GB per launch, 1.13 -> 1.07 ms).
    int64_t bx = blockIdx.x, by = blockIdx.y;
    if (xcd_owns_tiles) {
        const int64_t id = (int64_t) blockIdx.y * gridDim.x + blockIdx.x, xcd = id % 8, place = id / 8;
        bx = place % gridDim.x;
        by = (place / gridDim.x) * 8 + xcd;
    }
    const int64_t first = (bx * 4 + wave) * STEPS;
    if (first >= nsteps) return;
    const StepRec<DS> *wrec = rec + first;                 // [0] = seed, [1 + j] = the wave's step j

    for (int64_t ct = by; ct * DL_WAVE < ncols; ct += gridDim.y) {
        const uint32_t col = (uint32_t) (ct * DL_WAVE) + (uint32_t) lane;
        if (col >= ncols) continue;
        auto row = [&](uint32_t start) -> V {                                  // scalar row base + the lane's offset
            if constexpr (BUF && sizeof(V) == 16) {
                const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void *) x, 0, (int) x_bytes, 0x00027000);
                return __builtin_bit_cast(V, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int) (col * 16u), (int) (start * 16u), 0));
            } else {
                return (x + start)[col];
            }
        };
        V prev;
        {
            const StepRec<DS> r = wrec[0];
            V leaves0[G];
#pragma unroll
            for (int g = 0; g < G; ++g) leaves0[g] = any_value<V>();
#pragma unroll
            for (int g = 0; g < G; ++g)
                if (r.leaf[g] != DL_STEP_DEAD) leaves0[g] = row(r.leaf[g]);
            prev = fold_record<V, DS>(leaves0, r);
        }
        // NB steps at a time, so that the rows of up to 16 leaves are requested together whatever the subtrees' depth
        constexpr int NB = DS >= 3 ? 2 : DS == 2 ? 4 : 8;
        static_assert(STEPS % NB == 0 && 8 % NB == 0, "the schedule is a whole number of batches (of chunks of 8 steps)");
#pragma unroll 1
        for (int j = 0; j < STEPS; j += NB) {
            if (first + j >= nsteps) break;
            StepRec<DS> r[NB];
#pragma unroll
            for (int i = 0; i < NB; ++i) r[i] = wrec[1 + j + i];
            // a row that no gate looks at (wave-uniform marker) is not fetched, and nothing is executed in its place:
            // the registers are "defined" here, before any request of this batch of steps is in flight
            V leaf[NB][G];
#pragma unroll
            for (int i = 0; i < NB; ++i)
#pragma unroll
                for (int g = 0; g < G; ++g) leaf[i][g] = any_value<V>();
#pragma unroll
            for (int i = 0; i < NB; ++i)
#pragma unroll
                for (int g = 0; g < G; ++g)
                    if (r[i].leaf[g] != DL_STEP_DEAD) leaf[i][g] = row(r[i].leaf[g]);
#pragma unroll
            for (int i = 0; i < NB; ++i) {
                const V v = fold_record<V, DS>(leaf[i], r[i]);
                if (r[i].out != 0xffffffffu)
                    __builtin_nontemporal_store(gate_apply<V>(prev, v, gate_masks(r[i].gates >> 28)), (y + r[i].out) + col);
                prev = v;
            }
        }
    }
}

template <typename V, int NPW, int ITERS>
int launch_eval(const void *x, const int64_t *a, const int64_t *b, const uint8_t *w, void *y, int64_t out_dim,
                int64_t row_bytes, hipStream_t stream) {
    const int64_t ncols = row_bytes / (int64_t) sizeof(V);
    const int64_t ntiles = dl_ceil_div(out_dim, 4 * NPW * ITERS);
    int64_t ctiles = dl_ceil_div(ncols, DL_WAVE);
    if (ntiles > 0x7fffffffLL) return DL_ERR_TOO_LARGE;
    if (ctiles > 65535) ctiles = 65535;
    dim3 grid((unsigned) ntiles, (unsigned) ctiles);
    DL_LAUNCH((eval_kernel<V, NPW, ITERS>), grid, dim3(DL_BLOCK), 0, stream, (const V *) x, a, b, w, (V *) y,
                       out_dim, ncols);
    return dl_launch_status();
}

// ------------------------------------------------------------------------------------------
// bool -> packed bytes.  Output byte j of a row holds samples 8j .. 8j+7, lowest sample in
// bit 0; bytes past the batch are zero.
// ------------------------------------------------------------------------------------------

// 8 bool bytes (any non-zero value counts as true) -> 8 bits, byte i -> bit i.
__device__ __forceinline__ uint32_t squeeze8(uint64_t v) {
    const uint64_t k7f = 0x7f7f7f7f7f7f7f7fULL;
    v = (((v & k7f) + k7f) | v) & ~k7f;                          // 0x80 in every non-zero byte
    return (uint32_t) (((v >> 7) * 0x0102040810204080ULL) >> 56);  // gather the eight flags
}

// Rows whose length is a multiple of 16 bools and 16-byte aligned: one 16-byte load and one
// 2-byte store per lane, both coalesced.
__global__ __launch_bounds__(DL_BLOCK) void packbits_vec16_kernel(const uint8_t *__restrict__ t,
                                                                  uint8_t *__restrict__ out, int64_t features,
                                                                  int64_t batch, int64_t out_row_bytes) {
    const int64_t chunks = batch / 16;                  // 16 samples -> 2 output bytes
    const int64_t out_pairs = out_row_bytes / 2;        // out_row_bytes is even here
    for (int64_t f = blockIdx.y; f < features; f += gridDim.y) {
        const dl_u32x4 *src = reinterpret_cast<const dl_u32x4 *>(t + f * batch);
        uint16_t *dst = reinterpret_cast<uint16_t *>(out + f * out_row_bytes);
        for (int64_t i = (int64_t) blockIdx.x * DL_BLOCK + threadIdx.x; i < out_pairs;
             i += (int64_t) gridDim.x * DL_BLOCK) {
            uint32_t r = 0;
            if (i < chunks) {
                const dl_u32x4 v = __builtin_nontemporal_load(&src[i]);
                const uint64_t lo = ((uint64_t) v.y << 32) | v.x, hi = ((uint64_t) v.w << 32) | v.z;
                r = squeeze8(lo) | (squeeze8(hi) << 8);
            }
            dst[i] = (uint16_t) r;
        }
    }
}

// Any batch length: one output byte per thread from up to 8 single-byte loads.
__global__ __launch_bounds__(DL_BLOCK) void packbits_generic_kernel(const uint8_t *__restrict__ t,
                                                                    uint8_t *__restrict__ out, int64_t features,
                                                                    int64_t batch, int64_t out_row_bytes) {
    for (int64_t f = blockIdx.y; f < features; f += gridDim.y) {
        const uint8_t *src = t + f * batch;
        uint8_t *dst = out + f * out_row_bytes;
        for (int64_t j = (int64_t) blockIdx.x * DL_BLOCK + threadIdx.x; j < out_row_bytes;
             j += (int64_t) gridDim.x * DL_BLOCK) {
            uint32_t r = 0;
            const int64_t s0 = j * 8;
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (s0 + i < batch) r |= (uint32_t) (src[s0 + i] != 0) << i;
            dst[j] = (uint8_t) r;
        }
    }
}

// Batch-major input: bool [batch, features] -> packed [features, row bytes] in one pass, i.e.
// the transpose and the packing fused.  A workgroup owns 64*BPL features x 16 word columns
// (1024 samples).  Each wave reads sample rows with lanes along the features (BPL bool bytes
// per lane, coalesced), folds 8 samples into one register whose byte k carries feature k's 8
// bits, assembles 64-sample words per feature, and parks them in LDS; the workgroup then writes
// 128 contiguous bytes per feature row.
template <int BPL> struct BoolLoad;
template <> struct BoolLoad<4> {
    static __device__ __forceinline__ uint32_t flags(const uint8_t *p) {
        const uint32_t v = __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(p));
        return ((((v & 0x7f7f7f7fu) + 0x7f7f7f7fu) | v) >> 7) & 0x01010101u;   // 1 per non-zero byte
    }
};
template <> struct BoolLoad<1> {
    static __device__ __forceinline__ uint32_t flags(const uint8_t *p) { return (uint32_t) (*p != 0); }
};

template <int BPL>
__global__ __launch_bounds__(DL_BLOCK) void packbits_batch_major_kernel(const uint8_t *__restrict__ x,
                                                                        uint8_t *__restrict__ out, int64_t batch,
                                                                        int64_t features, int64_t out_row_bytes) {
    constexpr int FW = DL_WAVE * BPL;   // features per workgroup
    constexpr int WC = 16;              // 64-sample word columns per workgroup
    __shared__ uint64_t tile[FW][WC + 1];

    const int wave = dl_wave_in_block();
    const int lane = dl_lane();
    const int64_t f0 = (int64_t) blockIdx.y * FW;
    const int64_t w0 = (int64_t) blockIdx.x * WC;
    const int64_t fl = f0 + (int64_t) lane * BPL;
    const bool feat_live = fl < features;           // features % BPL == 0

#pragma unroll 1
    for (int q = 0; q < WC / 4; ++q) {
        const int wc = wave * (WC / 4) + q;
        const int64_t s0 = (w0 + wc) * 64;
        uint32_t oct[8];                            // oct[j]: byte k = feature k, samples 8j .. 8j+7
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            uint32_t acc = 0;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int64_t s = s0 + 8 * j + i;
                uint32_t n = 0;
                if (feat_live && s < batch) n = BoolLoad<BPL>::flags(x + s * features + fl);
                acc |= n << i;
            }
            oct[j] = acc;
        }
#pragma unroll
        for (int k = 0; k < BPL; ++k) {
            uint32_t lo = 0, hi = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                lo |= ((oct[j] >> (8 * k)) & 0xffu) << (8 * j);
                hi |= ((oct[4 + j] >> (8 * k)) & 0xffu) << (8 * j);
            }
            tile[lane * BPL + k][wc] = ((uint64_t) hi << 32) | lo;
        }
    }
    __syncthreads();

    // 16 consecutive threads write the 16 words (128 bytes) of one feature row.
    const int wi = (int) (threadIdx.x & 15u);
    const int64_t byte0 = (w0 + wi) * 8;
    const bool whole_words = (out_row_bytes & 7) == 0;
    for (int r = (int) (threadIdx.x >> 4); r < FW; r += DL_BLOCK / 16) {
        const int64_t f = f0 + r;
        if (f >= features || byte0 >= out_row_bytes) continue;
        const uint64_t v = tile[r][wi];
        uint8_t *dst = out + f * out_row_bytes + byte0;
        if (whole_words) {
            *reinterpret_cast<uint64_t *>(dst) = v;
        } else {
            const int nb = (int) ((out_row_bytes - byte0 < 8) ? (out_row_bytes - byte0) : 8);
            for (int t = 0; t < nb; ++t) dst[t] = (uint8_t) (v >> (8 * t));
        }
    }
}

// Variant for features % 16 == 0 that stages nothing on the way in: a workgroup owns WC word columns
// (64 * WC consecutive samples, i.e. one contiguous region of the input) and a slice of the features.
// A thread takes 16 features x 8 samples at a time: eight 16-byte loads (a wave's loads of one sample
// row are contiguous), folded in registers into the 16 features' bytes for those 8 samples, which it
// drops into an LDS tile of output words; the workgroup then writes 8 * WC contiguous bytes per feature
// row.  The tile is laid out [feature % 16][feature / 16][WC words + 4 bytes] so that the lanes of a
// wave (consecutive 16-feature chunks) fall 17 dwords apart, on distinct banks.
#define DL_PACK_WC 8
#define DL_PACK_PITCH (DL_PACK_WC * 8 + 4)
#define DL_PACK_MAX_SLICE 2352                   // features per workgroup: 2352 * 68 bytes of LDS

__global__ __launch_bounds__(DL_BLOCK) void packbits_batch_major_rows_kernel(const uint8_t *__restrict__ x,
                                                                             uint8_t *__restrict__ out, int64_t batch,
                                                                             int64_t features, int slice, int nslices,
                                                                             int64_t out_row_bytes, uint32_t paired_blocks) {
    extern __shared__ __align__(16) uint8_t tile[];                                  // [16][per_row][PITCH]
    // Two workgroups share every 128-byte line of the output (64 bytes each): the DL_PACK_SHARE workgroups that
    // write one kilobyte of every row stay on one of the 8 XCDs, whose L2 merges the halves and holds neighbouring
    // lines until they are written back (workgroups are dealt to the XCDs round-robin by index).  Measured: sets of
    // 16 against pairs 0.198 -> 0.192 ms on 784 features, 0.486 -> 0.470 ms on 9216.
    uint32_t blk = blockIdx.x;
    if (blk < paired_blocks) {
        const uint32_t per = DL_PACK_SHARE * (uint32_t) nslices, xcd = blk % 8, j = blk / 8;
        blk = ((j / per) * 8 + xcd) * per + j % per;
    }
    const int64_t w0 = (int64_t) (blk / (unsigned) nslices) * DL_PACK_WC;
    const int64_t f0 = (int64_t) (blk % (unsigned) nslices) * slice;
    const int fs = (int) (features - f0 < slice ? features - f0 : slice);           // this slice's features
    const int per_row = fs / 16;                                                     // 16-byte chunks per sample
    const int items = DL_PACK_WC * 8 * per_row;
    const int64_t s0 = w0 * 64;

    // item = 16 features x 8 samples: (oct, c), oct = wc * 8 + j the byte of the output row, c the 16-byte chunk
    auto request = [&](int it, dl_u32x4 *v) __attribute__((always_inline)) {
        const int oct = it / per_row, c = it - oct * per_row;
        const int64_t row0 = s0 + 8 * oct;
        const uint8_t *src = x + row0 * features + f0 + 16 * c;
#pragma unroll
        for (int i = 0; i < 8; ++i)
            v[i] = row0 + i < batch ? __builtin_nontemporal_load(reinterpret_cast<const dl_u32x4 *>(src + i * features))
                                    : dl_u32x4{0, 0, 0, 0};
    };
    auto fold = [&](int it, const dl_u32x4 *v) __attribute__((always_inline)) {
        const int oct = it / per_row, c = it - oct * per_row;
        uint8_t *dst = tile + (size_t) c * DL_PACK_PITCH + oct;
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            uint32_t acc = 0;                                                        // byte k: feature 4 d + k, 8 samples
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const uint32_t u = v[i][d];
                acc |= (((((u & 0x7f7f7f7fu) + 0x7f7f7f7fu) | u) >> 7) & 0x01010101u) << i;
            }
#pragma unroll
            for (int k = 0; k < 4; ++k)
                dst[(size_t) (4 * d + k) * per_row * DL_PACK_PITCH] = (uint8_t) (acc >> (8 * k));
        }
    };
    // a thread's next item is requested before the current one is folded, so its loads never stop
    dl_u32x4 va[8], vb[8];
    int it = threadIdx.x;
    if (it < items) request(it, va);
    for (; it < items; it += 2 * DL_BLOCK) {
        const bool second = it + DL_BLOCK < items;
        if (second) request(it + DL_BLOCK, vb);
        fold(it, va);
        if (second) {
            if (it + 2 * DL_BLOCK < items) request(it + 2 * DL_BLOCK, va);
            fold(it + DL_BLOCK, vb);
        }
    }
    __syncthreads();
    // DL_PACK_WC consecutive threads write the words of one feature row (out_row_bytes % 8 == 0 here)
    const int64_t total_words = out_row_bytes / 8;
    for (int i = threadIdx.x; i < fs * DL_PACK_WC; i += DL_BLOCK) {
        const int f = i / DL_PACK_WC, wc = i - f * DL_PACK_WC;
        const uint32_t *w = reinterpret_cast<const uint32_t *>(tile + ((size_t) (f % 16) * per_row + f / 16) * DL_PACK_PITCH) + 2 * wc;
        if (w0 + wc < total_words)
            *reinterpret_cast<uint64_t *>(out + (f0 + f) * out_row_bytes + (w0 + wc) * 8) = ((uint64_t) w[1] << 32) | w[0];
    }
}

// ------------------------------------------------------------------------------------------
// Vertical bit count (GroupSum on packed words).  For each class (a contiguous block of
// per_class neuron rows) and each sample bit, the number of rows with that bit set.
//
// Lanes run along vectors V of the rows (16 bytes = 128 samples per lane where the row length
// allows it, else 8 bytes); each wave takes a quarter of the class's rows and keeps bit-sliced
// counters per lane: 16 rows at a time are compressed by a carry-save-adder tree into planes of
// weight 1, 2, 4, 8 and a carry of weight 16 that is rippled into NPH higher planes.  The four
// waves' planes are exchanged through LDS and each wave expands a quarter of every lane's sample
// bits to integers and stores them.
//
// TREE > 0: the counted rows are not read but computed on the fly as the last TREE layers of the
// net over the rows of `bits` (= the input of those layers), from the composites that
// compose_tree_kernel writes; the output of the last layer never exists in memory.
// ------------------------------------------------------------------------------------------

// A full adder per bit: two three-input bit operations per dword (truth tables 0xe8 = majority, 0x96 = parity),
// stated as such because the compiler otherwise rearranges a chain of adders into half as many again.
template <typename V> struct FullAdd;
template <> struct FullAdd<uint32_t> {
    static __device__ __forceinline__ void run(uint32_t &carry, uint32_t &sum, uint32_t a, uint32_t b, uint32_t c) {
        carry = __builtin_amdgcn_bitop3_b32(a, b, c, 0xe8);
        sum = __builtin_amdgcn_bitop3_b32(a, b, c, 0x96);
    }
};
template <> struct FullAdd<uint64_t> {
    static __device__ __forceinline__ void run(uint64_t &carry, uint64_t &sum, uint64_t a, uint64_t b, uint64_t c) {
        uint32_t cl, sl, ch, sh;
        FullAdd<uint32_t>::run(cl, sl, (uint32_t) a, (uint32_t) b, (uint32_t) c);
        FullAdd<uint32_t>::run(ch, sh, (uint32_t) (a >> 32), (uint32_t) (b >> 32), (uint32_t) (c >> 32));
        carry = ((uint64_t) ch << 32) | cl;
        sum = ((uint64_t) sh << 32) | sl;
    }
};
template <> struct FullAdd<dl_u32x4> {
    static __device__ __forceinline__ void run(dl_u32x4 &carry, dl_u32x4 &sum, dl_u32x4 a, dl_u32x4 b, dl_u32x4 c) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t cy, sm;
            FullAdd<uint32_t>::run(cy, sm, a[i], b[i], c[i]);
            carry[i] = cy;
            sum[i] = sm;
        }
    }
};

// A half adder in place (plane += carry, carry = what leaves the plane), also stated as two bit operations so that
// a ripple through the planes stays a chain of them: rearranged into wider operations on the planes' old values it
// needs every plane twice in registers.
template <typename V> struct HalfAdd;
template <> struct HalfAdd<uint32_t> {
    static __device__ __forceinline__ void run(uint32_t &plane, uint32_t &carry) {
        const uint32_t out = __builtin_amdgcn_bitop3_b32(plane, carry, carry, 0xc0);     // plane & carry
        plane = __builtin_amdgcn_bitop3_b32(plane, carry, carry, 0x3c);                  // plane ^ carry
        carry = out;
    }
};
template <> struct HalfAdd<uint64_t> {
    static __device__ __forceinline__ void run(uint64_t &plane, uint64_t &carry) {
        uint32_t pl = (uint32_t) plane, ph = (uint32_t) (plane >> 32), cl = (uint32_t) carry, ch = (uint32_t) (carry >> 32);
        HalfAdd<uint32_t>::run(pl, cl);
        HalfAdd<uint32_t>::run(ph, ch);
        plane = ((uint64_t) ph << 32) | pl;
        carry = ((uint64_t) ch << 32) | cl;
    }
};
template <> struct HalfAdd<dl_u32x4> {
    static __device__ __forceinline__ void run(dl_u32x4 &plane, dl_u32x4 &carry) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t p = plane[i], c = carry[i];
            HalfAdd<uint32_t>::run(p, c);
            plane[i] = p;
            carry[i] = c;
        }
    }
};

template <typename V> __device__ __forceinline__ void csa(V &carry, V &sum, V a, V b, V c) {
    V cy, sm;
    FullAdd<V>::run(cy, sm, a, b, c);
    carry = cy;
    sum = sm;
}

template <typename V> struct Words;        // access to the 32-bit components of a vector
template <> struct Words<uint64_t> {
    static constexpr int n = 2;
    static __device__ __forceinline__ uint32_t get(uint64_t v, int c) { return (uint32_t) (v >> (32 * c)); }
    static __device__ __forceinline__ uint64_t zero() { return 0; }
};
template <> struct Words<dl_u32x4> {
    static constexpr int n = 4;
    static __device__ __forceinline__ uint32_t get(dl_u32x4 v, int c) { return v[c]; }
    static __device__ __forceinline__ dl_u32x4 zero() { return dl_u32x4{0, 0, 0, 0}; }
};

// Expands bit-sliced counters to integers and stores them: planes[q][p][c][lane] is component c
// of plane p (weight 2^p) of partial counter q for the lane's vector; the workgroup's wave w
// handles bits [BITS*w, BITS*w + BITS) of the lane's 32*NC sample bits, summing the NQ partials.
// (Kept rolled: this phase must not set the kernel's register budget.)
template <typename V, int NP, int NQ>
__device__ __forceinline__ void expand_counts(const uint32_t (*planes)[NP][Words<V>::n][DL_WAVE], int wave, int lane,
                                              int64_t col, bool live, int64_t cls, int64_t k, int64_t batch,
                                              int32_t *__restrict__ out, int32_t base = 0) {
    constexpr int NC = Words<V>::n;
    constexpr int BITS = 8 * NC;
    int32_t cnt[BITS];
#pragma unroll
    for (int s = 0; s < BITS; ++s) cnt[s] = base;
    const int first_bit = BITS * wave;
    const int comp = first_bit >> 5, shift = first_bit & 31;
#pragma unroll 1
    for (int q = 0; q < NQ; ++q) {
#pragma unroll 1
        for (int p = 0; p < NP; ++p) {
            const uint32_t slice = planes[q][p][comp][lane] >> shift;
#pragma unroll
            for (int s = 0; s < BITS; ++s) cnt[s] += (int32_t) (((slice >> s) & 1u) << p);
        }
    }
    if (live) {
        const int64_t sample0 = col * (32 * NC) + first_bit;
#pragma unroll
        for (int s = 0; s < BITS; ++s)
            if (sample0 + s < batch) out[(sample0 + s) * k + cls] = cnt[s];
    }
}

// Four vectors -> one vector of weight 4, through the running planes of weight 1 and 2.
template <typename V> __device__ __forceinline__ V csa_quad(V &ones, V &twos, const V *v) {
    V t2a, t2b, t4;
    csa(t2a, ones, ones, v[0], v[1]);
    csa(t2b, ones, ones, v[2], v[3]);
    csa(t4, twos, twos, t2a, t2b);
    return t4;
}

// Single pass over stored rows: blockIdx.x = column tile, blockIdx.y = class; every row is read
// exactly once, so the dispatch order does not matter for cache reuse.
template <typename V, int NPH>
__global__ __launch_bounds__(DL_BLOCK) void groupbitsum_kernel(const V *__restrict__ bits, int32_t *__restrict__ out,
                                                               int64_t ncols, int64_t per_class, int64_t k,
                                                               int64_t batch) {
    constexpr int NP = NPH + 4;
    constexpr int NC = Words<V>::n;
    __shared__ uint32_t planes_lds[4][NP][NC][DL_WAVE];

    const int wave = dl_wave_in_block();
    const int lane = dl_lane();
    const int64_t cls = blockIdx.y;
    const int64_t col = (int64_t) blockIdx.x * DL_WAVE + lane;
    const bool live = col < ncols;

    const int64_t chunk = (per_class + 3) / 4;
    int64_t r_begin = (int64_t) wave * chunk;
    if (r_begin > per_class) r_begin = per_class;
    int64_t r_end = r_begin + chunk;
    if (r_end > per_class) r_end = per_class;

    V ones = Words<V>::zero(), twos = ones, fours = ones, eights = ones;
    V high[NPH];
#pragma unroll
    for (int p = 0; p < NPH; ++p) high[p] = Words<V>::zero();

    const V *row = bits + (cls * per_class + r_begin) * ncols + (live ? col : 0);
    auto quad = [&](int64_t q0) -> V {
        V v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
            v[j] = (live && q0 + j < r_end) ? __builtin_nontemporal_load(row + (q0 - r_begin + j) * ncols)
                                            : Words<V>::zero();
        return csa_quad(ones, twos, v);
    };
    for (int64_t r = r_begin; r < r_end; r += 16) {
        V t8a, t8b, t16;
        {
            const V t4a = quad(r), t4b = quad(r + 4);
            csa(t8a, fours, fours, t4a, t4b);
        }
        {
            const V t4a = quad(r + 8), t4b = quad(r + 12);
            csa(t8b, fours, fours, t4a, t4b);
        }
        csa(t16, eights, eights, t8a, t8b);
#pragma unroll
        for (int p = 0; p < NPH; ++p) {
            const V old = high[p];
            high[p] = old ^ t16;
            t16 = old & t16;
        }
    }

#pragma unroll
    for (int c = 0; c < NC; ++c) {
        planes_lds[wave][0][c][lane] = Words<V>::get(ones, c);
        planes_lds[wave][1][c][lane] = Words<V>::get(twos, c);
        planes_lds[wave][2][c][lane] = Words<V>::get(fours, c);
        planes_lds[wave][3][c][lane] = Words<V>::get(eights, c);
#pragma unroll
        for (int p = 0; p < NPH; ++p) planes_lds[wave][4 + p][c][lane] = Words<V>::get(high[p], c);
    }
    __syncthreads();
    expand_counts<V, NP, 4>(planes_lds, wave, lane, col, live, cls, k, batch, out);
}

// ------------------------------------------------------------------------------------------
// Count fused with the net's last TREE layers, in two passes so that the gathers keep their
// cache reuse.  A gathered input row is used by several neurons of every class; the reuse only
// hits the Infinity Cache if the chip works on few 1 KB column tiles at a time, i.e. if the
// dispatch is column-tile-major like eval_tree_kernel's, with all classes of a tile together.
//   pass 1: blockIdx.x = chunk of COUNT_ROWS neurons of one class, blockIdx.y = column tile.
//           The workgroup computes its neurons' output vectors (never stored), counts them
//           bit-sliced (32 per wave -> 6 planes, four waves added -> 8 planes) and writes the
//           planes: 8 vectors per lane per 128 neurons instead of 128 output vectors.
//   pass 2: blockIdx.x = column tile, blockIdx.y = class: adds the chunks' planes bit-sliced,
//           expands them to integers and stores the counts.
// ------------------------------------------------------------------------------------------
#define DL_COUNT_ROWS 128     // neurons per workgroup in pass 1 (32 per wave)
#define DL_COUNT_PLANES 8     // planes a workgroup writes: counts 0 .. 128

// a + b for bit-sliced numbers: a has NA planes, b NB <= NA planes; result NA + 1 planes in a.
template <typename V, int NA, int NB> __device__ __forceinline__ void sliced_add(V *a, const V *b) {
    V carry = Words<V>::zero();
#pragma unroll
    for (int p = 0; p < NA; ++p) {
        if (p < NB) {
            V c2, sum;
            csa(c2, sum, a[p], b[p], carry);
            a[p] = sum;
            carry = c2;
        } else {
            const V old = a[p];
            a[p] = old ^ carry;
            carry = old & carry;
        }
    }
    a[NA] = carry;
}

template <typename V, int TREE>
__global__ __launch_bounds__(DL_BLOCK) void count_partial_kernel(const V *__restrict__ x,
                                                                 const int32_t *__restrict__ leaves,
                                                                 const uint64_t *__restrict__ gates,
                                                                 V *__restrict__ partial, int64_t ncols,
                                                                 int64_t per_class, int64_t chunks_per_class) {
    constexpr int G = 1 << TREE;
    __shared__ V lds[3][6][DL_WAVE];

    const int wave = dl_wave_in_block();
    const int lane = dl_lane();
    const int64_t chunk = blockIdx.x;
    const int64_t cls = chunk / chunks_per_class;
    const int64_t r_begin = (chunk - cls * chunks_per_class) * DL_COUNT_ROWS + (int64_t) wave * (DL_COUNT_ROWS / 4);
    int64_t r_end = r_begin + DL_COUNT_ROWS / 4;
    if (r_end > per_class) r_end = per_class;
    const int64_t col = (int64_t) blockIdx.y * DL_WAVE + lane;
    const bool live = col < ncols;
    const V *xcol = x + (live ? col : 0);

    V n[8];                                  // this wave's count: planes of weight 1 .. 32 (+2 spare)
#pragma unroll
    for (int p = 0; p < 8; ++p) n[p] = Words<V>::zero();
    auto quad = [&](int64_t q0) -> V {
        V v[4];
        V leaf[4][G];
        uint64_t gt[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            int64_t r = q0 + j;
            if (r >= per_class) r = per_class - 1;
            const int64_t nn = cls * per_class + r;
            gt[j] = gates[nn];
#pragma unroll
            for (int g = 0; g < G; ++g) {
                const int32_t id = leaves[nn * G + g];           // wave-uniform; -1: no gate looks at this row
                leaf[j][g] = live && id >= 0 ? xcol[(int64_t) id * ncols] : Words<V>::zero();
            }
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const V y = TreeFold<V, TREE>::run(leaf[j], gt[j]);
            v[j] = (live && q0 + j < r_end) ? y : Words<V>::zero();
        }
        return csa_quad(n[0], n[1], v);
    };
#pragma unroll
    for (int h = 0; h < 2; ++h) {            // two blocks of 16 neurons
        const int64_t r = r_begin + 16 * h;
        V t8a, t8b, t16;
        {
            const V t4a = quad(r), t4b = quad(r + 4);
            csa(t8a, n[2], n[2], t4a, t4b);
        }
        {
            const V t4a = quad(r + 8), t4b = quad(r + 12);
            csa(t8b, n[2], n[2], t4a, t4b);
        }
        csa(t16, n[3], n[3], t8a, t8b);
        const V old = n[4];                  // weight 16, then 32
        n[4] = old ^ t16;
        n[5] = n[5] | (old & t16);
    }

    // waves 1..3 park their six planes; wave 0 adds them: (w0 + w1) + (w2 + w3)
    if (wave != 0) {
#pragma unroll
        for (int p = 0; p < 6; ++p) lds[wave - 1][p][lane] = n[p];
    }
    __syncthreads();
    if (wave != 0) return;
    V m[8], t[8];
#pragma unroll
    for (int p = 0; p < 6; ++p) t[p] = lds[0][p][lane];
    sliced_add<V, 6, 6>(n, t);               // n: 7 planes
#pragma unroll
    for (int p = 0; p < 6; ++p) {
        m[p] = lds[1][p][lane];
        t[p] = lds[2][p][lane];
    }
    m[6] = m[7] = Words<V>::zero();
    sliced_add<V, 6, 6>(m, t);               // m: 7 planes
    sliced_add<V, 7, 7>(n, m);               // n: 8 planes
    if (live) {
        V *dst = partial + (((int64_t) blockIdx.y * gridDim.x + chunk) * DL_COUNT_PLANES) * DL_WAVE + lane;
#pragma unroll
        for (int p = 0; p < DL_COUNT_PLANES; ++p) __builtin_nontemporal_store(n[p], dst + (int64_t) p * DL_WAVE);
    }
}

// ------------------------------------------------------------------------------------------
// Count fused with the last one or two layers, the top layer walked along its evaluation
// schedule (schedule.cpp): consecutive top-layer neurons share an input vertex, whose value stays
// in registers, so a neuron costs 2^DS gathered rows instead of 2^(DS+1) (DS = 1: the vertex is a
// neuron of the layer below, a gate over two rows of x; DS = 0: a row of x itself).
//
// Consecutive neurons of a trail belong to arbitrary classes, so a wave cannot keep one counter.
// Instead a workgroup of DL_CC_WAVES waves proceeds in blocks: every wave walks DL_CC_WAVE_STEPS
// steps of its own contiguous range of the schedule and parks each output vector in LDS, at a
// slot (precomputed per wiring) that sorts the block's outputs by class; after a barrier the wave
// that owns a class reads that class's run of slots and adds it to bit-sliced counters it keeps
// in registers for the whole workgroup (DL_CC_PLANES planes: the plan guarantees at most 255
// neurons of a class per workgroup).  The counters go to the same partial-plane layout that
// count_finish_kernel sums: one "chunk" per workgroup.
//
// Per step the wave reads one 16-byte record (wave-uniform: a scalar load) that a small kernel
// composes per call from the schedule and the current gate ids:
//   rec[i + 1] = { la, lb, sub gate | top gate << 4 | slot << 8 } for step i, rec[0] for the
//   vertex before step 0; a wave that starts at step f seeds its chain from rec[f].
// ------------------------------------------------------------------------------------------
// Neurons of the top layer whose gate is constant (0 or 15, as it stands after constants were folded into it)
// output the same word for every sample: they are not parked and not counted.  What the ones among them add to
// every sample's count of their class goes into the result at the very end (count_finish_kernel's base).
#define DL_ONES_THREADS 1024
__global__ __launch_bounds__(DL_ONES_THREADS) void count_constant_ones_kernel(const uint8_t *__restrict__ w_top, int64_t per_class,
                                                                              int32_t *__restrict__ ones) {
    __shared__ int32_t part[DL_ONES_THREADS / DL_WAVE];
    const int64_t cls = blockIdx.x;
    int32_t n = 0;
    constexpr int AT_ONCE = 8;                                 // loads in flight per thread (one at a time, the kernel
                                                               // waits out a memory latency per DL_ONES_THREADS neurons)
    for (int64_t first = threadIdx.x; first < per_class; first += AT_ONCE * DL_ONES_THREADS) {
        uint32_t v[AT_ONCE];
#pragma unroll
        for (int u = 0; u < AT_ONCE; ++u) {
            const int64_t i = first + u * DL_ONES_THREADS;
            v[u] = i < per_class ? w_top[cls * per_class + i] : 0u;
        }
#pragma unroll
        for (int u = 0; u < AT_ONCE; ++u) n += (v[u] & 15u) == 15u;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) n += __shfl_xor(n, off);
    if (dl_lane() == 0) part[dl_wave_in_block()] = n;
    __syncthreads();
    if (threadIdx.x == 0) {
        int32_t total = 0;
        for (int i = 0; i < DL_ONES_THREADS / DL_WAVE; ++i) total += part[i];
        ones[cls] = total;
    }
}

// The plan of a wiring (slot, runs: every neuron parked, a block's outputs sorted by class) thinned for this call:
// one wave per block takes the constant neurons out, moves the others of their class up and shortens the
// class's run.  Steps are numbered as the count kernel walks them (workgroup, wave, block, step); lane c keeps
// count of the constant neurons of class c met so far.
static_assert(DL_CC_MAX_CLASSES <= DL_WAVE, "a lane per class");
__global__ __launch_bounds__(DL_BLOCK) void count_chain_thin_kernel(const int32_t *__restrict__ neuron,
                                                                    const uint8_t *__restrict__ w_top,
                                                                    const uint8_t *__restrict__ slot,
                                                                    const uint16_t *__restrict__ runs, int64_t steps,
                                                                    int64_t per_class, int64_t k, int blocks,
                                                                    int64_t nblocks, uint8_t *__restrict__ slot_call,
                                                                    uint16_t *__restrict__ runs_call) {
    const int lane = dl_lane();
    const int64_t gb = (int64_t) blockIdx.x * (DL_BLOCK / DL_WAVE) + dl_wave_in_block();      // (workgroup g, block b)
    if (gb >= nblocks) return;
    const int64_t g = gb / blocks, b = gb % blocks;
    const int64_t wg_steps = (int64_t) DL_CC_BLOCK * blocks, span = (int64_t) DL_CC_WAVE_STEPS * blocks;
    uint32_t gone = 0;
    for (int first = 0; first < DL_CC_BLOCK; first += DL_WAVE) {
        const int i = first + lane;                           // the order in which the plan numbered a class's slots
        const int64_t s = g * wg_steps + (i / DL_CC_WAVE_STEPS) * span + b * DL_CC_WAVE_STEPS + i % DL_CC_WAVE_STEPS;
        const int32_t n = i < DL_CC_BLOCK && s < steps ? neuron[s] : -1;
        int cls = -1;
        bool constant = false;
        if (n >= 0) {
            cls = (int) (n / per_class);
            const uint32_t gate = w_top[n] & 15u;
            constant = gate == 0u || gate == 15u;
        }
        uint32_t before = 0;
        for (int c = 0; c < (int) k; ++c) {
            const uint64_t met = __ballot(cls == c && constant);
            const uint32_t carried = (uint32_t) __builtin_amdgcn_readlane((int) gone, c);
            if (cls == c) before = carried + (uint32_t) __popcll(met & ((1ull << lane) - 1ull));
            if (lane == c) gone += (uint32_t) __popcll(met);
        }
        if (i < DL_CC_BLOCK) slot_call[s] = n >= 0 && !constant ? (uint8_t) (slot[s] - before) : (uint8_t) 255;
    }
    if (lane < k) {
        const uint32_t run = runs[gb * k + lane];
        runs_call[gb * k + lane] = (uint16_t) ((run & 255u) | (((run >> 8) - gone) << 8));
    }
}

template <int DS>
__global__ __launch_bounds__(DL_BLOCK) void compose_count_chain_kernel(TreeTables t, const int32_t *__restrict__ verts,
                                                                       const int32_t *__restrict__ neuron,
                                                                       const uint8_t *__restrict__ flip,
                                                                       const uint8_t *__restrict__ slot, int64_t steps,
                                                                       int64_t padded, dl_u32x4 *__restrict__ rec) {
    const int64_t i = (int64_t) blockIdx.x * DL_BLOCK + threadIdx.x;      // record index: step i - 1
    if (i > padded) return;
    const int64_t v = verts[i < steps ? i : steps];                        // vertex reached by step i - 1
    uint32_t la, lb = 0, bits = 0;
    if (DS == 1) {
        la = (uint32_t) t.a[0][v];
        lb = (uint32_t) t.b[0][v];
        bits = t.w[0][v] & 15u;
    } else {
        la = (uint32_t) v;
    }
    uint32_t where = 255;
    // the vertex is the second input of step i - 1's neuron and the first input of step i's; rows that no gate
    // looks at are not fetched (.w: bit 0 = skip la, bit 1 = skip lb, bit 2 = the vertex itself is not looked at)
    bool needed = false;
    if (i >= 1) {
        const int64_t s = i - 1;
        where = slot[s];
        if (s < steps && neuron[s] >= 0) {
            uint32_t top = t.w[DS][neuron[s]] & 15u;
            if (flip[s]) top = swap_gate_inputs(top);
            bits |= top << 4;
            needed = gate_uses_b(top);
        }
    }
    if (i < steps && neuron[i] >= 0) {
        uint32_t next = t.w[DS][neuron[i]] & 15u;
        if (flip[i]) next = swap_gate_inputs(next);
        needed = needed || gate_uses_a(next);
    }
    uint32_t skip = 0;
    if (!needed || (DS == 1 && !gate_uses_a(bits & 15u))) skip |= 1u;
    if (DS == 1 && (!needed || !gate_uses_b(bits & 15u))) skip |= 2u;
    if (!needed) skip |= 4u;                                  // nobody looks at the vertex: not evaluated either
    rec[i] = dl_u32x4{la, lb, bits | (where << 8), skip};
}

template <typename V, int DS, int CPW>
__global__ __launch_bounds__(DL_CC_WAVES * DL_WAVE) void count_chain_kernel(const V *__restrict__ x,
                                                                            const dl_u32x4 *__restrict__ rec,
                                                                            const uint16_t *__restrict__ runs,
                                                                            V *__restrict__ partial, int64_t ncols,
                                                                            int64_t k, int64_t nwg, int blocks,
                                                                            uint32_t xcd_owns_tiles) {
    __shared__ V stage[DL_CC_BLOCK + 1][DL_WAVE];        // the last slot stays zero: what a run's padding reads
    const int wave = dl_wave_in_block();
    const int lane = dl_lane();
    if (wave == 0) stage[DL_CC_BLOCK][lane] = Words<V>::zero();   // (visible after the first block's barrier)
    // Workgroups are dealt round-robin to the 8 XCDs.  xcd_owns_tiles (a whole number of column tiles per XCD): XCD j
    // takes the tiles j, j + 8, ...: the workgroups that gather from one column tile then share an L2 and an XCD
    // works on one column tile at a time.  Measured on 64000-row inputs: count group 2.71 -> 2.62 ms on a net where
    // no gate ignores an input (every row is fetched, twice), no change where many rows are skipped; the L2 hit rate
    // hardly moves (3 -> 4 %), so it is not second reads served by the L2 that is gained.  On 256000-row inputs it
    // loses (1.43 -> 1.58 ms): eight column tiles in flight are 2 GB, far beyond the 256 MB Infinity Cache that
    // serves a row's second read while the whole chip sweeps one tile; the launcher asks for it up to 64 MB a tile.
    int64_t g = blockIdx.x, tile = blockIdx.y;
    if (xcd_owns_tiles) {
        const int64_t id = (int64_t) blockIdx.y * gridDim.x + blockIdx.x, xcd = id % 8, place = id / 8;
        g = place % gridDim.x;
        tile = (place / gridDim.x) * 8 + xcd;
    }
    const int64_t col = tile * DL_WAVE + lane;
    const bool live = col < ncols;
    const V *xcol = x + (live ? col : 0);
    // the wave's range of the schedule: [0] = seed, [1 + j] = its step j
    const dl_u32x4 *wrec = rec + (g * DL_CC_WAVES + wave) * (int64_t) (DL_CC_WAVE_STEPS * blocks);

    auto vertex = [&](V ra, V rb, uint32_t bits) -> V {
        if (DS == 1) return gate_apply<V>(ra, rb, gate_masks(bits & 15u));
        return ra;
    };
    V prev;
    {
        const dl_u32x4 r = wrec[0];
        const V ra = (r.w & 1u) ? any_value<V>() : xcol[(int64_t) r.x * ncols];
        const V rb = DS != 1 ? ra : (r.w & 2u) ? any_value<V>() : xcol[(int64_t) r.y * ncols];
        prev = vertex(ra, rb, r.z);
    }
    // counter planes; carries of weight 4 and (with one set of counters, where the registers allow it) 8 waiting for a partner
    constexpr bool WAIT8 = CPW == 1;
    V cnt[CPW][DL_CC_PLANES], wait4[CPW], wait8[WAIT8 ? CPW : 1];
    uint32_t quads[CPW];
#pragma unroll
    for (int i = 0; i < CPW; ++i) {
#pragma unroll
        for (int p = 0; p < DL_CC_PLANES; ++p) cnt[i][p] = Words<V>::zero();
        wait4[i] = Words<V>::zero();
        if (WAIT8) wait8[i] = Words<V>::zero();
        quads[i] = 0;
    }

    // Phase A walks the wave's DL_CC_WAVE_STEPS steps of the block.  With one class per wave the registers hold the
    // rows of all of them, and they are requested before the block before is counted, so that the counting phase
    // hides most of their latency; with two sets of counters the rows are requested in two batches as the walk
    // needs them.  (Rows that no gate looks at are not fetched: wave-uniform flags.  Loads return in order and a
    // wait cannot tell how many of the conditional ones were issued since, so it covers all of them: nothing in the
    // counting phase may wait on a load.)
    constexpr int FIRST = CPW == 1 ? DL_CC_WAVE_STEPS : DL_CC_WAVE_STEPS / 2, REST = DL_CC_WAVE_STEPS - FIRST;
    constexpr bool AHEAD = CPW == 1;
    dl_u32x4 r0[FIRST];
    V ra0[FIRST], rb0[FIRST];
    auto issue = [&](auto count, const dl_u32x4 *r, V *ra, V *rb) {
#pragma unroll
        for (int j = 0; j < decltype(count)::value; ++j) {
            ra[j] = (r[j].w & 1u) ? any_value<V>() : xcol[(int64_t) r[j].x * ncols];
            if (DS == 1) rb[j] = (r[j].w & 2u) ? any_value<V>() : xcol[(int64_t) r[j].y * ncols];
        }
    };
    auto request = [&](auto count, int first, dl_u32x4 *r, V *ra, V *rb) {
#pragma unroll
        for (int j = 0; j < decltype(count)::value; ++j) r[j] = wrec[1 + first + j];
        issue(count, r, ra, rb);
    };
    auto walk = [&](auto count, const dl_u32x4 *r, const V *ra, const V *rb) {
#pragma unroll
        for (int j = 0; j < decltype(count)::value; ++j) {
            V cur = ra[j];
            if (DS == 1 && !(r[j].w & 4u)) cur = vertex(ra[j], rb[j], r[j].z);
            const uint32_t where = (r[j].z >> 8) & 255u;
            if (where != 255u) stage[where][lane] = gate_apply<V>(prev, cur, gate_masks((r[j].z >> 4) & 15u));
            prev = cur;
        }
    };
    const std::integral_constant<int, FIRST> first_batch;
    const std::integral_constant<int, REST> second_batch;
    if constexpr (AHEAD) request(first_batch, 0, r0, ra0, rb0);
    // this block's runs of parked outputs per owned class: read a block ahead (a scalar load: a vector load in the
    // counting phase would have to wait for the rows requested above, which return in order), so that the counting
    // phase starts without waiting for it
    auto run_of = [&](int b, int i) -> uint32_t {
        const int64_t cls = wave + i * DL_CC_WAVES;
        if (cls >= k || b >= blocks) return 0u;
        const int64_t at = (g * blocks + b) * k + cls;
        const uint32_t pair = reinterpret_cast<const uint32_t *>(runs)[at >> 1];
        return (at & 1) ? pair >> 16 : pair & 0xffffu;
    };
    uint32_t run_next[CPW];
#pragma unroll
    for (int i = 0; i < CPW; ++i) run_next[i] = run_of(0, i);
#pragma unroll 1
    for (int b = 0; b < blocks; ++b) {
        uint32_t run_now[CPW];
#pragma unroll
        for (int i = 0; i < CPW; ++i) {
            run_now[i] = run_next[i];
            run_next[i] = run_of(b + 1, i);
        }
        if constexpr (!AHEAD) request(first_batch, b * DL_CC_WAVE_STEPS, r0, ra0, rb0);
        if constexpr (AHEAD) {
            // The next block's rows are requested as soon as registers are free for them: part by part, right after
            // this block's steps that held those registers have been walked (the rows have a whole block's time to
            // arrive either way; asked for earlier, more of that time has requests in flight).
            constexpr int PART = FIRST / DL_CC_REQUEST_PARTS;
            const std::integral_constant<int, PART> part;
            const bool more = b + 1 < blocks;
#pragma unroll
            for (int i = 0; i < DL_CC_REQUEST_PARTS; ++i) {
                walk(part, r0 + i * PART, ra0 + i * PART, rb0 + i * PART);
                __builtin_amdgcn_sched_barrier(0);
                if (more) request(part, (b + 1) * DL_CC_WAVE_STEPS + i * PART, r0 + i * PART, ra0 + i * PART, rb0 + i * PART);
                __builtin_amdgcn_sched_barrier(0);
            }
        } else {
            walk(first_batch, r0, ra0, rb0);
        }
        if constexpr (REST > 0) {
            dl_u32x4 r[REST > 0 ? REST : 1];
            V ra[REST > 0 ? REST : 1], rb[REST > 0 ? REST : 1];
            request(second_batch, b * DL_CC_WAVE_STEPS + FIRST, r, ra, rb);
            walk(second_batch, r, ra, rb);
        }
        __builtin_amdgcn_sched_barrier(0);          // (requests moved up into the walk would not fit the registers)
        __syncthreads();
        // phase B: the owner of a class adds that class's run of parked outputs to its counters
#pragma unroll
        for (int i = 0; i < CPW; ++i) {
            const int64_t cls = wave + i * DL_CC_WAVES;
            if (cls < k) {
                const uint32_t run = run_now[i];
                const int start = (int) (run & 255u), n = (int) (run >> 8);
#pragma unroll 1
                for (int q = 0; q < n; q += 4) {
                    V v[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u) v[u] = stage[q + u < n ? start + q + u : DL_CC_BLOCK][lane];
                    const V c4 = csa_quad(cnt[i][0], cnt[i][1], v);       // weight 4
                    // A carry waits for the next one of its weight instead of rippling through the planes alone:
                    // every second quad a full adder at weight 4, every fourth one at weight 8 and the ripple
                    // (quads[i]: how many quads this counter has taken, wave-uniform).
                    if (!(quads[i] & 1u)) {
                        wait4[i] = c4;
                    } else {
                        V c8;
                        csa(c8, cnt[i][2], cnt[i][2], wait4[i], c4);
                        if (WAIT8 && !(quads[i] & 2u)) {
                            wait8[i] = c8;
                        } else if (WAIT8) {
                            V c16;
                            csa(c16, cnt[i][3], cnt[i][3], wait8[i], c8);
#pragma unroll
                            for (int p = 4; p < DL_CC_PLANES; ++p) HalfAdd<V>::run(cnt[i][p], c16);
                        } else {
#pragma unroll
                            for (int p = 3; p < DL_CC_PLANES; ++p) HalfAdd<V>::run(cnt[i][p], c8);
                        }
                    }
                    ++quads[i];
                }
            }
        }
        __syncthreads();
    }
    // the carries still waiting join the planes
#pragma unroll
    for (int i = 0; i < CPW; ++i) {
        if (quads[i] & 1u) {
            V c = wait4[i];
#pragma unroll
            for (int p = 2; p < DL_CC_PLANES; ++p) HalfAdd<V>::run(cnt[i][p], c);
        }
        if (WAIT8 && (quads[i] & 2u)) {
            V c = wait8[i];
#pragma unroll
            for (int p = 3; p < DL_CC_PLANES; ++p) HalfAdd<V>::run(cnt[i][p], c);
        }
    }
    if (live) {
#pragma unroll
        for (int i = 0; i < CPW; ++i) {
            const int64_t cls = wave + i * DL_CC_WAVES;
            if (cls < k) {
                V *dst = partial + (((tile * k + cls) * nwg + g) * DL_CC_PLANES) * DL_WAVE + lane;
#pragma unroll
                for (int p = 0; p < DL_CC_PLANES; ++p) __builtin_nontemporal_store(cnt[i][p], dst + (int64_t) p * DL_WAVE);
            }
        }
    }
}

template <typename V, int NP>
__global__ __launch_bounds__(DL_BLOCK) void count_finish_kernel(const V *__restrict__ partial, int32_t *__restrict__ out,
                                                                int64_t ncols, int64_t chunks_per_class, int64_t k,
                                                                int64_t batch, const int32_t *__restrict__ base) {
    constexpr int NC = Words<V>::n;
    __shared__ uint32_t planes_lds[4][NP][NC][DL_WAVE];
    const int wave = dl_wave_in_block();
    const int lane = dl_lane();
    // A sample's k counts are 4k consecutive bytes of the output, written by k workgroups.  Workgroups are dealt
    // round-robin to the 8 XCDs; the k of a column tile get consecutive places on ONE of them, so that they run at
    // about the same time and their 4-byte stores meet in that XCD's L2 before the lines are written back.
    const int64_t place = blockIdx.x / 8, xcd = blockIdx.x % 8;
    const int64_t tile = (place / k) * 8 + xcd, cls = place % k;
    if (tile * DL_WAVE >= ncols) return;
    const int64_t col = tile * DL_WAVE + lane;
    const bool live = col < ncols;

    V acc[NP + 1];
#pragma unroll
    for (int p = 0; p <= NP; ++p) acc[p] = Words<V>::zero();
    const V *src = partial + ((tile * (k * chunks_per_class) + cls * chunks_per_class) * DL_COUNT_PLANES) * DL_WAVE + lane;
    for (int64_t c = wave; c < chunks_per_class; c += 4) {
        V part[DL_COUNT_PLANES];
#pragma unroll
        for (int p = 0; p < DL_COUNT_PLANES; ++p)
            part[p] = live ? __builtin_nontemporal_load(src + (c * DL_COUNT_PLANES + p) * DL_WAVE) : Words<V>::zero();
        sliced_add<V, NP, DL_COUNT_PLANES>(acc, part);      // the carry out of plane NP-1 is zero by construction
    }
#pragma unroll
    for (int c = 0; c < NC; ++c) {
#pragma unroll
        for (int p = 0; p < NP; ++p) planes_lds[wave][p][c][lane] = Words<V>::get(acc[p], c);
    }
    __syncthreads();
    // (base: what the class's neurons that were left out of the partial counters add to every sample)
    expand_counts<V, NP, 4>(planes_lds, wave, lane, col, live, cls, k, batch, out, base ? base[cls] : 0);
}

// count_finish_kernel for 16-byte lanes and k <= 16 with whole-line stores.  A sample's k counts are 4k consecutive
// bytes of the output; one workgroup per (column tile, class) writes them as 4-byte stores 4k bytes apart, which
// costs half of that kernel's time.  Here a workgroup owns 16 columns of a tile (2048 consecutive samples) and ALL
// classes, wave c summing class c: a lane is (column l = lane % 16, chunk slot q = lane / 16) and adds up every
// fourth chunk; the four slots (rows of 16 lanes) are added bit-sliced with gfx950's row and half swaps; row q then
// expands the 32 samples of dword q, half of them per round, into an LDS stage laid out as the output is
// ([column][dword][sample][class], a pad per run so that a wave's stores spread over the banks), which the
// workgroup writes out in 256-byte pieces.
#define DL_FINISH_COLS 16
template <int NP>
__global__ __launch_bounds__(16 * DL_WAVE) void count_finish_rows_kernel(const dl_u32x4 *__restrict__ partial,
                                                                         int32_t *__restrict__ out, int64_t ncols,
                                                                         int64_t chunks_per_class, int k, int64_t batch,
                                                                         const int32_t *__restrict__ base) {
    using V = dl_u32x4;
    extern __shared__ int32_t finish_stage[];                  // [64 runs][16 samples * k + 1]
    const int wave = dl_wave_in_block(), lane = dl_lane();
    const int l = lane & (DL_FINISH_COLS - 1), q = lane / DL_FINISH_COLS;
    constexpr int GROUPS = DL_WAVE / DL_FINISH_COLS;
    // (the four workgroups of a column tile read a quarter each of the same 1 KB rows of partial counters: dealt to
    // ONE of the 8 XCDs, at consecutive places, what one of them fetches beyond its quarter serves the others:
    // fetched 0.50 -> 0.35 GB on the headline net)
    const int64_t place = blockIdx.x / 8, xcd = blockIdx.x % 8;
    const int64_t tile = (place / GROUPS) * 8 + xcd, group = place % GROUPS;
    if (tile * DL_WAVE >= ncols) return;
    const int64_t col0 = tile * DL_WAVE + group * DL_FINISH_COLS;              // first column of the workgroup
    const bool live = col0 + l < ncols;
    const int cls = wave;                                      // (the launch has k waves)

    V acc[NP + 1];
#pragma unroll
    for (int p = 0; p <= NP; ++p) acc[p] = V{0, 0, 0, 0};
    const V *src = partial + ((tile * ((int64_t) k * chunks_per_class) + (int64_t) cls * chunks_per_class) * DL_COUNT_PLANES) * DL_WAVE +
                   group * DL_FINISH_COLS + l;
    for (int64_t c = q; c < chunks_per_class; c += GROUPS) {
        V part[DL_COUNT_PLANES];
#pragma unroll
        for (int p = 0; p < DL_COUNT_PLANES; ++p)
            part[p] = live ? src[(c * DL_COUNT_PLANES + p) * DL_WAVE] : V{0, 0, 0, 0};
        sliced_add<V, NP, DL_COUNT_PLANES>(acc, part);         // the carry out of plane NP-1 is zero by construction
    }
    // rows 0 + 1 and 2 + 3, then the two halves: every row ends up with the total
#pragma unroll
    for (int round = 0; round < 2; ++round) {
        V other[NP];
#pragma unroll
        for (int p = 0; p < NP; ++p) {
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                const auto r = round == 0 ? __builtin_amdgcn_permlane16_swap(acc[p][d], acc[p][d], false, false)
                                          : __builtin_amdgcn_permlane32_swap(acc[p][d], acc[p][d], false, false);
                acc[p][d] = (uint32_t) r[0];
                other[p][d] = (uint32_t) r[1];
            }
        }
        sliced_add<V, NP, NP>(acc, other);
    }
    uint32_t slice[NP];
#pragma unroll
    for (int p = 0; p < NP; ++p) slice[p] = q == 0 ? acc[p][0] : q == 1 ? acc[p][1] : q == 2 ? acc[p][2] : acc[p][3];

    const int run = 16 * k + 1;                                // ints per (column, dword, half) run of the stage
    const int32_t add = base ? base[cls] : 0;
    const int64_t sample_group = col0 * 128;                   // first sample of the workgroup
    const int nwaves = k;
#pragma unroll 1
    for (int half = 0; half < 2; ++half) {
        int32_t *mine = finish_stage + (l * 4 + q) * run + cls;
#pragma unroll
        for (int s = 0; s < 16; ++s) {
            int32_t cnt = add;
#pragma unroll
            for (int p = 0; p < NP; ++p) cnt += (int32_t) (((slice[p] >> (16 * half + s)) & 1u) << p);
            mine[s * k] = cnt;
        }
        __syncthreads();
        // run m = 4 l + q holds samples 128 l + 32 q + 16 half .. + 15 of the workgroup, k counts each
        for (int m = wave; m < 4 * DL_FINISH_COLS; m += nwaves) {
            const int64_t first = sample_group + (m >> 2) * 128 + (m & 3) * 32 + 16 * half;
            const int64_t limit = first < batch ? (batch - first < 16 ? (batch - first) * k : 16 * k) : 0;
            for (int i = lane; i < 16 * k; i += DL_WAVE)
                if (i < limit) out[first * k + i] = finish_stage[m * run + i];
        }
        __syncthreads();
    }
}

// Any word width / row length: one thread per (sample, class), like the reference, but with
// lanes on consecutive samples of the sample-major output.
__global__ __launch_bounds__(DL_BLOCK) void groupbitsum_generic_kernel(const uint8_t *__restrict__ bits,
                                                                       int32_t *__restrict__ out, int64_t row_bytes,
                                                                       int64_t per_class, int64_t k, int64_t batch) {
    for (int64_t cls = blockIdx.y; cls < k; cls += gridDim.y) {
        for (int64_t s = (int64_t) blockIdx.x * DL_BLOCK + threadIdx.x; s < batch;
             s += (int64_t) gridDim.x * DL_BLOCK) {
            const uint8_t *p = bits + cls * per_class * row_bytes + (s >> 3);
            const int sh = (int) (s & 7);
            int32_t acc = 0;
            for (int64_t r = 0; r < per_class; ++r) acc += (p[r * row_bytes] >> sh) & 1;
            out[s * k + cls] = acc;
        }
    }
}

template <typename V>
void launch_groupbitsum_v(const void *bits, int32_t *out, int64_t row_bytes, int64_t per_class, int64_t k,
                          int64_t batch, hipStream_t s) {
    const int64_t ncols = row_bytes / (int64_t) sizeof(V);
    const dim3 grid((unsigned) dl_ceil_div(ncols, DL_WAVE), (unsigned) k);
    const int64_t chunk = (per_class + 3) / 4;      // rows one wave counts
    const V *b = (const V *) bits;
    // NPH planes above weight 8 hold counts up to 16 * 2^NPH - 1.
    if (chunk < (16LL << 8))
        DL_LAUNCH((groupbitsum_kernel<V, 8>), grid, dim3(DL_BLOCK), 0, s, b, out, ncols, per_class, k, batch);
    else if (chunk < (16LL << 14))
        DL_LAUNCH((groupbitsum_kernel<V, 14>), grid, dim3(DL_BLOCK), 0, s, b, out, ncols, per_class, k, batch);
    else
        DL_LAUNCH((groupbitsum_kernel<V, 27>), grid, dim3(DL_BLOCK), 0, s, b, out, ncols, per_class, k, batch);
}

// Rows of whole 64-bit words, 8-byte aligned: 16-byte lanes where rows and base allow it.
void launch_groupbitsum(const void *bits, int32_t *out, int64_t row_bytes, int64_t per_class, int64_t k, int64_t batch,
                        hipStream_t s) {
    if (row_bytes % 16 == 0 && dl_aligned(bits, 16))
        launch_groupbitsum_v<dl_u32x4>(bits, out, row_bytes, per_class, k, batch, s);
    else
        launch_groupbitsum_v<uint64_t>(bits, out, row_bytes, per_class, k, batch, s);
}

// Scratch of the two-pass fused count: DL_COUNT_PLANES row vectors per chunk per column tile.
int64_t count_scratch_bytes(int64_t out_dim, int64_t k, int64_t row_bytes) {
    const int64_t chunks = k * dl_ceil_div(out_dim / k, DL_COUNT_ROWS);
    const int64_t vec = row_bytes % 16 == 0 ? 16 : 8;
    const int64_t tiles = dl_ceil_div(row_bytes / vec, DL_WAVE);
    return tiles * chunks * DL_COUNT_PLANES * DL_WAVE * vec;
}

template <typename V, int TREE>
int launch_count_fused_v(const void *x, const int32_t *leaves, const uint64_t *gates, void *scratch, int32_t *out,
                         int64_t row_bytes, int64_t per_class, int64_t k, int64_t batch, hipStream_t s) {
    const int64_t ncols = row_bytes / (int64_t) sizeof(V);
    const int64_t tiles = dl_ceil_div(ncols, DL_WAVE);
    const int64_t chunks_per_class = dl_ceil_div(per_class, DL_COUNT_ROWS);
    if (k * chunks_per_class > 0x7fffffffLL || tiles > 65535 || dl_ceil_div(tiles, 8) * 8 * k > 0x7fffffffLL) return DL_ERR_TOO_LARGE;
    DL_LAUNCH((count_partial_kernel<V, TREE>), dim3((unsigned) (k * chunks_per_class), (unsigned) tiles),
                       dim3(DL_BLOCK), 0, s, (const V *) x, leaves, gates, (V *) scratch, ncols, per_class,
                       chunks_per_class);
    int st = dl_launch_status();
    if (st != DL_OK) return st;
    const dim3 grid((unsigned) (dl_ceil_div(tiles, 8) * 8 * k));
    // planes needed for counts up to per_class (pass 1 rounds a class up to whole chunks of 128)
    const int64_t top = chunks_per_class * DL_COUNT_ROWS;
    if (top < (1LL << 13))
        DL_LAUNCH((count_finish_kernel<V, 13>), grid, dim3(DL_BLOCK), 0, s, (const V *) scratch, out, ncols,
                           chunks_per_class, k, batch, (const int32_t *) nullptr);
    else if (top < (1LL << 18))
        DL_LAUNCH((count_finish_kernel<V, 18>), grid, dim3(DL_BLOCK), 0, s, (const V *) scratch, out, ncols,
                           chunks_per_class, k, batch, (const int32_t *) nullptr);
    else
        DL_LAUNCH((count_finish_kernel<V, 31>), grid, dim3(DL_BLOCK), 0, s, (const V *) scratch, out, ncols,
                           chunks_per_class, k, batch, (const int32_t *) nullptr);
    return dl_launch_status();
}

template <int TREE>
int launch_count_fused(const void *x, const int32_t *leaves, const uint64_t *gates, void *scratch, int32_t *out,
                       int64_t row_bytes, int64_t per_class, int64_t k, int64_t batch, hipStream_t s) {
    if (row_bytes % 16 == 0 && dl_aligned(x, 16) && dl_aligned(scratch, 16))
        return launch_count_fused_v<dl_u32x4, TREE>(x, leaves, gates, scratch, out, row_bytes, per_class, k, batch, s);
    return launch_count_fused_v<uint64_t, TREE>(x, leaves, gates, scratch, out, row_bytes, per_class, k, batch, s);
}

// Validates the description of a fused group and launches the composite builder.
// dims = {in_dim, width of layer 0, ..., width of layer depth-1} (host array).
int compose_tree(int depth, const int64_t *const *a, const int64_t *const *b, const uint8_t *const *w,
                 const int64_t *dims, const int32_t *order, void *workspace, int32_t **leaves, uint64_t **gates,
                 hipStream_t s) {
    if (depth < 1 || depth > DL_MAX_FUSE_DEPTH || !a || !b || !w || !dims || !workspace) return DL_ERR_INVALID_ARGUMENT;
    TreeTables t;
    for (int l = 0; l < depth; ++l) {
        if (!a[l] || !b[l] || !w[l] || dims[l] <= 0 || dims[l + 1] <= 0) return DL_ERR_INVALID_ARGUMENT;
        if (dims[l] > 0x7fffffffLL) return DL_ERR_TOO_LARGE;
        t.a[l] = a[l];
        t.b[l] = b[l];
        t.w[l] = w[l];
    }
    for (int l = depth; l < DL_MAX_FUSE_DEPTH; ++l) t.a[l] = t.b[l] = nullptr, t.w[l] = nullptr;
    if (!dl_aligned(workspace, 8)) return DL_ERR_INVALID_ARGUMENT;
    const int64_t out_dim = dims[depth];
    *gates = (uint64_t *) workspace;
    *leaves = (int32_t *) ((uint64_t *) workspace + out_dim);
    const int64_t blocks = dl_ceil_div(out_dim, DL_BLOCK);
    if (blocks > 0x7fffffffLL) return DL_ERR_TOO_LARGE;
    const dim3 grid((unsigned) blocks), block(DL_BLOCK);
    switch (depth) {
    case 1: DL_LAUNCH(compose_tree_kernel<1>, grid, block, 0, s, t, order, *leaves, *gates, out_dim); break;
    case 2: DL_LAUNCH(compose_tree_kernel<2>, grid, block, 0, s, t, order, *leaves, *gates, out_dim); break;
    case 3: DL_LAUNCH(compose_tree_kernel<3>, grid, block, 0, s, t, order, *leaves, *gates, out_dim); break;
    default: DL_LAUNCH(compose_tree_kernel<4>, grid, block, 0, s, t, order, *leaves, *gates, out_dim); break;
    }
    return dl_launch_status();
}

template <typename V>
int launch_eval_tree(int depth, const void *x, const int32_t *leaves, const uint64_t *gates, void *y, int64_t out_dim,
                     int64_t row_bytes, hipStream_t s) {
    const int64_t ncols = row_bytes / (int64_t) sizeof(V);
    int64_t ctiles = dl_ceil_div(ncols, DL_WAVE);
    if (ctiles > 65535) ctiles = 65535;
    const V *xv = (const V *) x;
    V *yv = (V *) y;
#define DL_TREE_LAUNCH(D, NPW, ITERS)                                                                                 \
    {                                                                                                                  \
        const int64_t ntiles = dl_ceil_div(out_dim, 4 * NPW * ITERS);                                                  \
        if (ntiles > 0x7fffffffLL) return DL_ERR_TOO_LARGE;                                                            \
        DL_LAUNCH((eval_tree_kernel<V, D, NPW, ITERS>), dim3((unsigned) ntiles, (unsigned) ctiles),           \
                           dim3(DL_BLOCK), 0, s, xv, leaves, gates, yv, out_dim, ncols);                               \
    }
    switch (depth) {
    case 1: DL_TREE_LAUNCH(1, 4, 4) break;
    case 2: DL_TREE_LAUNCH(2, 2, 4) break;
    case 3: DL_TREE_LAUNCH(3, 2, 4) break;
    default: DL_TREE_LAUNCH(4, 1, 8) break;
    }
#undef DL_TREE_LAUNCH
    return dl_launch_status();
}

bool valid_bit_count(int bit_count) { return bit_count == 8 || bit_count == 16 || bit_count == 32 || bit_count == 64; }

}  // namespace

thread_local int dl_last_hip_error_code = 0;
thread_local int dl_launch_result = 0;

extern "C" const char *dl_last_hip_error(void) { return hipGetErrorString((hipError_t) dl_last_hip_error_code); }

extern "C" int dl_logic_eval(const void *x, const int64_t *a, const int64_t *b, const uint8_t *w, void *y,
                             int64_t in_dim, int64_t out_dim, int64_t words, int bit_count, void *stream) {
    if (!valid_bit_count(bit_count)) return DL_ERR_BIT_COUNT;
    if (in_dim < 0 || out_dim < 0 || words < 0) return DL_ERR_INVALID_ARGUMENT;
    if (out_dim == 0 || words == 0) return DL_OK;
    if (!x || !a || !b || !w || !y || in_dim == 0) return DL_ERR_INVALID_ARGUMENT;
    hipStream_t s = (hipStream_t) stream;
    const int64_t row_bytes = words * (bit_count / 8);
    const uintptr_t mis = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y) | (uintptr_t) row_bytes;
    if (mis % 16 == 0) return launch_eval<dl_u32x4, 4, 4>(x, a, b, w, y, out_dim, row_bytes, s);
    if (mis % 8 == 0) return launch_eval<dl_u32x2, 4, 4>(x, a, b, w, y, out_dim, row_bytes, s);
    if (mis % 4 == 0) return launch_eval<uint32_t, 4, 4>(x, a, b, w, y, out_dim, row_bytes, s);
    if (mis % 2 == 0) return launch_eval<uint16_t, 4, 4>(x, a, b, w, y, out_dim, row_bytes, s);
    return launch_eval<uint8_t, 4, 4>(x, a, b, w, y, out_dim, row_bytes, s);
}

extern "C" int dl_tensor_packbits(const uint8_t *t, void *out, int64_t features, int64_t batch, int bit_count,
                                  int64_t *pad_len, void *stream) {
    if (!valid_bit_count(bit_count)) return DL_ERR_BIT_COUNT;
    if (features < 0 || batch < 0) return DL_ERR_INVALID_ARGUMENT;
    if (pad_len) *pad_len = (bit_count - batch % bit_count) % bit_count;
    if (features == 0 || batch == 0) return DL_OK;
    if (!t || !out) return DL_ERR_INVALID_ARGUMENT;
    hipStream_t s = (hipStream_t) stream;
    const int64_t words = dl_ceil_div(batch, bit_count);
    const int64_t out_row_bytes = words * (bit_count / 8);
    const unsigned gy = (unsigned) (features < 65535 ? features : 65535);
    const bool vec = batch % 16 == 0 && dl_aligned(t, 16) && out_row_bytes % 2 == 0 && dl_aligned(out, 2);
    if (vec) {
        int64_t gx = dl_ceil_div(out_row_bytes / 2, DL_BLOCK);
        if (gx > 65535) gx = 65535;
        DL_LAUNCH(packbits_vec16_kernel, dim3((unsigned) gx, gy), dim3(DL_BLOCK), 0, s, t, (uint8_t *) out,
                           features, batch, out_row_bytes);
    } else {
        int64_t gx = dl_ceil_div(out_row_bytes, DL_BLOCK);
        if (gx > 65535) gx = 65535;
        DL_LAUNCH(packbits_generic_kernel, dim3((unsigned) gx, gy), dim3(DL_BLOCK), 0, s, t,
                           (uint8_t *) out, features, batch, out_row_bytes);
    }
    return dl_launch_status();
}

// Gate ids of a layer for packed inference: argmax over each neuron's 16 weights, as
// weights.argmax(-1).to(uint8): the first maximal value wins, a NaN counts as maximal.
template <typename T, typename C> __device__ __forceinline__ uint32_t argmax16(const T *__restrict__ w) {
    C best = (C) w[0];
    uint32_t at = 0;
    if (best == best) {                                   // not NaN: look on
#pragma unroll
        for (int i = 1; i < 16; ++i) {
            const C v = (C) w[i];
            if (v != v) {                                 // the first NaN
                at = i;
                break;
            }
            if (v > best) best = v, at = i;
        }
    }
    return at;
}

template <typename T, typename C>
__global__ __launch_bounds__(DL_BLOCK) void gate_ids_kernel(const T *__restrict__ w, uint8_t *__restrict__ ids,
                                                            int64_t out_dim) {
    const int64_t n = (int64_t) blockIdx.x * DL_BLOCK + threadIdx.x;
    if (n >= out_dim) return;
    ids[n] = (uint8_t) argmax16<T, C>(w + n * 16);
}

// f'(a, b) = f(a, b) with the inputs that are constant (state 1: all zeros, 2: all ones; 0: varies) put in: the
// gate the neuron amounts to on the inputs that vary.  Gate ids are (f(0,0) f(0,1) f(1,0) f(1,1)), MSB first.
__device__ __forceinline__ uint32_t fold_gate(uint32_t op, uint32_t sa, uint32_t sb) {
    if (sa) {                                                   // a is the constant sa - 1
        const uint32_t f0 = sa == 2 ? (op >> 1) & 1u : (op >> 3) & 1u, f1 = sa == 2 ? op & 1u : (op >> 2) & 1u;
        op = f0 << 3 | f1 << 2 | f0 << 1 | f1;
    }
    if (sb) {
        const uint32_t f0 = sb == 2 ? (op >> 2) & 1u : (op >> 3) & 1u, f1 = sb == 2 ? op & 1u : (op >> 1) & 1u;
        op = f0 << 3 | f0 << 2 | f1 << 1 | f1;
    }
    return op;
}

// gate_ids_kernel and fold_gate_constants_kernel in one: the argmax gate with the constants among the layer's input
// rows folded in, and which of the layer's own outputs are constant
template <typename T, typename C>
__global__ __launch_bounds__(DL_BLOCK) void gate_ids_folded_kernel(const T *__restrict__ w, const int64_t *__restrict__ a,
                                                                   const int64_t *__restrict__ b,
                                                                   const uint8_t *__restrict__ state_in,
                                                                   uint8_t *__restrict__ ids, uint8_t *__restrict__ state_out,
                                                                   int64_t out_dim) {
    const int64_t n = (int64_t) blockIdx.x * DL_BLOCK + threadIdx.x;
    if (n >= out_dim) return;
    const uint32_t sa = state_in ? state_in[a[n]] : 0u, sb = state_in ? state_in[b[n]] : 0u;
    const uint32_t op = fold_gate(argmax16<T, C>(w + n * 16), sa, sb);
    ids[n] = (uint8_t) op;
    state_out[n] = op == 0u ? 1 : op == 15u ? 2 : 0;
}

extern "C" int dl_gate_ids(const void *w, uint8_t *ids, int64_t out_dim, int dtype, void *stream) {
    if (dtype != DL_F16 && dtype != DL_F32 && dtype != DL_F64) return DL_ERR_DTYPE;
    if (out_dim < 0) return DL_ERR_INVALID_ARGUMENT;
    if (out_dim == 0) return DL_OK;
    if (!w || !ids) return DL_ERR_INVALID_ARGUMENT;
    const int64_t blocks = dl_ceil_div(out_dim, DL_BLOCK);
    if (blocks > 0x7fffffffLL) return DL_ERR_TOO_LARGE;
    hipStream_t s = (hipStream_t) stream;
    const dim3 grid((unsigned) blocks), block(DL_BLOCK);
    if (dtype == DL_F16) DL_LAUNCH((gate_ids_kernel<__half, float>), grid, block, 0, s, (const __half *) w, ids, out_dim);
    else if (dtype == DL_F32) DL_LAUNCH((gate_ids_kernel<float, float>), grid, block, 0, s, (const float *) w, ids, out_dim);
    else DL_LAUNCH((gate_ids_kernel<double, double>), grid, block, 0, s, (const double *) w, ids, out_dim);
    return dl_launch_status();
}

extern "C" int dl_gate_ids_folded(const void *w, int dtype, const int64_t *a, const int64_t *b, const uint8_t *state_in,
                                  uint8_t *ids, uint8_t *state_out, int64_t out_dim, void *stream) {
    if (dtype != DL_F16 && dtype != DL_F32 && dtype != DL_F64) return DL_ERR_DTYPE;
    if (out_dim < 0) return DL_ERR_INVALID_ARGUMENT;
    if (out_dim == 0) return DL_OK;
    if (!w || !a || !b || !ids || !state_out) return DL_ERR_INVALID_ARGUMENT;
    const int64_t blocks = dl_ceil_div(out_dim, DL_BLOCK);
    if (blocks > 0x7fffffffLL) return DL_ERR_TOO_LARGE;
    hipStream_t s = (hipStream_t) stream;
    const dim3 grid((unsigned) blocks), block(DL_BLOCK);
    if (dtype == DL_F16)
        DL_LAUNCH((gate_ids_folded_kernel<__half, float>), grid, block, 0, s, (const __half *) w, a, b, state_in, ids, state_out,
                  out_dim);
    else if (dtype == DL_F32)
        DL_LAUNCH((gate_ids_folded_kernel<float, float>), grid, block, 0, s, (const float *) w, a, b, state_in, ids, state_out,
                  out_dim);
    else
        DL_LAUNCH((gate_ids_folded_kernel<double, double>), grid, block, 0, s, (const double *) w, a, b, state_in, ids,
                  state_out, out_dim);
    return dl_launch_status();
}

// Constants folded into the gates above them.  A neuron whose gate is constant (ids 0 and 15), or becomes so
// because its inputs are, has the same output word for every sample; the gate that reads it can be replaced by the
// one-input gate it amounts to: f'(a, b) = f(c, b) for every a.  The replaced gate ignores that input, so nothing is
// fetched for it.  Layer by layer: `state_in` says which input rows are constant (0 varies, 1 all zeros, 2 all ones;
// NULL: all vary), `w_out` receives the gate ids to evaluate (the same function of the varying inputs, bit for bit),
// `state_out` the constants among this layer's outputs.
__global__ __launch_bounds__(DL_BLOCK) void fold_gate_constants_kernel(const int64_t *__restrict__ a,
                                                                       const int64_t *__restrict__ b,
                                                                       const uint8_t *__restrict__ w,
                                                                       const uint8_t *__restrict__ state_in,
                                                                       uint8_t *__restrict__ w_out,
                                                                       uint8_t *__restrict__ state_out, int64_t out_dim) {
    const int64_t n = (int64_t) blockIdx.x * DL_BLOCK + threadIdx.x;
    if (n >= out_dim) return;
    const uint32_t sa = state_in ? state_in[a[n]] : 0u, sb = state_in ? state_in[b[n]] : 0u;
    const uint32_t op = fold_gate(w[n] & 15u, sa, sb);
    w_out[n] = (uint8_t) op;
    state_out[n] = op == 0u ? 1 : op == 15u ? 2 : 0;
}

extern "C" int dl_fold_gate_constants(const int64_t *a, const int64_t *b, const uint8_t *w, const uint8_t *state_in,
                                      uint8_t *w_out, uint8_t *state_out, int64_t out_dim, void *stream) {
    if (out_dim < 0) return DL_ERR_INVALID_ARGUMENT;
    if (out_dim == 0) return DL_OK;
    if (!a || !b || !w || !w_out || !state_out) return DL_ERR_INVALID_ARGUMENT;
    const int64_t blocks = dl_ceil_div(out_dim, DL_BLOCK);
    if (blocks > 0x7fffffffLL) return DL_ERR_TOO_LARGE;
    DL_LAUNCH(fold_gate_constants_kernel, dim3((unsigned) blocks), dim3(DL_BLOCK), 0, (hipStream_t) stream, a, b, w, state_in,
              w_out, state_out, out_dim);
    return dl_launch_status();
}

// Input rows that a layer looks at: live_in[r] = 1 where some neuron n with live_out[n] (NULL: every neuron) reads
// row r through an input its gate does not ignore.  live_in is cleared by the caller; the stores all write 1.
__global__ __launch_bounds__(DL_BLOCK) void mark_live_inputs_kernel(const int64_t *__restrict__ a,
                                                                    const int64_t *__restrict__ b,
                                                                    const uint8_t *__restrict__ w,
                                                                    const uint8_t *__restrict__ live_out,
                                                                    uint8_t *__restrict__ live_in, int64_t out_dim) {
    const int64_t n = (int64_t) blockIdx.x * DL_BLOCK + threadIdx.x;
    if (n >= out_dim || (live_out && !live_out[n])) return;
    const uint32_t op = w[n] & 15u;
    if (gate_uses_a(op)) live_in[a[n]] = 1;
    if (gate_uses_b(op)) live_in[b[n]] = 1;
}

extern "C" int dl_mark_live_inputs(const int64_t *a, const int64_t *b, const uint8_t *w, const uint8_t *live_out,
                                   uint8_t *live_in, int64_t out_dim, void *stream) {
    if (out_dim < 0) return DL_ERR_INVALID_ARGUMENT;
    if (out_dim == 0) return DL_OK;
    if (!a || !b || !w || !live_in) return DL_ERR_INVALID_ARGUMENT;
    const int64_t blocks = dl_ceil_div(out_dim, DL_BLOCK);
    if (blocks > 0x7fffffffLL) return DL_ERR_TOO_LARGE;
    DL_LAUNCH(mark_live_inputs_kernel, dim3((unsigned) blocks), dim3(DL_BLOCK), 0, (hipStream_t) stream, a, b, w, live_out,
              live_in, out_dim);
    return dl_launch_status();
}

// Sample-major bool bytes -> feature rows of `out_row_bytes` bytes each (a little-endian bit stream: sample s is
// bit s % 8 of byte s / 8, whatever the word width); bits past the batch are zero.
static int pack_batch_major_rows(const uint8_t *x, void *out, int64_t batch, int64_t features, int64_t out_row_bytes,
                                 hipStream_t s) {
    if (out_row_bytes % 8 == 0 && !dl_aligned(out, 8)) return DL_ERR_INVALID_ARGUMENT;
    const int64_t cols = dl_ceil_div(out_row_bytes, 8);          // 64-sample columns of the output
    const int64_t gx = dl_ceil_div(cols, 16);
    if (gx > 0x7fffffffLL) return DL_ERR_TOO_LARGE;
    if (features % 16 == 0 && dl_aligned(x, 16) && out_row_bytes % 8 == 0) {
        // A workgroup takes 8 word columns and a slice of the features, 68 bytes of LDS per feature.  Measured:
        // the longer the contiguous piece of a sample row a workgroup reads the better, down to one workgroup
        // per CU (2352 features); slices are whole 128-byte lines where the rows are.
        const int64_t unit = features % 128 == 0 ? 128 : 16;
        const int64_t want = dl_ceil_div(features, DL_PACK_MAX_SLICE / unit * unit);
        const int64_t slice = dl_ceil_div(dl_ceil_div(features, want), unit) * unit;
        const int64_t nslices = dl_ceil_div(features, slice);
        const int64_t blocks = dl_ceil_div(cols, DL_PACK_WC) * nslices;
        if (blocks > 0x3fffffffLL) return DL_ERR_TOO_LARGE;
        const size_t lds = (size_t) slice * DL_PACK_PITCH;
        const int64_t group = 8 * DL_PACK_SHARE * nslices;       // sets of neighbouring column groups, one set per XCD
        DL_LAUNCH(packbits_batch_major_rows_kernel, dim3((unsigned) blocks), dim3(DL_BLOCK), lds, s, x, (uint8_t *) out,
                  batch, features, (int) slice, (int) nslices, out_row_bytes, (uint32_t) (blocks / group * group));
    } else if (features % 4 == 0 && dl_aligned(x, 4)) {
        const int64_t gy = dl_ceil_div(features, 256);
        if (gy > 65535) return DL_ERR_TOO_LARGE;
        DL_LAUNCH(packbits_batch_major_kernel<4>, dim3((unsigned) gx, (unsigned) gy), dim3(DL_BLOCK), 0, s, x,
                           (uint8_t *) out, batch, features, out_row_bytes);
    } else {
        const int64_t gy = dl_ceil_div(features, 64);
        if (gy > 65535) return DL_ERR_TOO_LARGE;
        DL_LAUNCH(packbits_batch_major_kernel<1>, dim3((unsigned) gx, (unsigned) gy), dim3(DL_BLOCK), 0, s, x,
                           (uint8_t *) out, batch, features, out_row_bytes);
    }
    return dl_launch_status();
}

extern "C" int dl_tensor_packbits_batch_major(const uint8_t *x, void *out, int64_t batch, int64_t features,
                                              int bit_count, int64_t *pad_len, void *stream) {
    if (!valid_bit_count(bit_count)) return DL_ERR_BIT_COUNT;
    if (features < 0 || batch < 0) return DL_ERR_INVALID_ARGUMENT;
    if (pad_len) *pad_len = (bit_count - batch % bit_count) % bit_count;
    if (features == 0 || batch == 0) return DL_OK;
    if (!x || !out) return DL_ERR_INVALID_ARGUMENT;
    return pack_batch_major_rows(x, out, batch, features, dl_ceil_div(batch, bit_count) * (bit_count / 8),
                                 (hipStream_t) stream);
}

extern "C" int dl_tensor_packbits_batch_major_rows(const uint8_t *x, void *out, int64_t batch, int64_t features,
                                                   int64_t out_row_bytes, void *stream) {
    if (features < 0 || batch < 0 || out_row_bytes < 0 || batch > 8 * out_row_bytes) return DL_ERR_INVALID_ARGUMENT;
    if (features == 0 || out_row_bytes == 0) return DL_OK;
    if (!out || (!x && batch > 0)) return DL_ERR_INVALID_ARGUMENT;
    return pack_batch_major_rows(x, out, batch, features, out_row_bytes, (hipStream_t) stream);
}

extern "C" int dl_groupbitsum(const void *b, int32_t *out, int64_t in_dim, int64_t words, int bit_count,
                              int64_t pad_len, int64_t k, void *stream) {
    if (!valid_bit_count(bit_count)) return DL_ERR_BIT_COUNT;
    if (in_dim < 0 || words < 0 || k <= 0 || pad_len < 0) return DL_ERR_INVALID_ARGUMENT;
    if (in_dim % k != 0) return DL_ERR_NOT_DIVISIBLE;
    const int64_t batch = words * bit_count - pad_len;
    if (batch < 0) return DL_ERR_INVALID_ARGUMENT;
    if (batch == 0) return DL_OK;
    if (!out || (!b && in_dim > 0)) return DL_ERR_INVALID_ARGUMENT;
    hipStream_t s = (hipStream_t) stream;
    const int64_t per_class = in_dim / k;
    const int64_t row_bytes = words * (bit_count / 8);
    if (per_class > 0x7fffffffLL) return DL_ERR_TOO_LARGE;

    if (row_bytes % 8 == 0 && dl_aligned(b, 8) && k <= 65535) {
        if (dl_ceil_div(row_bytes / 8, DL_WAVE) > 0x7fffffffLL) return DL_ERR_TOO_LARGE;
        launch_groupbitsum(b, out, row_bytes, per_class, k, batch, s);
    } else {
        int64_t gx = dl_ceil_div(batch, DL_BLOCK);
        if (gx > 0x7fffffffLL) gx = 0x7fffffffLL;
        const unsigned gy = (unsigned) (k < 65535 ? k : 65535);
        DL_LAUNCH(groupbitsum_generic_kernel, dim3((unsigned) gx, gy), dim3(DL_BLOCK), 0, s,
                           (const uint8_t *) b, out, row_bytes, per_class, k, batch);
    }
    return dl_launch_status();
}

extern "C" int64_t dl_logic_eval_fused_workspace_bytes(int depth, int64_t out_dim) {
    if (depth < 1 || depth > DL_MAX_FUSE_DEPTH || out_dim < 0) return 0;
    return out_dim * (8 + 4 * (int64_t) (1 << depth));
}

extern "C" int dl_logic_eval_fused(const void *x, int depth, const int64_t *const *a, const int64_t *const *b,
                                   const uint8_t *const *w, const int64_t *dims, void *y, int64_t words, int bit_count,
                                   void *workspace, void *stream) {
    if (!valid_bit_count(bit_count)) return DL_ERR_BIT_COUNT;
    if (depth < 1 || depth > DL_MAX_FUSE_DEPTH || !dims || words < 0) return DL_ERR_INVALID_ARGUMENT;
    if (words == 0) return DL_OK;
    if (!x || !y) return DL_ERR_INVALID_ARGUMENT;
    const int64_t row_bytes = words * (bit_count / 8);
    const uintptr_t mis = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y) | (uintptr_t) row_bytes;
    if (mis % 8 != 0) return DL_ERR_TOO_LARGE;       // rows are not whole 64-bit words: use dl_logic_eval per layer
    hipStream_t s = (hipStream_t) stream;
    int32_t *leaves;
    uint64_t *gates;
    const int st = compose_tree(depth, a, b, w, dims, nullptr, workspace, &leaves, &gates, s);
    if (st != DL_OK) return st;
    if (mis % 16 == 0) return launch_eval_tree<dl_u32x4>(depth, x, leaves, gates, y, dims[depth], row_bytes, s);
    return launch_eval_tree<dl_u32x2>(depth, x, leaves, gates, y, dims[depth], row_bytes, s);
}

extern "C" int dl_logic_eval_fused_groupbitsum(const void *x, int depth, const int64_t *const *a,
                                               const int64_t *const *b, const uint8_t *const *w, const int64_t *dims,
                                               int32_t *out, int64_t words, int bit_count, int64_t pad_len, int64_t k,
                                               const int32_t *order, void *workspace, void *stream) {
    if (!valid_bit_count(bit_count)) return DL_ERR_BIT_COUNT;
    if (depth < 1 || depth > 2 || !dims || words < 0 || k <= 0 || pad_len < 0) return DL_ERR_INVALID_ARGUMENT;
    const int64_t out_dim = dims[depth];
    if (out_dim <= 0) return DL_ERR_INVALID_ARGUMENT;
    if (out_dim % k != 0) return DL_ERR_NOT_DIVISIBLE;
    const int64_t batch = words * bit_count - pad_len;
    if (batch < 0) return DL_ERR_INVALID_ARGUMENT;
    if (batch == 0) return DL_OK;
    if (!out || !x) return DL_ERR_INVALID_ARGUMENT;
    const int64_t per_class = out_dim / k;
    const int64_t row_bytes = words * (bit_count / 8);
    if (row_bytes % 8 != 0 || !dl_aligned(x, 8) || k > 65535 || per_class > 0x7fffffffLL) return DL_ERR_TOO_LARGE;
    if (dl_ceil_div(row_bytes / 8, DL_WAVE) > 0x7fffffffLL) return DL_ERR_TOO_LARGE;
    hipStream_t s = (hipStream_t) stream;
    int32_t *leaves;
    uint64_t *gates;
    const int st = compose_tree(depth, a, b, w, dims, order, workspace, &leaves, &gates, s);
    if (st != DL_OK) return st;
    // scratch for the partial counters follows the flattened wiring in the workspace
    const int64_t tables = dl_logic_eval_fused_workspace_bytes(depth, out_dim);
    void *scratch = (char *) workspace + ((tables + 15) / 16) * 16;
    if (depth == 1)
        return launch_count_fused<1>(x, leaves, gates, scratch, out, row_bytes, per_class, k, batch, s);
    return launch_count_fused<2>(x, leaves, gates, scratch, out, row_bytes, per_class, k, batch, s);
}

extern "C" int dl_count_group(void) { return DL_COUNT_ROWS; }

// ------------------------------------------------------------------------------------------
// dl_logic_eval_fused_groupbitsum for callers that cannot allocate (code under HIP graph capture,
// serving loops, harnesses that forbid hipMalloc): the workspace of the allocating entry point
// (flattened wiring + the bit-sliced partial counters the first pass hands to the second) lives in
// a file-scope device array.  Each GPU holds its own copy of the array at its own address, looked
// up once per device; host code only ever uses that looked-up address, never the array's name.
// Nothing in the array has to start at zero: compose_tree_kernel rewrites the wiring tables and
// pass 1 writes every counter that pass 2 reads.
// ------------------------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[DL_STATIC_SCRATCH_BYTES];

#define DL_MAX_DEVICES 64
static void *scratch_address[DL_MAX_DEVICES];      // per device: where that GPU's copy of `scratch` lives
static std::mutex scratch_mutex;

// Address of the current device's copy of `scratch` (looked up on the first call per device; that lookup is a
// runtime call that must not run while `stream` is being captured into a graph: refused then).
static int static_scratch(void **ptr, hipStream_t stream) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) {
        dl_last_hip_error_code = (int) e;
        return DL_ERR_LAUNCH;
    }
    if (dev < 0 || dev >= DL_MAX_DEVICES) return DL_ERR_TOO_LARGE;
    std::lock_guard<std::mutex> lock(scratch_mutex);
    if (!scratch_address[dev]) {
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        e = hipStreamIsCapturing(stream, &capturing);
        if (e != hipSuccess) {
            dl_last_hip_error_code = (int) e;
            return DL_ERR_LAUNCH;
        }
        if (capturing != hipStreamCaptureStatusNone) return DL_ERR_CAPTURING;
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            dl_last_hip_error_code = (int) (e != hipSuccess ? e : hipErrorInvalidSymbol);
            return DL_ERR_LAUNCH;
        }
        scratch_address[dev] = p;
    }
    *ptr = scratch_address[dev];
    return DL_OK;
}

extern "C" int dl_logic_eval_fused_groupbitsum_noalloc(const void *x, int depth, const int64_t *const *a,
                                                       const int64_t *const *b, const uint8_t *const *w,
                                                       const int64_t *dims, int32_t *out, int64_t words, int bit_count,
                                                       int64_t pad_len, int64_t k, const int32_t *order, void *stream) {
    if (!valid_bit_count(bit_count)) return DL_ERR_BIT_COUNT;
    if (depth < 1 || depth > 2 || !dims || words < 0 || k <= 0 || pad_len < 0) return DL_ERR_INVALID_ARGUMENT;
    const int64_t out_dim = dims[depth];
    if (out_dim <= 0) return DL_ERR_INVALID_ARGUMENT;
    if (out_dim % k != 0) return DL_ERR_NOT_DIVISIBLE;
    const int64_t row_bytes = words * (bit_count / 8);
    if (row_bytes % 8 != 0) return DL_ERR_TOO_LARGE;          // rows of whole 64-bit words only, as the allocating call
    const int64_t need = dl_logic_eval_fused_groupbitsum_workspace_bytes(depth, out_dim, words, bit_count, k);
    if (need > (int64_t) DL_STATIC_SCRATCH_BYTES) return DL_ERR_SCRATCH_LIMIT;
    void *ws = nullptr;
    const int st = static_scratch(&ws, (hipStream_t) stream);
    if (st != DL_OK) return st;
    return dl_logic_eval_fused_groupbitsum(x, depth, a, b, w, dims, out, words, bit_count, pad_len, k, order, ws, stream);
}

extern "C" int64_t dl_logic_eval_fused_groupbitsum_workspace_bytes(int depth, int64_t out_dim, int64_t words,
                                                                    int bit_count, int64_t k) {
    if (depth < 1 || depth > 2 || out_dim < 0 || words < 0 || k <= 0 || !valid_bit_count(bit_count)) return 0;
    if (out_dim % k != 0) return 0;
    const int64_t row_bytes = words * (bit_count / 8);
    if (row_bytes % 8 != 0) return 0;
    const int64_t tables = dl_logic_eval_fused_workspace_bytes(depth, out_dim);
    return ((tables + 15) / 16) * 16 + count_scratch_bytes(out_dim, k, row_bytes);
}

#define DL_EVAL_SCHEDULE_CHUNK 8
static_assert(DL_EVAL_SCHEDULE_CHUNK % 8 == 0, "eval_steps_kernel walks up to 8 steps at a time");

extern "C" int dl_eval_schedule_chunk(void) { return DL_EVAL_SCHEDULE_CHUNK; }

template <typename V>
int launch_eval_chain(int sub_depth, const void *x, const int32_t *sub_leaves, const uint64_t *sub_gates,
                      const int32_t *verts, const int32_t *neuron, const uint8_t *flip, const uint8_t *w_top, void *y,
                      int64_t nchunks, int64_t row_bytes, hipStream_t s) {
    const int64_t ncols = row_bytes / (int64_t) sizeof(V);
    int64_t ctiles = dl_ceil_div(ncols, DL_WAVE);
    if (ctiles > 65535) ctiles = 65535;
#define DL_CHAIN_LAUNCH(DS, ITERS)                                                                                     \
    {                                                                                                                  \
        const int64_t gx = dl_ceil_div(nchunks, 4 * ITERS);                                                            \
        if (gx > 0x7fffffffLL) return DL_ERR_TOO_LARGE;                                                                \
        DL_LAUNCH((eval_chain_kernel<V, DS, DL_EVAL_SCHEDULE_CHUNK, ITERS>),                                  \
                           dim3((unsigned) gx, (unsigned) ctiles), dim3(DL_BLOCK), 0, s, (const V *) x, sub_leaves,    \
                           sub_gates, verts, neuron, flip, w_top, (V *) y, nchunks, ncols);                            \
    }
    // Two consecutive chunks per wave halve the vertices that are evaluated only to seed a chain, but
    // also the workgroups per column tile; deep subtrees want enough of those to keep the chip on few
    // column tiles (whose input rows are what the L2 caches hold).
    const bool pair = sub_depth <= 1 || nchunks >= 4096;
    switch (sub_depth) {
    case 0: DL_CHAIN_LAUNCH(0, 2) break;
    case 1: DL_CHAIN_LAUNCH(1, 2) break;
    case 2:
        if (pair) DL_CHAIN_LAUNCH(2, 2) else DL_CHAIN_LAUNCH(2, 1)
        break;
    default:
        if (pair) DL_CHAIN_LAUNCH(3, 2) else DL_CHAIN_LAUNCH(3, 1)
        break;
    }
#undef DL_CHAIN_LAUNCH
    return dl_launch_status();
}

template <typename V, int DS>
int launch_eval_steps(const void *x, const int32_t *sub_leaves, const uint64_t *sub_gates, const int32_t *verts,
                      const int32_t *neuron, const uint8_t *flip, const uint8_t *w_top, const uint8_t *out_live, void *y,
                      void *records, int64_t steps, int64_t row_bytes, int64_t x_bytes, hipStream_t s) {
    constexpr int STEPS = DL_STEPS_PER_WAVE;
    const int64_t ncols = row_bytes / (int64_t) sizeof(V);
    StepRec<DS> *rec = (StepRec<DS> *) records;
    DL_LAUNCH(compose_steps_kernel<DS>, dim3((unsigned) dl_ceil_div(steps + 1, DL_BLOCK)), dim3(DL_BLOCK), 0, s, sub_leaves,
              sub_gates, verts, neuron, flip, w_top, out_live, steps, (uint32_t) ncols, rec);
    const int st = dl_launch_status();
    if (st != DL_OK) return st;
    int64_t ctiles = dl_ceil_div(ncols, DL_WAVE);
    // an input whose column tile (rows x 64 lanes) fits an XCD's 4 MB L2 with room to spare: one XCD per column tile
    const int64_t in_rows = ncols > 0 ? x_bytes / (ncols * (int64_t) sizeof(V)) : 0;
    // (and enough column tiles to keep the eight XCDs evenly busy: a whole number each, or many)
    const bool own = in_rows * DL_WAVE * (int64_t) sizeof(V) <= DL_XCD_TILE_BYTES && (ctiles % 8 == 0 || ctiles >= 64);
    if (own) ctiles = dl_ceil_div(ctiles, 8) * 8;                // (tiles past the last column do nothing)
    if (ctiles > 65528) ctiles = 65528;
    const int64_t gx = dl_ceil_div(steps, 4 * STEPS);
    if (gx > 0x7fffffffLL) return DL_ERR_TOO_LARGE;
    const dim3 grid((unsigned) gx, (unsigned) ctiles);
    if (x_bytes <= 0xffffffffLL)
        DL_LAUNCH((eval_steps_kernel<V, DS, STEPS, true>), grid, dim3(DL_BLOCK), 0, s, (const V *) x, rec, (V *) y, steps,
                  ncols, (uint32_t) x_bytes, own ? 1u : 0u);
    else
        DL_LAUNCH((eval_steps_kernel<V, DS, STEPS, false>), grid, dim3(DL_BLOCK), 0, s, (const V *) x, rec, (V *) y, steps,
                  ncols, 0u, own ? 1u : 0u);
    return dl_launch_status();
}

static int64_t step_record_bytes(int sub_depth) { return sub_depth == 3 ? 64 : sub_depth == 2 ? 32 : 16; }

extern "C" int64_t dl_logic_eval_chained_workspace_bytes(int depth, int64_t sub_dim, int64_t steps) {
    if (depth < 1 || depth > DL_MAX_FUSE_DEPTH || sub_dim < 0 || steps < 0) return 0;
    const int64_t tables = depth > 1 ? dl_logic_eval_fused_workspace_bytes(depth - 1, sub_dim) : 0;
    return ((tables + 63) / 64) * 64 + (steps + 1) * step_record_bytes(depth - 1);
}

extern "C" int dl_logic_eval_chained(const void *x, int depth, const int64_t *const *a, const int64_t *const *b,
                                     const uint8_t *const *w, const int64_t *dims, const int32_t *verts,
                                     const int32_t *neuron, const uint8_t *flip, int64_t steps, const uint8_t *out_live,
                                     void *y, int64_t words, int bit_count, void *workspace, void *stream) {
    if (!valid_bit_count(bit_count)) return DL_ERR_BIT_COUNT;
    if (depth < 1 || depth > DL_MAX_FUSE_DEPTH || !dims || !w || words < 0 || steps < 0 ||
        steps % DL_EVAL_SCHEDULE_CHUNK != 0)
        return DL_ERR_INVALID_ARGUMENT;
    if (words == 0 || dims[depth] == 0) return DL_OK;
    if (!x || !y || !verts || !neuron || !flip || !w[depth - 1] || steps < dims[depth]) return DL_ERR_INVALID_ARGUMENT;
    const int64_t row_bytes = words * (bit_count / 8);
    const uintptr_t mis = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y) | (uintptr_t) row_bytes;
    if (mis % 8 != 0) return DL_ERR_TOO_LARGE;       // rows are not whole 64-bit words: use dl_logic_eval per layer
    hipStream_t s = (hipStream_t) stream;
    int32_t *sub_leaves = nullptr;
    uint64_t *sub_gates = nullptr;
    if (depth > 1) {                                 // flatten the layers below the top one, per vertex
        const int st = compose_tree(depth - 1, a, b, w, dims, nullptr, workspace, &sub_leaves, &sub_gates, s);
        if (st != DL_OK) return st;
    }
    // one record per step where the pre-multiplied row offsets fit 32 bits (16-byte lanes only)
    const int64_t ncols16 = row_bytes / 16;
    if (mis % 16 == 0 && workspace && dl_aligned(workspace, 64) && dims[0] * ncols16 < 0xffffffffLL && dims[depth] * ncols16 < 0xffffffffLL) {
        const int64_t tables = depth > 1 ? dl_logic_eval_fused_workspace_bytes(depth - 1, dims[depth - 1]) : 0;
        void *records = (char *) workspace + ((tables + 63) / 64) * 64;
        const uint8_t *w_top = w[depth - 1];
        switch (depth - 1) {
        case 0: return launch_eval_steps<dl_u32x4, 0>(x, sub_leaves, sub_gates, verts, neuron, flip, w_top, out_live, y, records, steps, row_bytes, dims[0] * row_bytes, s);
        case 1: return launch_eval_steps<dl_u32x4, 1>(x, sub_leaves, sub_gates, verts, neuron, flip, w_top, out_live, y, records, steps, row_bytes, dims[0] * row_bytes, s);
        case 2: return launch_eval_steps<dl_u32x4, 2>(x, sub_leaves, sub_gates, verts, neuron, flip, w_top, out_live, y, records, steps, row_bytes, dims[0] * row_bytes, s);
        default: return launch_eval_steps<dl_u32x4, 3>(x, sub_leaves, sub_gates, verts, neuron, flip, w_top, out_live, y, records, steps, row_bytes, dims[0] * row_bytes, s);
        }
    }
    const int64_t nchunks = steps / DL_EVAL_SCHEDULE_CHUNK;
    if (mis % 16 == 0)
        return launch_eval_chain<dl_u32x4>(depth - 1, x, sub_leaves, sub_gates, verts, neuron, flip, w[depth - 1], y,
                                           nchunks, row_bytes, s);
    return launch_eval_chain<dl_u32x2>(depth - 1, x, sub_leaves, sub_gates, verts, neuron, flip, w[depth - 1], y, nchunks,
                                       row_bytes, s);
}

// ---- count fused with the last layers, walked along the evaluation schedule ----------------
static_assert(DL_CC_PLANES == DL_COUNT_PLANES, "count_finish_kernel reads DL_COUNT_PLANES planes per chunk");
static_assert(DL_CC_BLOCK <= 255, "slots are bytes, 255 = none");

namespace {

int64_t count_chain_partial_bytes(int64_t padded_steps, int blocks, int64_t k, int64_t row_bytes) {
    const int64_t vec = row_bytes % 16 == 0 ? 16 : 8;
    const int64_t tiles = dl_ceil_div(row_bytes / vec, DL_WAVE);
    return tiles * k * (padded_steps / (DL_CC_BLOCK * blocks)) * DL_CC_PLANES * DL_WAVE * vec;
}

// the plan as thinned per call: slot [padded], runs [blocks of the whole schedule x k], ones [k]; each 16-byte aligned
int64_t count_chain_call_plan_bytes(int64_t padded_steps, int64_t k) {
    const int64_t nblocks = padded_steps / DL_CC_BLOCK;
    return dl_ceil_div(padded_steps, 16) * 16 + dl_ceil_div(nblocks * k * 2, 16) * 16 + dl_ceil_div(k * 4, 16) * 16;
}

bool valid_cc_blocks(int blocks) { return blocks == 1 || blocks == 2 || blocks == 4 || blocks == 8 || blocks == 16; }

template <typename V, int DS>
int launch_count_chain(const void *x, const dl_u32x4 *rec, const uint16_t *runs, void *partial, int32_t *out,
                       const int32_t *ones, int64_t row_bytes, int64_t padded_steps, int blocks, int64_t per_class,
                       int64_t k, int64_t batch, int64_t in_rows, hipStream_t s) {
    const int64_t ncols = row_bytes / (int64_t) sizeof(V);
    const int64_t tiles = dl_ceil_div(ncols, DL_WAVE);
    const int64_t nwg = padded_steps / (DL_CC_BLOCK * blocks);
    if (nwg > 0x7fffffffLL || tiles > 65535 || dl_ceil_div(tiles, 8) * 8 * k > 0x7fffffffLL) return DL_ERR_TOO_LARGE;
    const dim3 grid((unsigned) nwg, (unsigned) tiles), block(DL_CC_WAVES * DL_WAVE);
    const uint32_t own = tiles % 8 == 0 && in_rows * DL_WAVE * (int64_t) sizeof(V) <= DL_CC_XCD_TILE_BYTES ? 1u : 0u;
    if (k <= DL_CC_WAVES)
        DL_LAUNCH((count_chain_kernel<V, DS, 1>), grid, block, 0, s, (const V *) x, rec, runs, (V *) partial, ncols, k, nwg,
                  blocks, own);
    else
        DL_LAUNCH((count_chain_kernel<V, DS, 2>), grid, block, 0, s, (const V *) x, rec, runs, (V *) partial, ncols, k, nwg,
                  blocks, own);
    int st = dl_launch_status();
    if (st != DL_OK) return st;
    if constexpr (sizeof(V) == 16) {
        // whole-line stores where a wave per class fits a workgroup
        const size_t lds = (size_t) 64 * (16 * k + 1) * 4;
        if (k <= 16 && per_class < (1LL << 13)) {              // (tiles <= 65535: the grid fits)
            const dim3 rgrid((unsigned) (dl_ceil_div(tiles, 8) * 8 * 4)), rblock((unsigned) (k * DL_WAVE));
            DL_LAUNCH((count_finish_rows_kernel<13>), rgrid, rblock, lds, s, (const dl_u32x4 *) partial, out, ncols, nwg, (int) k, batch,
                      ones);
            return dl_launch_status();
        }
    }
    const dim3 fgrid((unsigned) (dl_ceil_div(tiles, 8) * 8 * k));
    if (per_class < (1LL << 13))
        DL_LAUNCH((count_finish_kernel<V, 13>), fgrid, dim3(DL_BLOCK), 0, s, (const V *) partial, out, ncols, nwg, k, batch,
                  ones);
    else if (per_class < (1LL << 18))
        DL_LAUNCH((count_finish_kernel<V, 18>), fgrid, dim3(DL_BLOCK), 0, s, (const V *) partial, out, ncols, nwg, k, batch,
                  ones);
    else
        DL_LAUNCH((count_finish_kernel<V, 31>), fgrid, dim3(DL_BLOCK), 0, s, (const V *) partial, out, ncols, nwg, k, batch,
                  ones);
    return dl_launch_status();
}

}  // namespace

extern "C" int64_t dl_logic_eval_chained_groupbitsum_workspace_bytes(int64_t padded_steps, int blocks, int64_t words,
                                                                      int bit_count, int64_t k) {
    if (padded_steps < 0 || padded_steps % DL_CC_MAX_WG_STEPS != 0 || !valid_cc_blocks(blocks) || words < 0 || k <= 0 ||
        !valid_bit_count(bit_count))
        return 0;
    const int64_t row_bytes = words * (bit_count / 8);
    if (row_bytes % 8 != 0) return 0;
    return (padded_steps + 1) * 16 + count_chain_partial_bytes(padded_steps, blocks, k, row_bytes) +
           count_chain_call_plan_bytes(padded_steps, k);
}

extern "C" int dl_logic_eval_chained_groupbitsum(const void *x, int depth, const int64_t *const *a, const int64_t *const *b,
                                                 const uint8_t *const *w, const int64_t *dims, const int32_t *verts,
                                                 const int32_t *neuron, const uint8_t *flip, int64_t steps,
                                                 const uint8_t *slot, const uint16_t *runs, int64_t padded_steps,
                                                 int blocks, int32_t *out, int64_t words, int bit_count, int64_t pad_len,
                                                 int64_t k, void *workspace, void *stream) {
    if (!valid_bit_count(bit_count)) return DL_ERR_BIT_COUNT;
    if (depth < 1 || depth > 2 || !dims || !w || words < 0 || k <= 0 || pad_len < 0 || steps < 0 || padded_steps < steps ||
        padded_steps % DL_CC_MAX_WG_STEPS != 0 || !valid_cc_blocks(blocks))
        return DL_ERR_INVALID_ARGUMENT;
    const int64_t out_dim = dims[depth];
    if (out_dim <= 0 || steps < out_dim) return DL_ERR_INVALID_ARGUMENT;
    if (out_dim % k != 0) return DL_ERR_NOT_DIVISIBLE;
    const int64_t batch = words * bit_count - pad_len;
    if (batch < 0) return DL_ERR_INVALID_ARGUMENT;
    if (batch == 0) return DL_OK;
    if (!out || !x || !verts || !neuron || !flip || !slot || !runs || !workspace) return DL_ERR_INVALID_ARGUMENT;
    if (!dl_aligned(runs, 4)) return DL_ERR_INVALID_ARGUMENT;       // read two entries at a time (their number is even)
    for (int l = 0; l < depth; ++l)
        if (!w[l] || (l + 1 < depth && (!a || !b || !a[l] || !b[l])) || dims[l] <= 0) return DL_ERR_INVALID_ARGUMENT;
    const int64_t per_class = out_dim / k;
    const int64_t row_bytes = words * (bit_count / 8);
    if (row_bytes % 8 != 0 || !dl_aligned(x, 8) || k > DL_CC_MAX_CLASSES || per_class > 0x7fffffffLL ||
        dims[0] > 0x7fffffffLL || padded_steps > 0x7ffffff0LL)
        return DL_ERR_TOO_LARGE;
    if (!dl_aligned(workspace, 16)) return DL_ERR_INVALID_ARGUMENT;
    hipStream_t s = (hipStream_t) stream;

    TreeTables t;
    for (int l = 0; l < DL_MAX_FUSE_DEPTH; ++l) t.a[l] = t.b[l] = nullptr, t.w[l] = nullptr;
    for (int l = 0; l < depth; ++l) {
        t.a[l] = a ? a[l] : nullptr;
        t.b[l] = b ? b[l] : nullptr;
        t.w[l] = w[l];
    }
    dl_u32x4 *rec = (dl_u32x4 *) workspace;
    char *partial = (char *) workspace + (padded_steps + 1) * 16;
    const int64_t nblocks = padded_steps / DL_CC_BLOCK;
    uint8_t *slot_call = (uint8_t *) (partial + count_chain_partial_bytes(padded_steps, blocks, k, row_bytes));
    uint16_t *runs_call = (uint16_t *) (slot_call + dl_ceil_div(padded_steps, 16) * 16);
    int32_t *ones = (int32_t *) ((char *) runs_call + dl_ceil_div(nblocks * k * 2, 16) * 16);
    const uint8_t *w_top = w[depth - 1];
    DL_LAUNCH(count_constant_ones_kernel, dim3((unsigned) k), dim3(DL_ONES_THREADS), 0, s, w_top, per_class, ones);
    int st = dl_launch_status();
    if (st != DL_OK) return st;
    DL_LAUNCH(count_chain_thin_kernel, dim3((unsigned) dl_ceil_div(nblocks, DL_BLOCK / DL_WAVE)), dim3(DL_BLOCK), 0, s, neuron, w_top,
              slot, runs, steps, per_class, k, blocks, nblocks, slot_call, runs_call);
    st = dl_launch_status();
    if (st != DL_OK) return st;
    const dim3 cgrid((unsigned) dl_ceil_div(padded_steps + 1, DL_BLOCK));
    if (depth == 2)
        DL_LAUNCH(compose_count_chain_kernel<1>, cgrid, dim3(DL_BLOCK), 0, s, t, verts, neuron, flip, slot_call, steps,
                  padded_steps, rec);
    else
        DL_LAUNCH(compose_count_chain_kernel<0>, cgrid, dim3(DL_BLOCK), 0, s, t, verts, neuron, flip, slot_call, steps,
                  padded_steps, rec);
    st = dl_launch_status();
    if (st != DL_OK) return st;
    const bool wide = row_bytes % 16 == 0 && dl_aligned(x, 16);
    if (depth == 2) {
        if (wide) return launch_count_chain<dl_u32x4, 1>(x, rec, runs_call, partial, out, ones, row_bytes, padded_steps, blocks, per_class, k, batch, dims[0], s);
        return launch_count_chain<uint64_t, 1>(x, rec, runs_call, partial, out, ones, row_bytes, padded_steps, blocks, per_class, k, batch, dims[0], s);
    }
    if (wide) return launch_count_chain<dl_u32x4, 0>(x, rec, runs_call, partial, out, ones, row_bytes, padded_steps, blocks, per_class, k, batch, dims[0], s);
    return launch_count_chain<uint64_t, 0>(x, rec, runs_call, partial, out, ones, row_bytes, padded_steps, blocks, per_class, k, batch, dims[0], s);
}
