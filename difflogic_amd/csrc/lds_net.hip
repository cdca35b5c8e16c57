// Whole-net packed inference for narrow nets, resident in LDS: one workgroup carries COLS 64-bit
// word columns (COLS * 64 samples) through every layer of the net and counts the last layer's
// outputs per class, so HBM sees the packed input once and the [batch, k] counts once
// (F/8 + 4k bytes per sample) instead of one round trip per layer.
//
// Layout in LDS: one buffer act[row][COLS] of 64-bit words (8 * COLS bytes per row, rows = the
// widest layer).  Lanes run over NEURONS here (not over the batch as in the streaming kernels):
// a thread owns up to GPT neurons of a layer, reads both input rows of each from LDS, evaluates
// the gate with per-lane masks, keeps the results in registers until every thread has finished
// reading the layer's input, then overwrites the buffer with the layer's output.  The last layer
// is evaluated class by class (one wave per class): every lane adds its neurons' output words
// into bit-sliced counters, and the 64 lanes' counters are summed by a butterfly that halves
// the sample range a lane is responsible for at every exchange, so after six exchanges lane s
// holds the counts of samples COLS * s .. COLS * s + COLS - 1 of the workgroup.
//
// The wiring is read from a compact table built per call (one 32-bit record per gate: two
// 14-bit row ids and the 4-bit gate id), which every workgroup streams from L2.
//
// A hidden layer whose evaluation schedule is given (schedule.cpp: its neurons ordered along
// trails, consecutive ones sharing an input) is walked along it instead: a thread takes one chunk
// of 8 steps, reads 9 rows instead of 16, and its records hold one row id and the gate (inputs
// swapped where the schedule says so); the records are stored transposed (a thread's j-th entry at
// [j][thread]) so that a wave's loads are lane-consecutive.  A schedule of more than 1024 chunks
// has its remaining steps (at most 1024) evaluated one per thread from records of the
// neuron-by-neuron form.  Such a layer stores its outputs in SCHEDULE order, step s at row
// (s % 8) * stride + s / 8, so that a wave's stores are lane-consecutive; the records of the
// layer above are composed with its inputs renamed accordingly (the order of a hidden layer's rows
// is nobody else's business).
//
// One workgroup of 1024 threads fills a CU (its LDS), so nothing else runs there to hide a
// latency that all of its threads wait out together: every layer's records are requested one
// layer ahead, and the class phase's an iteration ahead.
#include "dl_common.h"

#define DL_NET_MAX_DEPTH 16
#define DL_NET_THREADS 1024
#define DL_NET_MAX_WIDTH 10240          // rows of act[] at COLS = 2: 160 KB of LDS
#define DL_NET_ID_BITS 14               // row ids in a gate record

namespace {

struct NetWiring {
    const int64_t *a[DL_NET_MAX_DEPTH];
    const int64_t *b[DL_NET_MAX_DEPTH];
    const uint8_t *w[DL_NET_MAX_DEPTH];
    const int32_t *verts[DL_NET_MAX_DEPTH];     // schedule of layer l, or null: evaluated neuron by neuron
    const int32_t *neuron[DL_NET_MAX_DEPTH];
    const uint8_t *flip[DL_NET_MAX_DEPTH];
    int32_t *pos[DL_NET_MAX_DEPTH];             // scheduled layers: row at which neuron n's output is stored
    int32_t width[DL_NET_MAX_DEPTH];            // neurons of layer l
    int32_t offset[DL_NET_MAX_DEPTH];           // first record of layer l
    int32_t steps[DL_NET_MAX_DEPTH];            // scheduled layers: steps (a multiple of 8); else 0
    int32_t stride[DL_NET_MAX_DEPTH];           // scheduled layers: row stride between a chunk's steps
    int32_t in_base;                            // row of act[] at which the net's input starts
};

struct NetShape {
    int32_t depth, in_dim, in_base;
    int32_t width[DL_NET_MAX_DEPTH];
    int32_t offset[DL_NET_MAX_DEPTH];
    int32_t steps[DL_NET_MAX_DEPTH];
    int32_t stride[DL_NET_MAX_DEPTH];
};

#define DL_NET_CHUNK 8                           // steps per thread of a scheduled layer (the schedule's chunk)

__device__ __forceinline__ uint32_t swap_gate(uint32_t op) {   // f'(a, b) = f(b, a)
    return (op & 9u) | ((op & 4u) >> 1) | ((op & 2u) << 1);
}

// rows of scheduled layers: neuron n of layer blockIdx.y -> (s % 8) * stride + s / 8 for its step s
__global__ __launch_bounds__(DL_BLOCK) void compose_net_pos_kernel(NetWiring t) {
    const int l = blockIdx.y;
    const int s = (int) (blockIdx.x * DL_BLOCK + threadIdx.x);
    if (s >= t.steps[l]) return;
    const int32_t n = t.neuron[l][s];
    if (n >= 0) t.pos[l][n] = (s % DL_NET_CHUNK) * t.stride[l] + s / DL_NET_CHUNK;
}

// Records of layer blockIdx.y.  Evaluated neuron by neuron: a | b << 14 | gate << 28 for neuron n.
// Scheduled: entry i = row of vertex verts[i] | gate of step i - 1 << 28 (the gate with its inputs
// swapped where the schedule walks the neuron from b to a; steps without a neuron keep gate 0 and
// their output row is never read).  Row ids are those of the layer below: its pos[] if scheduled.
__global__ __launch_bounds__(DL_BLOCK) void compose_net_kernel(NetWiring t, uint32_t *__restrict__ rec) {
    const int l = blockIdx.y;
    const int i = (int) (blockIdx.x * DL_BLOCK + threadIdx.x);
    const int32_t *below = (l > 0 && t.steps[l - 1] > 0) ? t.pos[l - 1] : nullptr;
    const int64_t first_row = l == 0 ? t.in_base : 0;
    auto row = [&](int64_t v) -> uint32_t { return (uint32_t) (below ? below[v] : v + first_row); };
    if (t.steps[l] > 0) {
        if (i > t.steps[l]) return;
        uint32_t gate = 0;
        if (i >= 1) {
            const int32_t n = t.neuron[l][i - 1];
            if (n >= 0) {
                gate = t.w[l][n] & 15u;
                if (t.flip[l][i - 1]) gate = swap_gate(gate);
            }
        }
        // entry 8 c + j is read by thread c as its j-th: stored at [j][c]; a chunk's ninth is the next one's first
        const uint32_t entry = row(t.verts[l][i]) | (gate << (2 * DL_NET_ID_BITS));
        uint32_t *tab = rec + t.offset[l];
        const int stride = t.stride[l];
        if (i < t.steps[l]) tab[(i % DL_NET_CHUNK) * stride + i / DL_NET_CHUNK] = entry;
        if (i % DL_NET_CHUNK == 0 && i > 0) tab[DL_NET_CHUNK * stride + i / DL_NET_CHUNK - 1] = entry;
        // steps past the chunks the workgroup's threads take (one each) are evaluated one per thread, from a record
        // of the neuron-by-neuron form; `gate` is that of step i - 1, which reads entries i - 1 and i
        const int first = DL_NET_CHUNK * DL_NET_THREADS;
        if (i > first)
            tab[(DL_NET_CHUNK + 1) * stride + i - 1 - first] =
                row(t.verts[l][i - 1]) | (row(t.verts[l][i]) << DL_NET_ID_BITS) | (gate << (2 * DL_NET_ID_BITS));
        return;
    }
    if (i >= t.width[l]) return;
    rec[t.offset[l] + i] = row(t.a[l][i]) | (row(t.b[l][i]) << DL_NET_ID_BITS) | ((t.w[l][i] & 15u) << (2 * DL_NET_ID_BITS));
}

// ------------------------------------------------------------------------------------------
// The net thinned for one call.  Constants are folded through the gate ids (a gate that reads a constant neuron is
// replaced by the one-input gate it amounts to), the neurons that some gate above still looks at are marked from the
// last layer downwards, and everything else is neither evaluated nor stored: a hidden layer keeps its marked neurons
// only, renumbered 0, 1, ... in their order (their rank is the row their output is stored at), the last layer's
// classes keep their non-constant neurons, and what the constant ones among them add to every sample's count goes
// into the result at the end.  The kernel reads the numbers of neurons left from `thin`:
//   thin[l], l < depth - 1        neurons left of hidden layer l
//   thin[depth - 1 + c]           neurons left of class c of the last layer
//   thin[depth - 1 + k + c]       constant-one neurons of class c
// ------------------------------------------------------------------------------------------
struct ThinTables {
    uint8_t *folded[DL_NET_MAX_DEPTH];          // gate ids of layer l with the constants below folded in
    uint8_t *live[DL_NET_MAX_DEPTH];            // hidden layer l: neuron n is looked at (the last layer: null)
    int32_t *rank[DL_NET_MAX_DEPTH];            // rank of neuron n among the neurons left (of its class, in the last layer)
    int32_t *thin;
    int32_t k;
};

__device__ __forceinline__ bool net_gate_uses_a(uint32_t op) { return (((op >> 3) ^ (op >> 1)) & 1u) || (((op >> 2) ^ op) & 1u); }
__device__ __forceinline__ bool net_gate_uses_b(uint32_t op) { return (((op >> 3) ^ (op >> 2)) & 1u) || (((op >> 1) ^ op) & 1u); }

#define DL_NET_RANK_ITEMS (DL_NET_MAX_WIDTH / DL_NET_THREADS)        // consecutive neurons per thread

// Gate ids of layer l with the constants of the layer below folded in (launched layer by layer, upwards); clears
// the layer's marks.  Gate ids are (f(0,0) f(0,1) f(1,0) f(1,1)), most significant bit first.
__global__ __launch_bounds__(DL_BLOCK) void net_thin_fold_kernel(NetWiring t, ThinTables thin, int l, int depth) {
    const int n = (int) (blockIdx.x * DL_BLOCK + threadIdx.x);
    if (n >= t.width[l]) return;
    uint32_t op = t.w[l][n] & 15u;
    if (l > 0) {
        const uint32_t ga = thin.folded[l - 1][t.a[l][n]], gb = thin.folded[l - 1][t.b[l][n]];
        if (ga == 0u || ga == 15u) {                             // a is constant: f'(a, b) = f(that constant, b)
            const uint32_t f0 = ga ? (op >> 1) & 1u : (op >> 3) & 1u, f1 = ga ? op & 1u : (op >> 2) & 1u;
            op = f0 << 3 | f1 << 2 | f0 << 1 | f1;
        }
        if (gb == 0u || gb == 15u) {
            const uint32_t f0 = gb ? (op >> 2) & 1u : (op >> 3) & 1u, f1 = gb ? op & 1u : (op >> 1) & 1u;
            op = f0 << 3 | f0 << 2 | f1 << 1 | f1;
        }
    }
    thin.folded[l][n] = (uint8_t) op;
    if (l + 1 < depth) thin.live[l][n] = 0;
}

// Where the caller's gate ids are folded already: only the marks of the hidden layers are cleared (in one launch;
// `marks` is the first layer's, the others follow it, `total` bytes in all).
__global__ __launch_bounds__(DL_BLOCK) void net_thin_clear_kernel(uint8_t *__restrict__ marks, int64_t total) {
    const int64_t i = (int64_t) blockIdx.x * DL_BLOCK + threadIdx.x;
    if (i < total) marks[i] = 0;
}

// Marks the neurons of layer l - 1 that a neuron of layer l which is itself looked at (the last layer: every neuron)
// looks at (launched layer by layer, downwards).  A constant neuron marks nothing and, its readers having been
// folded, is marked by nobody.
__global__ __launch_bounds__(DL_BLOCK) void net_thin_mark_kernel(NetWiring t, ThinTables thin, int l, int depth) {
    const int n = (int) (blockIdx.x * DL_BLOCK + threadIdx.x);
    if (n >= t.width[l] || (l + 1 < depth && !thin.live[l][n])) return;
    const uint32_t op = thin.folded[l][n];
    if (net_gate_uses_a(op)) thin.live[l - 1][t.a[l][n]] = 1;
    if (net_gate_uses_b(op)) thin.live[l - 1][t.b[l][n]] = 1;
}

// blockIdx.x = layer: exclusive prefix sums of "this neuron is left" over the layer's neurons.  One scan carries two
// counts: the neurons left in the low half of the word and, in the last layer, the constant-one neurons in the high
// half (neither exceeds DL_NET_MAX_WIDTH < 2^16, and both only grow along the layer, so differences of two scan
// values are the differences of the halves).
__global__ __launch_bounds__(DL_NET_THREADS) void net_thin_rank_kernel(NetWiring t, ThinTables thin, int depth) {
    static_assert(DL_NET_MAX_WIDTH < (1 << 16), "two counts per word");
    __shared__ int32_t wave_total[DL_NET_THREADS / DL_WAVE];
    __shared__ int32_t class_at[DL_NET_MAX_WIDTH + 1];       // last layer: the scan at each class's first neuron, then the total
    const int l = blockIdx.x, tid = (int) threadIdx.x, lane = dl_lane(), wave = dl_wave_in_block();
    const int width = t.width[l];
    const bool last = l == depth - 1;
    const uint8_t *flag_src = last ? thin.folded[l] : thin.live[l];
    int32_t local[DL_NET_RANK_ITEMS], sum = 0;
#pragma unroll
    for (int i = 0; i < DL_NET_RANK_ITEMS; ++i) {
        const int n = tid * DL_NET_RANK_ITEMS + i;
        int32_t f = 0;
        if (n < width) {
            const uint32_t v = flag_src[n];
            f = last ? (int32_t) (v != 0u && v != 15u) | ((int32_t) (v == 15u) << 16) : (int32_t) (v != 0u);
        }
        local[i] = sum;
        sum += f;
    }
    int32_t incl = sum;                                      // inclusive scan of the threads' sums within the wave
#pragma unroll
    for (int off = 1; off < DL_WAVE; off <<= 1) {
        const int32_t up = __shfl_up(incl, off, DL_WAVE);
        if (lane >= off) incl += up;
    }
    if (lane == DL_WAVE - 1) wave_total[wave] = incl;
    __syncthreads();
    int32_t before = 0, total = 0;
    for (int w = 0; w < DL_NET_THREADS / DL_WAVE; ++w) {
        if (w < wave) before += wave_total[w];
        total += wave_total[w];
    }
    const int32_t mine = before + incl - sum;                // the scan before this thread's first neuron
    int32_t *rank = thin.rank[l];
    if (!last) {
#pragma unroll
        for (int i = 0; i < DL_NET_RANK_ITEMS; ++i) {
            const int n = tid * DL_NET_RANK_ITEMS + i;
            if (n < width) rank[n] = mine + local[i];
        }
        if (tid == 0) thin.thin[l] = total;
        return;
    }
    // the last layer: ranks within each class, the classes' numbers of neurons left and of constant ones
    const int per_class = width / thin.k;
#pragma unroll
    for (int i = 0; i < DL_NET_RANK_ITEMS; ++i) {
        const int n = tid * DL_NET_RANK_ITEMS + i;
        if (n < width && n % per_class == 0) class_at[n / per_class] = mine + local[i];
    }
    if (tid == 0) class_at[thin.k] = total;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < DL_NET_RANK_ITEMS; ++i) {
        const int n = tid * DL_NET_RANK_ITEMS + i;
        if (n < width) rank[n] = ((mine + local[i]) & 0xffff) - (class_at[n / per_class] & 0xffff);
    }
    for (int c = tid; c < thin.k; c += DL_NET_THREADS) {
        const int32_t d = class_at[c + 1] - class_at[c];
        thin.thin[depth - 1 + c] = d & 0xffff;
        thin.thin[depth - 1 + thin.k + c] = d >> 16;
    }
}

// records of the neurons left (layer blockIdx.y): a | b << 14 | gate << 28 at the neuron's rank, the inputs' rows being
// the ranks of the layer below (an input that the gate does not look at: row 0)
__global__ __launch_bounds__(DL_BLOCK) void compose_net_thin_kernel(NetWiring t, ThinTables thin, int depth,
                                                                    uint32_t *__restrict__ rec) {
    const int l = blockIdx.y;
    const int n = (int) (blockIdx.x * DL_BLOCK + threadIdx.x);
    if (n >= t.width[l]) return;
    const uint32_t gate = thin.folded[l][n];
    int64_t at;
    if (l < depth - 1) {
        if (!thin.live[l][n]) return;
        at = thin.rank[l][n];
    } else {
        if (gate == 0u || gate == 15u) return;
        const int per_class = t.width[l] / thin.k;
        at = (int64_t) (n / per_class) * per_class + thin.rank[l][n];
    }
    auto row = [&](int64_t v) -> uint32_t { return (uint32_t) (l == 0 ? v + t.in_base : thin.rank[l - 1][v]); };
    const uint32_t ra = net_gate_uses_a(gate) ? row(t.a[l][n]) : 0u, rb = net_gate_uses_b(gate) ? row(t.b[l][n]) : 0u;
    rec[t.offset[l] + at] = ra | (rb << DL_NET_ID_BITS) | (gate << (2 * DL_NET_ID_BITS));
}

// COLS 64-bit words as 2 * COLS dwords
template <int COLS> struct Row { uint32_t d[2 * COLS]; };

// act[] is addressed in units of one row (8 * COLS bytes): 16-byte accesses for COLS >= 2, one
// 8-byte access for COLS = 1
template <int COLS> __device__ __forceinline__ Row<COLS> lds_row(const void *act, uint32_t row) {
    Row<COLS> r;
    if constexpr (COLS == 1) {
        const dl_u32x2 v = static_cast<const dl_u32x2 *>(act)[row];
        r.d[0] = v.x, r.d[1] = v.y;
    } else {
#pragma unroll
        for (int q = 0; q < COLS / 2; ++q) {
            const dl_u32x4 v = static_cast<const dl_u32x4 *>(act)[row * (COLS / 2) + q];
            r.d[4 * q] = v.x, r.d[4 * q + 1] = v.y, r.d[4 * q + 2] = v.z, r.d[4 * q + 3] = v.w;
        }
    }
    return r;
}

template <int COLS> __device__ __forceinline__ void lds_store(void *act, uint32_t row, const Row<COLS> &r) {
    if constexpr (COLS == 1) {
        static_cast<dl_u32x2 *>(act)[row] = dl_u32x2{r.d[0], r.d[1]};
    } else {
#pragma unroll
        for (int q = 0; q < COLS / 2; ++q)
            static_cast<dl_u32x4 *>(act)[row * (COLS / 2) + q] =
                dl_u32x4{r.d[4 * q], r.d[4 * q + 1], r.d[4 * q + 2], r.d[4 * q + 3]};
    }
}

// gate id = truth table (f(0,0) f(0,1) f(1,0) f(1,1)), MSB first, in bits 28..31 of the record;
// masks are per lane here
template <int COLS>
__device__ __forceinline__ Row<COLS> gate_mix(const Row<COLS> &a, const Row<COLS> &b, uint32_t rec) {
    const uint32_t m00 = 0u - ((rec >> 31) & 1u), m01 = 0u - ((rec >> 30) & 1u);
    const uint32_t m10 = 0u - ((rec >> 29) & 1u), m11 = 0u - ((rec >> 28) & 1u);
    Row<COLS> y;
#pragma unroll
    for (int i = 0; i < 2 * COLS; ++i) {
        const uint32_t hi = (b.d[i] & m11) | (~b.d[i] & m10);
        const uint32_t lo = (b.d[i] & m01) | (~b.d[i] & m00);
        y.d[i] = (a.d[i] & hi) | (~a.d[i] & lo);
    }
    return y;
}

template <int COLS>
__device__ __forceinline__ Row<COLS> gate_rows(const void *act, uint32_t rec) {
    const uint32_t ia = rec & ((1u << DL_NET_ID_BITS) - 1), ib = (rec >> DL_NET_ID_BITS) & ((1u << DL_NET_ID_BITS) - 1);
    return gate_mix<COLS>(lds_row<COLS>(act, ia), lds_row<COLS>(act, ib), rec);
}

// carry-save adder on dwords: a + b + c = 2 * carry + sum, bit by bit
// (two three-input bit operations, truth tables 0xe8 = majority and 0x96 = parity, stated as such: the compiler
// otherwise rearranges a chain of adders into half as many instructions again)
__device__ __forceinline__ void csa32(uint32_t &carry, uint32_t &sum, uint32_t a, uint32_t b, uint32_t c) {
    const uint32_t cy = __builtin_amdgcn_bitop3_b32(a, b, c, 0xe8);
    sum = __builtin_amdgcn_bitop3_b32(a, b, c, 0x96);
    carry = cy;
}

// plane += carry in place, carry = what leaves the plane (also two stated bit operations, so that a ripple stays a chain)
__device__ __forceinline__ void half_add32(uint32_t &plane, uint32_t &carry) {
    const uint32_t out = __builtin_amdgcn_bitop3_b32(plane, carry, carry, 0xc0);
    plane = __builtin_amdgcn_bitop3_b32(plane, carry, carry, 0x3c);
    carry = out;
}

// a (NP planes, one dword each) += b (NP planes); the sum takes NP + 1 planes
template <int NP> __device__ __forceinline__ void planes_add(uint32_t *a, const uint32_t *b) {
    uint32_t carry = 0;
#pragma unroll
    for (int p = 0; p < NP; ++p) {
        const uint32_t u = a[p] ^ b[p];
        const uint32_t c2 = (a[p] & b[p]) | (u & carry);
        a[p] = u ^ carry;
        carry = c2;
    }
    a[NP] = carry;
}

// ---- summing the 64 lanes' bit-sliced counters ---------------------------------------------------
// A lane enters with NP0 planes for each of the 2 * COLS dwords of its row (dword d = samples
// 32 d .. 32 d + 31 of the workgroup's COLS * 64).  Every exchange pairs each lane with one whose
// lane id differs in bit BIT, halves the set of samples a lane is responsible for, and adds the
// partner's counters for the half it keeps (one more plane).  After six exchanges lane s is left
// with the totals of samples COLS * s .. COLS * s + COLS - 1.  Any pairing that flips bit BIT
// will do (the other bits it flips have not been used yet), which lets the four low exchanges be
// DPP moves (mirrors and quad permutations) instead of trips through the LDS crossbar.

template <int BIT> __device__ __forceinline__ uint32_t lane_partner(uint32_t v) {
    if constexpr (BIT == 3)
        return (uint32_t) __builtin_amdgcn_update_dpp(0, (int) v, 0x140, 0xf, 0xf, false);   // row_mirror: lane ^ 15
    else if constexpr (BIT == 2)
        return (uint32_t) __builtin_amdgcn_update_dpp(0, (int) v, 0x141, 0xf, 0xf, false);   // row_half_mirror: lane ^ 7
    else if constexpr (BIT == 1)
        return (uint32_t) __builtin_amdgcn_update_dpp(0, (int) v, 0x4e, 0xf, 0xf, false);    // quad_perm [2,3,0,1]: lane ^ 2
    else if constexpr (BIT == 0)
        return (uint32_t) __builtin_amdgcn_update_dpp(0, (int) v, 0xb1, 0xf, 0xf, false);    // quad_perm [1,0,3,2]: lane ^ 1
    else
        return (uint32_t) __shfl_xor((int) v, 1 << BIT, DL_WAVE);
}

// D dwords per lane -> D / 2: the lane whose bit BIT is set keeps the upper half of the dwords
template <int D, int NP, int BIT, int NPMAX> __device__ __forceinline__ void fold_dwords(uint32_t (*q)[NPMAX], int lane) {
    const bool up = ((lane >> BIT) & 1) != 0;
#pragma unroll
    for (int i = 0; i < D / 2; ++i) {
        uint32_t other[NP];
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            const uint32_t lo = q[i][p], hi = q[D / 2 + i][p];
            if constexpr (BIT == 5 || BIT == 4) {
                // gfx950's swaps exchange the upper half (odd rows of 16) of the first operand with the lower half
                // (even rows) of the second: afterwards one holds the lane's own dword of the half it keeps and the
                // other its partner's, which one being the same to the sum
                const auto r = BIT == 5 ? __builtin_amdgcn_permlane32_swap(lo, hi, false, false)
                                        : __builtin_amdgcn_permlane16_swap(lo, hi, false, false);
                q[i][p] = (uint32_t) r[0];
                other[p] = (uint32_t) r[1];
            } else {
                other[p] = lane_partner<BIT>(up ? lo : hi);
                q[i][p] = up ? hi : lo;
            }
        }
        planes_add<NP>(q[i], other);
    }
}

// one dword per lane: the lane whose bit BIT is set keeps the bit positions whose index has bit J set
template <int NP, int J, int BIT> __device__ __forceinline__ void fold_bits(uint32_t *q, int lane) {
    constexpr uint32_t upper = J == 4 ? 0xffff0000u : J == 3 ? 0xff00ff00u : J == 2 ? 0xf0f0f0f0u
                             : J == 1 ? 0xccccccccu : 0xaaaaaaaau;
    const uint32_t keep = ((lane >> BIT) & 1) ? upper : ~upper;
    uint32_t other[NP];
#pragma unroll
    for (int p = 0; p < NP; ++p) {
        other[p] = lane_partner<BIT>(q[p]) & keep;
        q[p] &= keep;
    }
    planes_add<NP>(q, other);
}

// q[d][p]: plane p of dword d.  Returns in count[t] the total of sample COLS * lane + t.
template <int COLS, int NP0>
__device__ __forceinline__ void lanes_count(uint32_t (*q)[NP0 + 6], int lane, int32_t *count) {
    static_assert(COLS == 1 || COLS == 2 || COLS == 4, "columns per workgroup");
    if constexpr (COLS == 4) {
        fold_dwords<8, NP0, 5, NP0 + 6>(q, lane);
        fold_dwords<4, NP0 + 1, 4, NP0 + 6>(q, lane);
        fold_dwords<2, NP0 + 2, 3, NP0 + 6>(q, lane);
        fold_bits<NP0 + 3, 4, 2>(q[0], lane);
        fold_bits<NP0 + 4, 3, 1>(q[0], lane);
        fold_bits<NP0 + 5, 2, 0>(q[0], lane);
    } else if constexpr (COLS == 2) {
        fold_dwords<4, NP0, 5, NP0 + 6>(q, lane);
        fold_dwords<2, NP0 + 1, 4, NP0 + 6>(q, lane);
        fold_bits<NP0 + 2, 4, 3>(q[0], lane);
        fold_bits<NP0 + 3, 3, 2>(q[0], lane);
        fold_bits<NP0 + 4, 2, 1>(q[0], lane);
        fold_bits<NP0 + 5, 1, 0>(q[0], lane);
    } else {
        fold_dwords<2, NP0, 5, NP0 + 6>(q, lane);
        fold_bits<NP0 + 1, 4, 4>(q[0], lane);
        fold_bits<NP0 + 2, 3, 3>(q[0], lane);
        fold_bits<NP0 + 3, 2, 2>(q[0], lane);
        fold_bits<NP0 + 4, 1, 1>(q[0], lane);
        fold_bits<NP0 + 5, 0, 0>(q[0], lane);
    }
    const int first = (lane * COLS) & 31;                      // bit position of sample COLS * lane in its dword
#pragma unroll
    for (int t = 0; t < COLS; ++t) {
        count[t] = 0;
#pragma unroll
        for (int p = 0; p < NP0 + 6; ++p) count[t] |= (int32_t) ((q[0][p] >> (first + t)) & 1u) << p;
    }
}

// records of the class phase: four neurons of a lane at a time, past the end of the class -> the class's last
__device__ __forceinline__ void load_class_records(uint32_t *r4, const uint32_t *ctab, int64_t i0, int64_t per_class) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int64_t i = i0 + u * DL_WAVE;
        r4[u] = ctab[i < per_class ? i : (per_class > 0 ? per_class - 1 : 0)];
    }
}

// BOOLIN: the input is the bool matrix [batch, in_dim] itself (sample-major, as the user holds it) and is
// packed on the way into LDS, so neither the pack kernel nor the packed input exist: the workgroup reads
// the COLS * 64 sample rows of its columns (one contiguous region) and folds them into the input rows.
// THIN: the net thinned for this call (ThinTables): numbers of neurons from `thin`, no schedules.
template <int COLS, int GPT, int NP0, bool BOOLIN, bool THIN>
__global__ __launch_bounds__(DL_NET_THREADS) void eval_net_lds_kernel(const uint64_t *__restrict__ x,
                                                                      const uint8_t *__restrict__ xb,
                                                                      const uint32_t *__restrict__ rec, NetShape net,
                                                                      int32_t *__restrict__ out, int64_t ncols,
                                                                      int64_t per_class, int64_t k, int64_t batch,
                                                                      uint32_t grouped_blocks,
                                                                      const int32_t *__restrict__ thin) {
    extern __shared__ __align__(16) uint8_t act[];             // [rows][COLS] 64-bit words
    const int tid = (int) threadIdx.x;
    const int wave = dl_wave_in_block(), lane = dl_lane();

    // Packed input: workgroups are dealt round-robin to the 8 XCDs, each with an L2 of its own.  The
    // 16 / COLS workgroups whose columns share a 128-byte line of every input row are given to ONE XCD,
    // so a line is fetched into one L2 instead of eight (the blocks past the last whole group of
    // 8 * 16 / COLS keep their index).
    constexpr uint32_t SHARE = 16 / COLS;
    int64_t group = blockIdx.x;
    if (!BOOLIN && blockIdx.x < grouped_blocks) {
        const uint32_t xcd = blockIdx.x % 8, j = blockIdx.x / 8;
        group = ((j / SHARE) * 8 + xcd) * SHARE + j % SHARE;
    }
    const int64_t col0 = group * COLS;

    // records a thread needs for layer l, requested one layer ahead of their use
    constexpr int NR = THIN || GPT > DL_NET_CHUNK + 2 ? GPT : DL_NET_CHUNK + 2;
    const int rt = tid;
    auto load_records = [&](int l, uint32_t *r) __attribute__((always_inline)) {
        const uint32_t *tab = rec + net.offset[l];
        // scheduled: entry 8 tid + i sits at tab[i * stride + tid], i = 0..8, and the record of step 8192 + tid at
        // tab[9 * stride + tid]; else neuron tid + 1024 i at tab[tid + 1024 i]
        const bool sched = !THIN && net.steps[l] > 0;
        const int chunks = net.steps[l] / DL_NET_CHUNK;
        const int limit = sched ? (chunks < DL_NET_THREADS ? chunks : DL_NET_THREADS) : THIN ? thin[l] : net.width[l];
        const int extra = net.steps[l] - DL_NET_CHUNK * limit;
        const int step = sched ? net.stride[l] : DL_NET_THREADS;
        const int entries = sched ? DL_NET_CHUNK + 2 : GPT;
#pragma unroll
        for (int i = 0; i < NR; ++i) {
            // (threads and entries without work read entry 0 and compute on it; only their stores are skipped)
            const bool live = i < entries && (!sched ? rt + i * DL_NET_THREADS < limit
                                              : i <= DL_NET_CHUNK ? rt < limit : rt < extra);
            r[i] = tab[live ? rt + i * step : 0];
        }
    };
    // BOOLIN: packs group g's COLS * 64 samples of the bool input into the input rows.  A thread takes 16 features
    // x 8 samples at a time: eight 16-byte loads (a wave's loads of one sample row are contiguous), folded into one
    // register per 4 features (byte = feature, bit = sample), whose 16 bytes go to byte `oct` of the 16 features'
    // rows.  All of a workgroup's loads are in flight together.  Samples past the batch read as zero.
    auto stage_bool = [&](int64_t g, int t, int nthreads) __attribute__((always_inline)) {
        const int per_row = net.in_dim / 16;
        const int items = 8 * COLS * per_row;
        const int64_t s_base = g * (COLS * 64);
        for (int it = t; it < items; it += nthreads) {
            const int oct = it / per_row, c = it - oct * per_row;      // byte of the row, 16-feature chunk
            const int64_t s0 = s_base + 8 * oct;
            const uint8_t *src = xb + s0 * net.in_dim + 16 * c;
            dl_u32x4 v[8];
#pragma unroll
            for (int i = 0; i < 8; ++i)
                v[i] = s0 + i < batch ? __builtin_nontemporal_load(reinterpret_cast<const dl_u32x4 *>(src + (int64_t) i * net.in_dim))
                                      : dl_u32x4{0, 0, 0, 0};
            // bytes of a bool tensor are 0 or 1: then a shift and an OR per dword do; any other non-zero byte (a
            // uint8 tensor viewed as bool) counts as true as well and sends the item through the general form
            uint32_t acc[4], seen = 0;
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                acc[d] = 0;
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    acc[d] |= v[i][d] << i;
                    seen |= v[i][d];
                }
            }
            if (seen & 0xfefefefeu) {
#pragma unroll
                for (int d = 0; d < 4; ++d) {
                    acc[d] = 0;
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        const uint32_t u = v[i][d];
                        acc[d] |= (((((u & 0x7f7f7f7fu) + 0x7f7f7f7fu) | u) >> 7) & 0x01010101u) << i;
                    }
                }
            }
            // byte 4 d + kk of acc[] belongs to feature 16 c + 4 d + kk.  A wave's lanes hold consecutive chunks, whose
            // rows lie 256 bytes apart, i.e. on one bank: every lane therefore starts with another of its 16 features
            uint8_t *dst = act + ((size_t) net.in_base + 16 * c) * (8 * COLS) + oct;
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const int idx = (j + t) & 15;
                const uint32_t lo = (idx & 4) ? acc[1] : acc[0], hi = (idx & 4) ? acc[3] : acc[2];
                const uint32_t word = (idx & 8) ? hi : lo;
                dst[(size_t) idx * (8 * COLS)] = (uint8_t) (word >> (8 * (idx & 3)));
            }
        }
    };
    const uint32_t *ltab = rec + net.offset[net.depth - 1];
    uint32_t r[NR];
    if (net.depth > 1) load_records(0, r);
    // the class phase's first records (wave = class)
    // (thinned for this call: a class keeps `left` of its per_class records, and `base` constant ones count for every sample)
    auto class_left = [&](int64_t cls) -> int64_t { return THIN ? (int64_t) thin[net.depth - 1 + cls] : per_class; };
    uint32_t rc[4] = {0, 0, 0, 0};
    if (wave < k) load_class_records(rc, ltab + wave * per_class, lane, class_left(wave));

    if (BOOLIN) {
        stage_bool(group, tid, DL_NET_THREADS);
    } else {
        // the workgroup's word columns of the packed input; columns past the end read as zero
        for (int f = tid; f < net.in_dim; f += DL_NET_THREADS) {
            Row<COLS> v;
            if (COLS > 1 && col0 + COLS <= ncols && ncols % 2 == 0 && ((uintptr_t) x & 15) == 0) {   // whole, 16-byte aligned
                const dl_u32x4 *src = reinterpret_cast<const dl_u32x4 *>(x + (int64_t) f * ncols + col0);
#pragma unroll
                for (int q = 0; q < COLS / 2; ++q) {
                    const dl_u32x4 t = src[q];
                    v.d[4 * q] = t.x, v.d[4 * q + 1] = t.y, v.d[4 * q + 2] = t.z, v.d[4 * q + 3] = t.w;
                }
            } else {
#pragma unroll
                for (int j = 0; j < COLS; ++j) {
                    const uint64_t t = col0 + j < ncols ? x[(int64_t) f * ncols + col0 + j] : 0;
                    v.d[2 * j] = (uint32_t) t, v.d[2 * j + 1] = (uint32_t) (t >> 32);
                }
            }
            lds_store<COLS>(act, (uint32_t) f, v);
        }
    }
    __syncthreads();

    // Every layer but the last: act <- layer(act).  The hidden layers are bound by LDS throughput (bank
    // conflicts of the random row reads included) and, run in lock step between barriers by the one
    // workgroup a CU holds, by every latency that all threads wait out together: the next layer's
    // records are therefore requested before this layer's rows are read.
    for (int l = 0; l + 1 < net.depth; ++l) {
        uint32_t rn[NR];
        if (l + 2 < net.depth) load_records(l + 1, rn);
        if (!THIN && net.steps[l] > 0) {
            // along the schedule: this thread's chunk of 8 steps, 9 rows read, outputs in schedule order
            // (and, of a schedule of more than 1024 chunks, one of the remaining steps)
            const int stride = net.stride[l];
            const int nchunks = net.steps[l] / DL_NET_CHUNK < DL_NET_THREADS ? net.steps[l] / DL_NET_CHUNK : DL_NET_THREADS;
            const int extra = net.steps[l] - DL_NET_CHUNK * nchunks;
            Row<COLS> y[DL_NET_CHUNK], ye;
            if (extra > 0) ye = gate_rows<COLS>(act, r[DL_NET_CHUNK + 1]);
            Row<COLS> prev = lds_row<COLS>(act, r[0] & ((1u << DL_NET_ID_BITS) - 1));
#pragma unroll
            for (int j = 0; j < DL_NET_CHUNK; ++j) {
                const Row<COLS> cur = lds_row<COLS>(act, r[j + 1] & ((1u << DL_NET_ID_BITS) - 1));
                y[j] = gate_mix<COLS>(prev, cur, r[j + 1]);
                prev = cur;
            }
            __syncthreads();                                    // every thread has read its inputs
            if (tid < nchunks) {
#pragma unroll
                for (int j = 0; j < DL_NET_CHUNK; ++j) lds_store<COLS>(act, (uint32_t) (j * stride + tid), y[j]);
            }
            if (tid < extra)                                    // step 8192 + tid
                lds_store<COLS>(act, (uint32_t) ((tid % DL_NET_CHUNK) * stride + DL_NET_THREADS + tid / DL_NET_CHUNK), ye);
        } else {
            const int width = THIN ? thin[l] : net.width[l];    // (thinned: the neurons left, at rows 0, 1, ...)
            Row<COLS> y[GPT];
#pragma unroll
            for (int g = 0; g < GPT; ++g)
                if (!THIN || g * DL_NET_THREADS + wave * DL_WAVE < width) y[g] = gate_rows<COLS>(act, r[g]);   // (a wave skips rounds in which it has no neuron)
            __syncthreads();                                    // every thread has read its inputs
#pragma unroll
            for (int g = 0; g < GPT; ++g) {
                const int n = tid + g * DL_NET_THREADS;
                if (n < width) lds_store<COLS>(act, (uint32_t) n, y[g]);
            }
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < NR; ++i) r[i] = rn[i];
    }

    // last layer, one wave per class: evaluate, count bit-sliced per lane, sum the lanes
    for (int64_t cls = wave; cls < k; cls += DL_NET_THREADS / DL_WAVE) {
        uint32_t pl[2 * COLS][NP0 + 6];                          // [dword of the row][plane]
#pragma unroll
        for (int i = 0; i < 2 * COLS; ++i)
#pragma unroll
            for (int p = 0; p < NP0; ++p) pl[i][p] = 0;
        // Four neurons at a time: their records are requested an iteration ahead, their output words are
        // compressed by a carry-save tree into one word of weight 4 that ripples into the planes above.
        // What is left of the class after the whole quads (fewer than 256 neurons) goes row by row: 64 neurons,
        // lanes past the end of the class contributing zero words, rippled in with weight 1.
        const uint32_t *ctab = ltab + cls * per_class;
        const int64_t left = class_left(cls);
        const int32_t base = THIN ? thin[net.depth - 1 + k + cls] : 0;
        if (cls != wave) load_class_records(rc, ctab, lane, left);
        const int64_t quads = left / (4 * DL_WAVE);
        for (int64_t q = 0; q < quads; ++q) {
            uint32_t r4[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) r4[u] = rc[u];
            load_class_records(rc, ctab, (q + 1) * 4 * DL_WAVE + lane, left);   // next quad, or the rest
            Row<COLS> y[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) y[u] = gate_rows<COLS>(act, r4[u]);
#pragma unroll
            for (int i = 0; i < 2 * COLS; ++i) {
                uint32_t t2a, t2b, carry;
                csa32(t2a, pl[i][0], pl[i][0], y[0].d[i], y[1].d[i]);
                csa32(t2b, pl[i][0], pl[i][0], y[2].d[i], y[3].d[i]);
                csa32(carry, pl[i][1], pl[i][1], t2a, t2b);
#pragma unroll
                for (int p = 2; p < NP0; ++p) half_add32(pl[i][p], carry);   // counter += carry * 4
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int64_t i = (quads * 4 + u) * DL_WAVE;          // first neuron of this row
            if (i >= left) break;                                 // uniform
            Row<COLS> y = gate_rows<COLS>(act, rc[u]);
            const uint32_t live = i + lane < left ? ~0u : 0u;
#pragma unroll
            for (int d = 0; d < 2 * COLS; ++d) {
                uint32_t carry = y.d[d] & live;
#pragma unroll
                for (int p = 0; p < NP0; ++p) {                  // counter += word
                    const uint32_t old = pl[d][p];
                    pl[d][p] = old ^ carry;
                    carry = old & carry;
                }
            }
        }
        int32_t count[COLS];
        lanes_count<COLS, NP0>(pl, lane, count);
#pragma unroll
        for (int t = 0; t < COLS; ++t) {
            const int64_t sample = col0 * 64 + lane * COLS + t;
            if (sample < batch && sample < ncols * 64) out[sample * k + cls] = count[t] + base;
        }
    }
}

template <int COLS, int GPT>
int launch_net(const void *x, bool bool_input, const uint32_t *rec, const NetShape &net, int32_t *out, int64_t ncols,
               int64_t per_class, int64_t k, int64_t batch, int64_t rows, const int32_t *thin, hipStream_t s) {
    const int64_t groups = dl_ceil_div(ncols, COLS);
    if (groups > 0x7fffffffLL) return DL_ERR_TOO_LARGE;
    const size_t lds = (size_t) rows * 8 * COLS;
    const dim3 block(DL_NET_THREADS);
    // a lane counts ceil(per_class / 64) neurons: NP0 planes hold up to 2^NP0 - 1
    const bool small = dl_ceil_div(per_class, DL_WAVE) < 16;
    const dim3 grid((unsigned) groups);
    const uint32_t share = 8 * (16 / COLS);                    // workgroups sharing input lines, one set per XCD
    const uint32_t grouped = bool_input ? 0u : (uint32_t) groups / share * share;
    const uint64_t *words = bool_input ? nullptr : (const uint64_t *) x;
    const uint8_t *bools = bool_input ? (const uint8_t *) x : nullptr;
#define DL_NET_LAUNCH(NP0, BOOLIN, THIN)                                                                                \
    DL_LAUNCH((eval_net_lds_kernel<COLS, GPT, NP0, BOOLIN, THIN>), grid, block, lds, s, words, bools, rec, net, out, ncols,    \
              per_class, k, batch, grouped, thin)
    if (bool_input) {
        if (thin) { if (small) DL_NET_LAUNCH(4, true, true); else DL_NET_LAUNCH(8, true, true); }
        else { if (small) DL_NET_LAUNCH(4, true, false); else DL_NET_LAUNCH(8, true, false); }
    } else {
        if (thin) { if (small) DL_NET_LAUNCH(4, false, true); else DL_NET_LAUNCH(8, false, true); }
        else { if (small) DL_NET_LAUNCH(4, false, false); else DL_NET_LAUNCH(8, false, false); }
    }
#undef DL_NET_LAUNCH
    return dl_launch_status();
}

bool net_shape_ok(int depth, const int64_t *dims, int64_t k) {
    if (depth < 1 || depth > DL_NET_MAX_DEPTH || !dims || k <= 0) return false;
    for (int l = 0; l <= depth; ++l)
        if (dims[l] <= 0 || dims[l] > DL_NET_MAX_WIDTH) return false;
    return dims[depth] % k == 0;
}

}  // namespace

extern "C" int64_t dl_logic_net_lds_max_width(void) { return DL_NET_MAX_WIDTH; }

extern "C" int64_t dl_logic_net_lds_workspace_bytes(int depth, const int64_t *dims) {
    if (depth < 1 || depth > DL_NET_MAX_DEPTH || !dims) return 0;
    // per layer: the records (9 per chunk of a schedule of at most width + width / 4 + 32 steps, chunks
    // rounded up to whole waves) and width row ids
    // (thinned: a record, a rank, a folded gate id and a mark per neuron = 10 bytes, and three numbers per layer /
    // class: fits the same bound with the last term, k <= dims[depth])
    int64_t bytes = 0;
    for (int l = 1; l <= depth; ++l) {
        const int64_t w = dims[l] > 0 ? dims[l] : 0;
        bytes += 4 * (w + w / 2 + 640 + DL_NET_THREADS) + 4 * w;
    }
    return bytes + 8 * (dims[depth] > 0 ? dims[depth] : 0);
}

// bool_input: x is the bool matrix [batch, dims[0]] (sample-major); words, bit_count and pad_len are then unused.
// thinned: the net thinned for this call (see ThinTables); the schedules are not used then.
static int net_lds_run(const void *x, bool bool_input, int64_t batch, int depth, const int64_t *const *a,
                       const int64_t *const *b, const uint8_t *const *w, const int64_t *dims, const int32_t *const *verts,
                       const int32_t *const *neuron, const uint8_t *const *flip, const int64_t *steps, int32_t *out,
                       int64_t words, int bit_count, int64_t pad_len, int64_t k, void *workspace, void *stream,
                       bool thinned = false, bool folded = false) {
    if (!bool_input && bit_count != 8 && bit_count != 16 && bit_count != 32 && bit_count != 64) return DL_ERR_BIT_COUNT;
    if (depth < 1 || !dims || !a || !b || !w || words < 0 || k <= 0 || pad_len < 0) return DL_ERR_INVALID_ARGUMENT;
    if (depth > DL_NET_MAX_DEPTH) return DL_ERR_TOO_LARGE;
    for (int l = 0; l <= depth; ++l)
        if (dims[l] <= 0) return DL_ERR_INVALID_ARGUMENT;
    if (dims[depth] % k != 0) return DL_ERR_NOT_DIVISIBLE;
    if (!bool_input) batch = words * bit_count - pad_len;
    if (batch < 0) return DL_ERR_INVALID_ARGUMENT;
    if (batch == 0) return DL_OK;
    if (!x || !out || !workspace) return DL_ERR_INVALID_ARGUMENT;
    const int64_t row_bytes = bool_input ? dl_ceil_div(batch, 64) * 8 : words * (bit_count / 8);
    // rows of whole 64-bit words and layers that fit the LDS buffer; otherwise the caller runs the streaming kernels
    if (!net_shape_ok(depth, dims, k) || row_bytes % 8 != 0 || !dl_aligned(x, 8) || !dl_aligned(workspace, 4))
        return DL_ERR_TOO_LARGE;
    // the bool input is read in 16-byte pieces of a sample row
    if (bool_input && (dims[0] % 16 != 0 || !dl_aligned(x, 16))) return DL_ERR_TOO_LARGE;
    hipStream_t s = (hipStream_t) stream;

    // The widest hidden layer (or the input) decides the columns per workgroup: rows * 8 * COLS bytes of LDS, and a
    // thread holds the outputs of ceil(width / 1024) neurons in registers.  A packed input occupies the rows the
    // first layer then overwrites; a bool input has rows of its own behind those of the hidden layers, because it is
    // filled for the next group of columns while this one is still being counted.
    const int64_t input_rows = bool_input ? dims[0] : 0;
    int64_t rows = bool_input ? 0 : dims[0], hidden = 0;
    for (int l = 0; l + 1 < depth; ++l) {
        if (dims[l + 1] > hidden) hidden = dims[l + 1];
        if (dims[l + 1] > rows) rows = dims[l + 1];              // the last layer's output is never stored
    }
    if (rows + input_rows > DL_NET_MAX_WIDTH) return DL_ERR_TOO_LARGE;
    const bool four = rows + input_rows <= DL_NET_MAX_WIDTH / 2 && hidden <= 5 * DL_NET_THREADS;
    const int64_t capacity = (four ? DL_NET_MAX_WIDTH / 2 : DL_NET_MAX_WIDTH) - input_rows;   // rows of the layers

    NetWiring wiring;
    NetShape net;
    net.depth = depth;
    net.in_dim = (int32_t) dims[0];
    net.in_base = wiring.in_base = 0;
    int64_t entries = 0, offset = 0, most_steps = 0;
    char *pos_base = nullptr;
    for (int l = 0; l < DL_NET_MAX_DEPTH; ++l) {
        wiring.a[l] = wiring.b[l] = nullptr, wiring.w[l] = nullptr;
        wiring.verts[l] = wiring.neuron[l] = nullptr, wiring.flip[l] = nullptr, wiring.pos[l] = nullptr;
        wiring.width[l] = wiring.offset[l] = wiring.steps[l] = wiring.stride[l] = 0;
        net.width[l] = net.offset[l] = net.steps[l] = net.stride[l] = 0;
    }
    for (int l = 0; l < depth; ++l) {
        if (!a[l] || !b[l] || !w[l]) return DL_ERR_INVALID_ARGUMENT;
        wiring.a[l] = a[l], wiring.b[l] = b[l], wiring.w[l] = w[l];
        wiring.width[l] = net.width[l] = (int32_t) dims[l + 1];
        wiring.offset[l] = net.offset[l] = (int32_t) offset;
        int64_t count = dims[l + 1];
        // A hidden layer is walked along its schedule when one is given, every chunk finds a thread, its outputs in
        // schedule order fit the buffer, and the schedule is not much longer than the layer (few, long trails).
        if (!thinned && l + 1 < depth && steps && verts && neuron && flip && verts[l] && neuron[l] && flip[l] &&
            steps[l] >= dims[l + 1] && steps[l] % DL_NET_CHUNK == 0) {
            const int64_t nchunks = steps[l] / DL_NET_CHUNK;
            const int64_t stride = dl_ceil_div(nchunks, DL_WAVE) * DL_WAVE;
            const int64_t extra = steps[l] > DL_NET_CHUNK * DL_NET_THREADS ? steps[l] - DL_NET_CHUNK * DL_NET_THREADS : 0;
            if (extra <= DL_NET_THREADS && DL_NET_CHUNK * stride <= capacity && steps[l] <= dims[l + 1] + dims[l + 1] / 4 + 32) {
                wiring.verts[l] = verts[l], wiring.neuron[l] = neuron[l], wiring.flip[l] = flip[l];
                wiring.steps[l] = net.steps[l] = (int32_t) steps[l];
                wiring.stride[l] = net.stride[l] = (int32_t) stride;
                count = (DL_NET_CHUNK + 1) * stride + extra;
                if (DL_NET_CHUNK * stride > rows) rows = DL_NET_CHUNK * stride;
                if (steps[l] > most_steps) most_steps = steps[l];
            }
        }
        offset += count;
        if (count > entries) entries = count;
    }
    uint32_t *rec = (uint32_t *) workspace;
    int32_t *pos = (int32_t *) workspace + offset;               // row ids of the scheduled layers follow the records
    for (int l = 0; l + 1 < depth; ++l) {
        if (wiring.steps[l] > 0) {
            wiring.pos[l] = pos;
            pos += dims[l + 1];
        }
    }
    (void) pos_base;
    if ((char *) pos - (char *) workspace > dl_logic_net_lds_workspace_bytes(depth, dims)) return DL_ERR_INVALID_ARGUMENT;
    if (most_steps > 0) {
        DL_LAUNCH(compose_net_pos_kernel, dim3((unsigned) dl_ceil_div(most_steps, DL_BLOCK), (unsigned) (depth - 1)),
                  dim3(DL_BLOCK), 0, s, wiring);
        const int st = dl_launch_status();
        if (st != DL_OK) return st;
    }
    net.in_base = wiring.in_base = (int32_t) (bool_input ? rows : 0);      // the input's rows follow the layers'
    const int32_t *thin = nullptr;
    int st;
    if (thinned) {
        // ranks follow the records, then the numbers of neurons left, the folded gate ids and the marks
        ThinTables th;
        int32_t *rank = (int32_t *) workspace + offset;
        for (int l = 0; l < DL_NET_MAX_DEPTH; ++l) th.folded[l] = th.live[l] = nullptr, th.rank[l] = nullptr;
        for (int l = 0; l < depth; ++l) {
            th.rank[l] = rank;
            rank += dims[l + 1];
        }
        th.thin = rank;
        th.k = (int32_t) k;
        uint8_t *bytes = (uint8_t *) (rank + depth + 2 * k);
        uint8_t *marks = bytes;                                  // the hidden layers' marks, one after the other
        int64_t nmarks = 0;
        for (int l = 0; l + 1 < depth; ++l) th.live[l] = bytes, bytes += dims[l + 1], nmarks += dims[l + 1];
        for (int l = 0; l < depth; ++l) {
            // (folded already: the caller's gate ids are read where the folded ones would be; nothing writes them)
            if (folded) th.folded[l] = const_cast<uint8_t *>(w[l]);
            else th.folded[l] = bytes, bytes += dims[l + 1];
        }
        if ((char *) bytes - (char *) workspace > dl_logic_net_lds_workspace_bytes(depth, dims)) return DL_ERR_INVALID_ARGUMENT;
        if (folded) {
            if (nmarks > 0) DL_LAUNCH(net_thin_clear_kernel, dim3((unsigned) dl_ceil_div(nmarks, DL_BLOCK)), dim3(DL_BLOCK), 0, s, marks, nmarks);
        } else {
            for (int l = 0; l < depth; ++l)
                DL_LAUNCH(net_thin_fold_kernel, dim3((unsigned) dl_ceil_div(dims[l + 1], DL_BLOCK)), dim3(DL_BLOCK), 0, s, wiring, th,
                          l, depth);
        }
        for (int l = depth - 1; l >= 1; --l)
            DL_LAUNCH(net_thin_mark_kernel, dim3((unsigned) dl_ceil_div(dims[l + 1], DL_BLOCK)), dim3(DL_BLOCK), 0, s, wiring, th, l,
                      depth);
        DL_LAUNCH(net_thin_rank_kernel, dim3((unsigned) depth), dim3(DL_NET_THREADS), 0, s, wiring, th, depth);
        st = dl_launch_status();
        if (st != DL_OK) return st;
        DL_LAUNCH(compose_net_thin_kernel, dim3((unsigned) dl_ceil_div(entries, DL_BLOCK), (unsigned) depth), dim3(DL_BLOCK), 0, s,
                  wiring, th, depth, rec);
        thin = th.thin;
    } else {
        DL_LAUNCH(compose_net_kernel, dim3((unsigned) dl_ceil_div(entries, DL_BLOCK), (unsigned) depth), dim3(DL_BLOCK), 0, s,
                  wiring, rec);
    }
    st = dl_launch_status();
    if (st != DL_OK) return st;

    const int64_t ncols = row_bytes / 8;
    const int64_t per_class = dims[depth] / k;
    if (four) return launch_net<4, 5>(x, bool_input, rec, net, out, ncols, per_class, k, batch, rows + input_rows, thin, s);
    return launch_net<2, 10>(x, bool_input, rec, net, out, ncols, per_class, k, batch, rows + input_rows, thin, s);
}

extern "C" int dl_logic_net_lds_groupbitsum(const void *x, int depth, const int64_t *const *a, const int64_t *const *b,
                                            const uint8_t *const *w, const int64_t *dims, int32_t *out, int64_t words,
                                            int bit_count, int64_t pad_len, int64_t k, void *workspace, void *stream) {
    return net_lds_run(x, false, 0, depth, a, b, w, dims, nullptr, nullptr, nullptr, nullptr, out, words, bit_count, pad_len,
                       k, workspace, stream);
}

extern "C" int dl_logic_net_lds_groupbitsum_scheduled(const void *x, int depth, const int64_t *const *a,
                                                      const int64_t *const *b, const uint8_t *const *w,
                                                      const int64_t *dims, const int32_t *const *verts,
                                                      const int32_t *const *neuron, const uint8_t *const *flip,
                                                      const int64_t *steps, int32_t *out, int64_t words, int bit_count,
                                                      int64_t pad_len, int64_t k, void *workspace, void *stream) {
    return net_lds_run(x, false, 0, depth, a, b, w, dims, verts, neuron, flip, steps, out, words, bit_count, pad_len, k,
                       workspace, stream);
}

extern "C" int dl_logic_net_lds_groupbitsum_thinned(const void *x, int bool_input, int64_t batch, int depth,
                                                    const int64_t *const *a, const int64_t *const *b,
                                                    const uint8_t *const *w, int folded, const int64_t *dims, int32_t *out,
                                                    int64_t words, int bit_count, int64_t pad_len, int64_t k,
                                                    void *workspace, void *stream) {
    if (batch < 0) return DL_ERR_INVALID_ARGUMENT;
    return net_lds_run(x, bool_input != 0, batch, depth, a, b, w, dims, nullptr, nullptr, nullptr, nullptr, out,
                       bool_input ? 0 : words, bool_input ? 64 : bit_count, bool_input ? 0 : pad_len, k, workspace, stream,
                       true, folded != 0);
}

extern "C" int dl_logic_net_lds_groupbitsum_bool(const uint8_t *x, int64_t batch, int depth, const int64_t *const *a,
                                                 const int64_t *const *b, const uint8_t *const *w, const int64_t *dims,
                                                 const int32_t *const *verts, const int32_t *const *neuron,
                                                 const uint8_t *const *flip, const int64_t *steps, int32_t *out,
                                                 int64_t k, void *workspace, void *stream) {
    if (batch < 0) return DL_ERR_INVALID_ARGUMENT;
    return net_lds_run(x, true, batch, depth, a, b, w, dims, verts, neuron, flip, steps, out, 0, 64, 0, k, workspace,
                       stream);
}
