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
// holds the count of sample s.
//
// The wiring is read from a compact table built per call (one 32-bit record per gate: two
// 14-bit row ids and the 4-bit gate id), which every workgroup streams from L2.
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
    int32_t width[DL_NET_MAX_DEPTH];    // neurons of layer l
    int32_t offset[DL_NET_MAX_DEPTH];   // first record of layer l
};

struct NetShape {
    int32_t depth, in_dim;
    int32_t width[DL_NET_MAX_DEPTH];
    int32_t offset[DL_NET_MAX_DEPTH];
};

// record of neuron n of layer blockIdx.y: a | b << 14 | gate << 28
__global__ __launch_bounds__(DL_BLOCK) void compose_net_kernel(NetWiring t, uint32_t *__restrict__ rec) {
    const int l = blockIdx.y;
    const int n = (int) (blockIdx.x * DL_BLOCK + threadIdx.x);
    if (n >= t.width[l]) return;
    const uint32_t a = (uint32_t) t.a[l][n], b = (uint32_t) t.b[l][n], op = t.w[l][n] & 15u;
    rec[t.offset[l] + n] = a | (b << DL_NET_ID_BITS) | (op << (2 * DL_NET_ID_BITS));
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

// gate id = truth table (f(0,0) f(0,1) f(1,0) f(1,1)), MSB first; masks are per lane here
template <int COLS>
__device__ __forceinline__ Row<COLS> gate_rows(const void *act, uint32_t rec) {
    const uint32_t ia = rec & ((1u << DL_NET_ID_BITS) - 1), ib = (rec >> DL_NET_ID_BITS) & ((1u << DL_NET_ID_BITS) - 1);
    const uint32_t m00 = 0u - ((rec >> 31) & 1u), m01 = 0u - ((rec >> 30) & 1u);
    const uint32_t m10 = 0u - ((rec >> 29) & 1u), m11 = 0u - ((rec >> 28) & 1u);
    const Row<COLS> a = lds_row<COLS>(act, ia), b = lds_row<COLS>(act, ib);
    Row<COLS> y;
#pragma unroll
    for (int i = 0; i < 2 * COLS; ++i) {
        const uint32_t hi = (b.d[i] & m11) | (~b.d[i] & m10);
        const uint32_t lo = (b.d[i] & m01) | (~b.d[i] & m00);
        y.d[i] = (a.d[i] & hi) | (~a.d[i] & lo);
    }
    return y;
}

// carry-save adder on dwords: a + b + c = 2 * carry + sum, bit by bit
__device__ __forceinline__ void csa32(uint32_t &carry, uint32_t &sum, uint32_t a, uint32_t b, uint32_t c) {
    const uint32_t u = a ^ b;
    carry = (a & b) | (u & c);
    sum = u ^ c;
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

// One exchange of the butterfly: lanes l and l ^ (1 << J) each hold counters for the same set of
// sample bits (those selected by the earlier exchanges); the lane whose bit J is set keeps the
// samples whose index has bit J set (dword positions `upper`), its partner the others, and each
// adds the partner's counters for the samples it keeps.
template <int NP, int J> __device__ __forceinline__ void butterfly(uint32_t *q, int lane) {
    constexpr uint32_t upper = J == 4 ? 0xffff0000u : J == 3 ? 0xff00ff00u : J == 2 ? 0xf0f0f0f0u
                             : J == 1 ? 0xccccccccu : 0xaaaaaaaau;
    const uint32_t keep = ((lane >> J) & 1) ? upper : ~upper;
    uint32_t other[NP];
#pragma unroll
    for (int p = 0; p < NP; ++p) {
        other[p] = (uint32_t) __shfl_xor((int) q[p], 1 << J, DL_WAVE) & keep;
        q[p] &= keep;
    }
    planes_add<NP>(q, other);
}

// Sums the 64 lanes' bit-sliced counters (NP0 planes of 64 sample bits: lo = samples 0..31,
// hi = samples 32..63) and returns, in lane s, the count of sample s.
template <int NP0> __device__ __forceinline__ int32_t lanes_count(const uint32_t *lo, const uint32_t *hi, int lane) {
    uint32_t q[NP0 + 6], other[NP0];
    const bool upper_half = (lane & 32) != 0;          // this lane keeps samples 32..63
#pragma unroll
    for (int p = 0; p < NP0; ++p) {
        q[p] = upper_half ? hi[p] : lo[p];
        other[p] = (uint32_t) __shfl_xor((int) (upper_half ? lo[p] : hi[p]), 32, DL_WAVE);
    }
    planes_add<NP0>(q, other);
    butterfly<NP0 + 1, 4>(q, lane);
    butterfly<NP0 + 2, 3>(q, lane);
    butterfly<NP0 + 3, 2>(q, lane);
    butterfly<NP0 + 4, 1>(q, lane);
    butterfly<NP0 + 5, 0>(q, lane);
    int32_t count = 0;
#pragma unroll
    for (int p = 0; p < NP0 + 6; ++p) count |= (int32_t) ((q[p] >> (lane & 31)) & 1u) << p;
    return count;
}

template <int COLS, int GPT, int NP0>
__global__ __launch_bounds__(DL_NET_THREADS) void eval_net_lds_kernel(const uint64_t *__restrict__ x,
                                                                      const uint32_t *__restrict__ rec, NetShape net,
                                                                      int32_t *__restrict__ out, int64_t ncols,
                                                                      int64_t per_class, int64_t k, int64_t batch) {
    extern __shared__ __align__(16) uint8_t act[];             // [rows][COLS] 64-bit words
    const int tid = (int) threadIdx.x;
    const int64_t col0 = (int64_t) blockIdx.x * COLS;

    // the workgroup's word columns of the packed input; columns past the end read as zero
    for (int f = tid; f < net.in_dim; f += DL_NET_THREADS) {
        Row<COLS> r;
#pragma unroll
        for (int j = 0; j < COLS; ++j) {
            const uint64_t v = col0 + j < ncols ? x[(int64_t) f * ncols + col0 + j] : 0;
            r.d[2 * j] = (uint32_t) v, r.d[2 * j + 1] = (uint32_t) (v >> 32);
        }
        lds_store<COLS>(act, (uint32_t) f, r);
    }
    __syncthreads();

    // every layer but the last: act <- layer(act).  The records of the next layer are requested
    // before this layer's barrier, so their latency overlaps the exchange through LDS.
    // every layer but the last: act <- layer(act).  (Measured: the hidden layers are bound by LDS
    // throughput, bank conflicts of the random row reads included, not by its latency: putting all
    // of a thread's reads in flight together is no faster than this gate-by-gate form.)
    for (int l = 0; l + 1 < net.depth; ++l) {
        const uint32_t *tab = rec + net.offset[l];
        const int width = net.width[l];
        uint32_t r[GPT];
#pragma unroll
        for (int g = 0; g < GPT; ++g) {
            const int n = tid + g * DL_NET_THREADS;
            r[g] = n < width ? tab[n] : 0u;
        }
        Row<COLS> y[GPT];
#pragma unroll
        for (int g = 0; g < GPT; ++g)
            if (tid + g * DL_NET_THREADS < width) y[g] = gate_rows<COLS>(act, r[g]);
        __syncthreads();                                        // every thread has read its inputs
#pragma unroll
        for (int g = 0; g < GPT; ++g) {
            const int n = tid + g * DL_NET_THREADS;
            if (n < width) lds_store<COLS>(act, (uint32_t) n, y[g]);
        }
        __syncthreads();
    }

    // last layer, one wave per class: evaluate, count bit-sliced per lane, sum the lanes
    const int wave = dl_wave_in_block(), lane = dl_lane();
    const uint32_t *tab = rec + net.offset[net.depth - 1];
    for (int64_t cls = wave; cls < k; cls += DL_NET_THREADS / DL_WAVE) {
        uint32_t pl[2 * COLS][NP0];                              // [dword of the row][plane]
#pragma unroll
        for (int i = 0; i < 2 * COLS; ++i)
#pragma unroll
            for (int p = 0; p < NP0; ++p) pl[i][p] = 0;
        // four neurons at a time: their records are requested together, their output words are
        // compressed by a carry-save tree into one word of weight 4 that ripples into the planes
        // above; neurons past the end of the class contribute zero words
        const uint32_t *ctab = tab + cls * per_class;
        for (int64_t i0 = lane; i0 < per_class; i0 += 4 * DL_WAVE) {
            uint32_t r4[4], live[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int64_t i = i0 + u * DL_WAVE;
                live[u] = i < per_class ? ~0u : 0u;
                r4[u] = ctab[i < per_class ? i : per_class - 1];
            }
            Row<COLS> y[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                y[u] = gate_rows<COLS>(act, r4[u]);
#pragma unroll
                for (int i = 0; i < 2 * COLS; ++i) y[u].d[i] &= live[u];
            }
#pragma unroll
            for (int i = 0; i < 2 * COLS; ++i) {
                uint32_t t2a, t2b, carry;
                csa32(t2a, pl[i][0], pl[i][0], y[0].d[i], y[1].d[i]);
                csa32(t2b, pl[i][0], pl[i][0], y[2].d[i], y[3].d[i]);
                csa32(carry, pl[i][1], pl[i][1], t2a, t2b);
#pragma unroll
                for (int p = 2; p < NP0; ++p) {                  // counter += carry * 4
                    const uint32_t old = pl[i][p];
                    pl[i][p] = old ^ carry;
                    carry = old & carry;
                }
            }
        }
#pragma unroll
        for (int j = 0; j < COLS; ++j) {
            const int32_t count = lanes_count<NP0>(pl[2 * j], pl[2 * j + 1], lane);
            const int64_t sample = (col0 + j) * 64 + lane;
            if (col0 + j < ncols && sample < batch) out[sample * k + cls] = count;
        }
    }
}

template <int COLS, int GPT>
int launch_net(const void *x, const uint32_t *rec, const NetShape &net, int32_t *out, int64_t ncols, int64_t per_class,
               int64_t k, int64_t batch, int64_t rows, hipStream_t s) {
    const int64_t blocks = dl_ceil_div(ncols, COLS);
    if (blocks > 0x7fffffffLL) return DL_ERR_TOO_LARGE;
    const size_t lds = (size_t) rows * 8 * COLS;
    const dim3 grid((unsigned) blocks), block(DL_NET_THREADS);
    // a lane counts ceil(per_class / 64) neurons: NP0 planes hold up to 2^NP0 - 1
    if (dl_ceil_div(per_class, DL_WAVE) < 16)
        DL_LAUNCH((eval_net_lds_kernel<COLS, GPT, 4>), grid, block, lds, s, (const uint64_t *) x, rec, net, out, ncols,
                  per_class, k, batch);
    else
        DL_LAUNCH((eval_net_lds_kernel<COLS, GPT, 8>), grid, block, lds, s, (const uint64_t *) x, rec, net, out, ncols,
                  per_class, k, batch);
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
    int64_t gates = 0;
    for (int l = 1; l <= depth; ++l) gates += dims[l] > 0 ? dims[l] : 0;
    return 4 * gates;
}

extern "C" int dl_logic_net_lds_groupbitsum(const void *x, int depth, const int64_t *const *a, const int64_t *const *b,
                                            const uint8_t *const *w, const int64_t *dims, int32_t *out, int64_t words,
                                            int bit_count, int64_t pad_len, int64_t k, void *workspace, void *stream) {
    if (bit_count != 8 && bit_count != 16 && bit_count != 32 && bit_count != 64) return DL_ERR_BIT_COUNT;
    if (depth < 1 || !dims || !a || !b || !w || words < 0 || k <= 0 || pad_len < 0) return DL_ERR_INVALID_ARGUMENT;
    if (depth > DL_NET_MAX_DEPTH) return DL_ERR_TOO_LARGE;
    for (int l = 0; l <= depth; ++l)
        if (dims[l] <= 0) return DL_ERR_INVALID_ARGUMENT;
    if (dims[depth] % k != 0) return DL_ERR_NOT_DIVISIBLE;
    const int64_t batch = words * bit_count - pad_len;
    if (batch < 0) return DL_ERR_INVALID_ARGUMENT;
    if (batch == 0) return DL_OK;
    if (!x || !out || !workspace) return DL_ERR_INVALID_ARGUMENT;
    const int64_t row_bytes = words * (bit_count / 8);
    // rows of whole 64-bit words and layers that fit the LDS buffer; otherwise the caller runs the streaming kernels
    if (!net_shape_ok(depth, dims, k) || row_bytes % 8 != 0 || !dl_aligned(x, 8) || !dl_aligned(workspace, 4))
        return DL_ERR_TOO_LARGE;
    hipStream_t s = (hipStream_t) stream;

    NetWiring wiring;
    NetShape net;
    net.depth = depth;
    net.in_dim = (int32_t) dims[0];
    int64_t rows = dims[0], widest = 0, offset = 0;
    for (int l = 0; l < depth; ++l) {
        if (!a[l] || !b[l] || !w[l]) return DL_ERR_INVALID_ARGUMENT;
        wiring.a[l] = a[l], wiring.b[l] = b[l], wiring.w[l] = w[l];
        wiring.width[l] = net.width[l] = (int32_t) dims[l + 1];
        wiring.offset[l] = net.offset[l] = (int32_t) offset;
        offset += dims[l + 1];
        if (dims[l + 1] > widest) widest = dims[l + 1];
        if (l + 1 < depth && dims[l + 1] > rows) rows = dims[l + 1];     // the last layer's output is never stored
    }
    for (int l = depth; l < DL_NET_MAX_DEPTH; ++l) {
        wiring.a[l] = wiring.b[l] = nullptr, wiring.w[l] = nullptr;
        wiring.width[l] = wiring.offset[l] = net.width[l] = net.offset[l] = 0;
    }
    uint32_t *rec = (uint32_t *) workspace;
    DL_LAUNCH(compose_net_kernel, dim3((unsigned) dl_ceil_div(widest, DL_BLOCK), (unsigned) depth), dim3(DL_BLOCK), 0, s,
              wiring, rec);
    int st = dl_launch_status();
    if (st != DL_OK) return st;

    const int64_t ncols = row_bytes / 8;
    const int64_t per_class = dims[depth] / k;
    // widest hidden layer (or input) decides the columns per workgroup: rows * 8 * COLS bytes of LDS, and a thread
    // holds the outputs of ceil(width / 1024) neurons in registers
    int64_t hidden = 0;
    for (int l = 0; l + 1 < depth; ++l)
        if (dims[l + 1] > hidden) hidden = dims[l + 1];
    if (rows <= DL_NET_MAX_WIDTH / 2 && hidden <= 5 * DL_NET_THREADS)
        return launch_net<4, 5>(x, rec, net, out, ncols, per_class, k, batch, rows, s);
    return launch_net<2, 10>(x, rec, net, out, ncols, per_class, k, batch, rows, s);
}
