// Host-side construction of the evaluation schedule used by dl_logic_eval_chained.
//
// The top layer of a fused group is a multigraph: its inputs (the neurons of the layer below,
// or the input rows for a single layer) are vertices, every top-layer neuron is an edge between
// the two vertices it reads.  Walking the edges along trails (each edge shares a vertex with the
// one before it) lets the kernel keep the shared vertex's value in registers, so a neuron costs
// ONE newly evaluated input instead of two.  For the reference's balanced 'random' wiring of a
// square layer every vertex has degree 2 and the graph is a handful of cycles, i.e. of trails.
//
// Schedule = a sequence of steps.  Step s evaluates vertex verts[s + 1]; if neuron[s] >= 0 it
// also evaluates that top-layer neuron from (previous vertex, new vertex) = (verts[s], verts[s+1]),
// with flip[s] = 1 when the previous vertex is the neuron's `b` input rather than its `a` input.
// neuron[s] = -1 marks a load-only step (start of a trail, or padding to whole chunks).
#include <stdint.h>

#include <algorithm>
#include <vector>

#include "count_chain.h"
#include "difflogic_hip.h"

extern "C" int64_t dl_eval_schedule_capacity(int64_t out_dim, int chunk) {
    if (out_dim < 0 || chunk <= 0) return -DL_ERR_INVALID_ARGUMENT;
    return 2 * out_dim + 2 * (int64_t) chunk;     // at most one load-only step per neuron, plus padding
}

extern "C" int64_t dl_eval_schedule_build(const int64_t *a, const int64_t *b, int64_t in_dim, int64_t out_dim,
                                          int chunk, int32_t *verts, int32_t *neuron, uint8_t *flip) {
    if (!a || !b || !verts || !neuron || !flip || in_dim <= 0 || out_dim < 0 || chunk <= 0)
        return -DL_ERR_INVALID_ARGUMENT;
    if (in_dim > 0x7fffffffLL || out_dim > 0x3fffffffLL) return -DL_ERR_TOO_LARGE;
    for (int64_t n = 0; n < out_dim; ++n)
        if (a[n] < 0 || a[n] >= in_dim || b[n] < 0 || b[n] >= in_dim) return -DL_ERR_INVALID_ARGUMENT;

    // adjacency in CSR form; a self-loop is listed twice under its vertex
    std::vector<int64_t> start((size_t) in_dim + 1, 0);
    for (int64_t n = 0; n < out_dim; ++n) {
        ++start[(size_t) a[n] + 1];
        ++start[(size_t) b[n] + 1];
    }
    for (int64_t v = 0; v < in_dim; ++v) start[(size_t) v + 1] += start[(size_t) v];
    std::vector<int32_t> adj((size_t) (2 * out_dim));
    {
        std::vector<int64_t> fill(start.begin(), start.end() - 1);
        for (int64_t n = 0; n < out_dim; ++n) {
            adj[(size_t) fill[(size_t) a[n]]++] = (int32_t) n;
            adj[(size_t) fill[(size_t) b[n]]++] = (int32_t) n;
        }
    }
    std::vector<int64_t> next(start.begin(), start.end() - 1);   // next adjacency slot to examine
    std::vector<uint8_t> used((size_t) out_dim, 0);

    int64_t steps = 0;
    verts[0] = 0;
    auto walk_from = [&](int64_t v0) {
        for (;;) {   // several trails may have to start at v0
            int64_t &p0 = next[(size_t) v0];
            while (p0 < start[(size_t) v0 + 1] && used[(size_t) adj[(size_t) p0]]) ++p0;
            if (p0 >= start[(size_t) v0 + 1]) return;
            verts[steps + 1] = (int32_t) v0;         // load-only step: the trail's first vertex
            neuron[steps] = -1;
            flip[steps] = 0;
            ++steps;
            int64_t cur = v0;
            for (;;) {
                int64_t &p = next[(size_t) cur];
                while (p < start[(size_t) cur + 1] && used[(size_t) adj[(size_t) p]]) ++p;
                if (p >= start[(size_t) cur + 1]) break;
                const int32_t e = adj[(size_t) p++];
                used[(size_t) e] = 1;
                const bool from_a = a[e] == cur;
                const int64_t other = from_a ? b[e] : a[e];
                verts[steps + 1] = (int32_t) other;
                neuron[steps] = e;
                flip[steps] = from_a ? 0 : 1;
                ++steps;
                cur = other;
            }
        }
    };
    // odd-degree vertices first: a trail that starts at one ends at another and none is wasted
    for (int64_t v = 0; v < in_dim; ++v)
        if ((start[(size_t) v + 1] - start[(size_t) v]) & 1) walk_from(v);
    for (int64_t v = 0; v < in_dim; ++v) walk_from(v);

    if (steps > 0) verts[0] = verts[1];
    while (steps % chunk != 0) {                     // pad with load-only steps
        verts[steps + 1] = verts[steps];
        neuron[steps] = -1;
        flip[steps] = 0;
        ++steps;
    }
    return steps;
}

// Destinations for dl_logic_backward_chained.  Position p of the schedule (vertex verts[p]) takes
// part in neuron[p - 1] and neuron[p]; if either exists the kernel produces one partial grad_x
// row there.  A vertex with exactly one such position is written straight to grad_x
// (dst[p] = vertex).  Every other vertex becomes a fix-up entry: its positions are numbered into
// consecutive overflow rows (dst[p] = in_dim + row), summed after the pass; a vertex at no
// position at all gets an entry with no rows (zero gradient).
extern "C" int64_t dl_backward_schedule_build(const int32_t *verts, const int32_t *neuron, int64_t steps,
                                              int64_t in_dim, int32_t *dst, int32_t *fix_vertex, int32_t *fix_start,
                                              int64_t *n_fix) {
    if (!verts || !neuron || !dst || !fix_vertex || !fix_start || !n_fix || steps < 0 || in_dim <= 0)
        return -DL_ERR_INVALID_ARGUMENT;
    if (in_dim > 0x3fffffffLL || steps > 0x3fffffffLL) return -DL_ERR_TOO_LARGE;
    auto produces = [&](int64_t p) { return (p > 0 && neuron[p - 1] >= 0) || (p < steps && neuron[p] >= 0); };
    std::vector<int32_t> count((size_t) in_dim, 0);
    for (int64_t p = 0; p <= steps; ++p) {
        if (verts[p] < 0 || verts[p] >= in_dim) return -DL_ERR_INVALID_ARGUMENT;
        if (produces(p)) ++count[(size_t) verts[p]];
    }
    // fix-up entries in vertex order; next_row[v] = the vertex's next free overflow row
    std::vector<int32_t> next_row((size_t) in_dim, -1);
    int64_t entries = 0, rows = 0;
    for (int64_t v = 0; v < in_dim; ++v) {
        if (count[(size_t) v] == 1) continue;
        fix_vertex[entries] = (int32_t) v;
        fix_start[entries] = (int32_t) rows;
        next_row[(size_t) v] = (int32_t) rows;
        rows += count[(size_t) v];
        ++entries;
    }
    fix_start[entries] = (int32_t) rows;
    if (in_dim + rows > 0x7fffffffLL) return -DL_ERR_TOO_LARGE;
    for (int64_t p = 0; p <= steps; ++p) {
        const int32_t v = verts[p];
        if (!produces(p))
            dst[p] = -1;
        else if (count[(size_t) v] == 1)
            dst[p] = v;
        else
            dst[p] = (int32_t) (in_dim + next_row[(size_t) v]++);
    }
    *n_fix = entries;
    return rows;
}

// Order in which dl_logic_eval_fused_groupbitsum walks the neurons of each class.  The count of a
// class does not depend on the order of its neurons, but the cache traffic does: a workgroup of
// the fused count kernel handles `group` consecutive neurons, and an input row that several of
// them read is fetched from beyond the L2 cache once instead of once per reader.  Neurons of a
// class are therefore collected breadth-first along shared input rows (the leaves of the
// depth-1 or depth-2 gate tree: a_low == NULL means the top layer reads the rows directly), so
// that readers of one row fall into one group wherever the class allows it.
//   order [out_dim]: a permutation of the neurons that maps every class onto itself.
extern "C" int dl_count_order_build(const int64_t *a_top, const int64_t *b_top, const int64_t *a_low,
                                    const int64_t *b_low, int64_t rows, int64_t mid_dim, int64_t out_dim, int64_t k,
                                    int group, int32_t *order) {
    if (!a_top || !b_top || !order || (!a_low) != (!b_low) || rows <= 0 || out_dim < 0 || k <= 0 || group <= 0)
        return DL_ERR_INVALID_ARGUMENT;
    if (out_dim % k != 0) return DL_ERR_NOT_DIVISIBLE;
    if (rows > 0x7fffffffLL || out_dim > 0x7fffffffLL || mid_dim > 0x7fffffffLL) return DL_ERR_TOO_LARGE;
    const int nl = a_low ? 4 : 2;
    const int64_t top_in = a_low ? mid_dim : rows;
    std::vector<int32_t> leaf((size_t) (out_dim * nl));
    for (int64_t n = 0; n < out_dim; ++n) {
        const int64_t u = a_top[n], v = b_top[n];
        if (u < 0 || u >= top_in || v < 0 || v >= top_in) return DL_ERR_INVALID_ARGUMENT;
        int64_t l[4] = {u, v, 0, 0};
        if (a_low) {
            l[0] = a_low[u];
            l[1] = b_low[u];
            l[2] = a_low[v];
            l[3] = b_low[v];
        }
        for (int i = 0; i < nl; ++i) {
            if (l[i] < 0 || l[i] >= rows) return DL_ERR_INVALID_ARGUMENT;
            leaf[(size_t) (n * nl + i)] = (int32_t) l[i];
        }
    }
    const int64_t per_class = out_dim / k;
    std::vector<int64_t> start((size_t) rows + 1);
    std::vector<int32_t> readers((size_t) (per_class * nl)), queue;
    std::vector<uint8_t> taken((size_t) per_class);
    for (int64_t c = 0; c < k; ++c) {
        const int64_t n0 = c * per_class;
        // readers of every row within this class (CSR)
        std::fill(start.begin(), start.end(), 0);
        for (int64_t i = 0; i < per_class * nl; ++i) ++start[(size_t) leaf[(size_t) (n0 * nl + i)] + 1];
        for (int64_t r = 0; r < rows; ++r) start[(size_t) r + 1] += start[(size_t) r];
        {
            std::vector<int64_t> fill(start.begin(), start.end() - 1);
            for (int64_t i = 0; i < per_class; ++i)
                for (int j = 0; j < nl; ++j) readers[(size_t) fill[(size_t) leaf[(size_t) ((n0 + i) * nl + j)]]++] = (int32_t) i;
        }
        std::fill(taken.begin(), taken.end(), 0);
        int64_t placed = 0, seed = 0;
        while (placed < per_class) {
            while (taken[(size_t) seed]) ++seed;
            // one group: breadth-first from the first free neuron; what is left in the queue when the
            // group is full goes back to the pool
            queue.assign(1, (int32_t) seed);
            taken[(size_t) seed] = 1;
            size_t head = 0;
            int in_group = 0;
            while (head < queue.size() && in_group < group) {
                const int32_t i = queue[head++];
                order[n0 + placed++] = (int32_t) (n0 + i);
                ++in_group;
                for (int j = 0; j < nl; ++j) {
                    const int32_t r = leaf[(size_t) ((n0 + i) * nl + j)];
                    for (int64_t q = start[(size_t) r]; q < start[(size_t) r + 1]; ++q) {
                        const int32_t other = readers[(size_t) q];
                        if (!taken[(size_t) other]) {
                            taken[(size_t) other] = 1;
                            queue.push_back(other);
                        }
                    }
                }
            }
            for (; head < queue.size(); ++head) taken[(size_t) queue[head]] = 0;
        }
    }
    return DL_OK;
}

// Plan for dl_logic_eval_chained_groupbitsum: the count kernel walks the top layer along the
// evaluation schedule, so consecutive outputs belong to arbitrary classes.  A workgroup of
// DL_CC_WAVES waves owns DL_CC_BLOCK * blocks consecutive steps (a contiguous range per wave) and proceeds
// in `blocks` blocks of DL_CC_BLOCK outputs (DL_CC_WAVE_STEPS per wave): every wave parks its
// outputs of the block in LDS at a slot that sorts the block by class, and the wave that owns a
// class then reads that class's run of slots and adds it to its bit-sliced counters.
//   slot [padded]           LDS slot of step s within its block, 255 = the step has no output
//   runs [padded / dl_count_chain_block() * k]  per block and class: first slot | number of slots << 8
//   *blocks                 blocks per workgroup: the largest of 16, 8, 4, 2, 1 for which no
//                           workgroup counts more than 255 neurons of one class (its counters have
//                           DL_CC_PLANES planes); fewer blocks mean more partial counters
// where step s of workgroup g, wave w, block b, position j is
// (g*DL_CC_WAVES + w)*DL_CC_WAVE_STEPS*blocks + b*DL_CC_WAVE_STEPS + j.  Returns the padded step count (a multiple of
// DL_CC_MAX_WG_STEPS; steps past `steps` have no output), or -DL_ERR_TOO_LARGE for more classes
// than the kernel's waves can own.
extern "C" int dl_count_chain_block(void) { return DL_CC_BLOCK; }

extern "C" int64_t dl_count_chain_padded_steps(int64_t steps) {
    if (steps < 0) return -DL_ERR_INVALID_ARGUMENT;
    return (steps + DL_CC_MAX_WG_STEPS - 1) / DL_CC_MAX_WG_STEPS * DL_CC_MAX_WG_STEPS;
}

static bool count_chain_plan(const int32_t *neuron, int64_t steps, int64_t per_class, int64_t k, int blocks,
                             int64_t padded, uint8_t *slot, uint16_t *runs) {
    const int64_t wg_steps = (int64_t) DL_CC_BLOCK * blocks, span = (int64_t) DL_CC_WAVE_STEPS * blocks;
    std::vector<int64_t> total((size_t) k);
    for (int64_t g = 0; g < padded / wg_steps; ++g) {
        std::fill(total.begin(), total.end(), 0);
        for (int64_t b = 0; b < blocks; ++b) {
            // class of every output of the block, in (wave, position) order
            int64_t cls[DL_CC_BLOCK], where[DL_CC_BLOCK];
            int count[DL_CC_MAX_CLASSES] = {0};
            for (int64_t w = 0; w < DL_CC_WAVES; ++w)
                for (int64_t j = 0; j < DL_CC_WAVE_STEPS; ++j) {
                    const int64_t s = g * wg_steps + w * span + b * DL_CC_WAVE_STEPS + j;
                    const int64_t i = w * DL_CC_WAVE_STEPS + j;
                    where[i] = s;
                    cls[i] = (s < steps && neuron[s] >= 0) ? neuron[s] / per_class : -1;
                    if (cls[i] >= 0) ++count[cls[i]];
                }
            int first[DL_CC_MAX_CLASSES];
            int at = 0;
            uint16_t *run = runs + (g * blocks + b) * k;
            for (int64_t c = 0; c < k; ++c) {
                first[c] = at;
                run[c] = (uint16_t) (at | (count[c] << 8));
                at += count[c];
                total[(size_t) c] += count[c];
            }
            for (int64_t i = 0; i < DL_CC_BLOCK; ++i) slot[where[i]] = cls[i] < 0 ? 255 : (uint8_t) first[cls[i]]++;
        }
        for (int64_t c = 0; c < k; ++c)
            if (total[(size_t) c] >= (1 << DL_CC_PLANES)) return false;
    }
    return true;
}

extern "C" int64_t dl_count_chain_plan_build(const int32_t *neuron, int64_t steps, int64_t out_dim, int64_t k,
                                             uint8_t *slot, uint16_t *runs, int *blocks) {
    if (!neuron || !slot || !runs || !blocks || steps < 0 || out_dim <= 0 || k <= 0) return -DL_ERR_INVALID_ARGUMENT;
    if (out_dim % k != 0) return -DL_ERR_NOT_DIVISIBLE;
    if (k > DL_CC_MAX_CLASSES) return -DL_ERR_TOO_LARGE;
    for (int64_t s = 0; s < steps; ++s)
        if (neuron[s] >= out_dim) return -DL_ERR_INVALID_ARGUMENT;
    const int64_t padded = dl_count_chain_padded_steps(steps);
    for (int nb = DL_CC_MAX_BLOCKS; nb >= 1; nb /= 2)       // one block holds at most DL_CC_BLOCK outputs: always fits
        if (count_chain_plan(neuron, steps, out_dim / k, k, nb, padded, slot, runs)) {
            *blocks = nb;
            return padded;
        }
    return -DL_ERR_TOO_LARGE;
}
