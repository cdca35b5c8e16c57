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

#include <vector>

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
