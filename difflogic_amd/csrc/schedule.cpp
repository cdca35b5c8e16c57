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
