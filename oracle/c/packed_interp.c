/* Table-driven CPU interpreter of a discretised logic-gate net on 64-sample words.
 *
 * TEST INFRASTRUCTURE, NOT PRODUCT: checker for the HIP kernels and CPU baseline of the
 * benchmark.  It performs, per block of 64 samples, the steps of the C program the
 * reference generates (difflogic/compiled_model.py:182-237) without emitting one line of C
 * per gate:
 *   1. bool -> word packing, sample s of the block in bit s        (:191-198)
 *   2. every gate as one of 16 bitwise forms on 64-bit words        (:97-128)
 *   3. per class, a ripple-carry counter over bit planes, plane 0
 *      most significant, ceil(log2(out/k + 1)) planes               (:180, :204-219)
 *   4. unpack the planes to one int32 per (sample, class)           (:222-230)
 * Samples beyond the batch are treated as all-zero inputs and their outputs dropped
 * (:349-366).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

typedef uint64_t word_t;

static inline word_t gate(word_t a, word_t b, unsigned op) {
    switch (op) {
    case 0: return 0;
    case 1: return a & b;
    case 2: return a & ~b;
    case 3: return a;
    case 4: return b & ~a;
    case 5: return b;
    case 6: return a ^ b;
    case 7: return a | b;
    case 8: return ~(a | b);
    case 9: return ~(a ^ b);
    case 10: return ~b;
    case 11: return ~b | a;
    case 12: return ~a;
    case 13: return ~a | b;
    case 14: return ~(a & b);
    default: return ~(word_t) 0;
    }
}

/* One layer on a single word column: y[n] = gate(x[a[n]], x[b[n]], op[n]). */
static void layer_column(const word_t *x, word_t *y, int64_t out, const int64_t *a,
                         const int64_t *b, const uint8_t *op) {
    for (int64_t n = 0; n < out; ++n) y[n] = gate(x[a[n]], x[b[n]], op[n]);
}

/* x_bool [B,F] row-major bytes; widths[L]; a/b/op are the layers' tables concatenated;
 * out [B,k] int32.  Blocks of 64 samples are independent: with threads > 1 they are split
 * over an OpenMP team.  Returns 0, or -1 on a bad argument / allocation failure. */
int dl_oracle_net_eval(const uint8_t *x_bool, int64_t B, int64_t F, int L, const int64_t *widths,
                       const int64_t *a, const int64_t *b, const uint8_t *op, int k, int32_t *out,
                       int threads) {
    if (L < 1 || k < 1 || B < 0) return -1;
    int64_t max_w = F;
    for (int l = 0; l < L; ++l) if (widths[l] > max_w) max_w = widths[l];
    const int64_t n_last = widths[L - 1];
    const int64_t per_class = n_last / k;
    const int planes = (int) ceil(log2((double) n_last / (double) k + 1.0));
    const int64_t blocks = (B + 63) / 64;
    int failed = 0;
    if (threads < 1) threads = 1;

#pragma omp parallel num_threads(threads)
    {
        word_t *cur = malloc(sizeof(word_t) * (size_t) max_w);
        word_t *nxt = malloc(sizeof(word_t) * (size_t) max_w);
        word_t *cnt = malloc(sizeof(word_t) * (size_t) (planes > 0 ? planes : 1));
        if (!cur || !nxt || !cnt) {
#pragma omp atomic write
            failed = 1;
        } else {
#pragma omp for schedule(dynamic, 4)
            for (int64_t blk = 0; blk < blocks; ++blk) {
                const int64_t s0 = blk * 64;
                const int64_t ns = (B - s0 < 64) ? (B - s0) : 64;
                for (int64_t f = 0; f < F; ++f) {
                    word_t w = 0;
                    for (int64_t s = ns - 1; s >= 0; --s) {
                        w <<= 1;
                        w += (word_t) (x_bool[(s0 + s) * F + f] != 0);
                    }
                    cur[f] = w;
                }
                int64_t off = 0;
                for (int l = 0; l < L; ++l) {
                    layer_column(cur, nxt, widths[l], a + off, b + off, op + off);
                    off += widths[l];
                    word_t *t = cur; cur = nxt; nxt = t;
                }
                for (int c = 0; c < k; ++c) {
                    for (int p = 0; p < planes; ++p) cnt[p] = 0;
                    for (int64_t n = 0; n < per_class; ++n) {
                        word_t carry = cur[c * per_class + n];
                        for (int p = planes - 1; p >= 0; --p) {
                            const word_t old = cnt[p];
                            cnt[p] = old ^ carry;
                            carry = old & carry;
                        }
                    }
                    for (int64_t s = 0; s < ns; ++s) {
                        int32_t v = 0;
                        for (int p = 0; p < planes; ++p) v = (v << 1) + (int32_t) ((cnt[p] >> s) & 1u);
                        out[(s0 + s) * k + c] = v;
                    }
                }
            }
        }
        free(cur);
        free(nxt);
        free(cnt);
    }
    return failed ? -1 : 0;
}

/* One layer on a word matrix: x [in,W], y [out,W], 64-bit words. */
int dl_oracle_eval_layer(const uint64_t *x, uint64_t *y, int64_t out, int64_t W, const int64_t *a,
                         const int64_t *b, const uint8_t *op, int threads) {
    if (threads < 1) threads = 1;
#pragma omp parallel for num_threads(threads) schedule(static)
    for (int64_t n = 0; n < out; ++n) {
        const uint64_t *ra = x + a[n] * W, *rb = x + b[n] * W;
        uint64_t *ry = y + n * W;
        const unsigned o = op[n];
        for (int64_t c = 0; c < W; ++c) ry[c] = gate(ra[c], rb[c], o);
    }
    return 0;
}
