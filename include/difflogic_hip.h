/* difflogic_hip.h -- C ABI of libdifflogic_hip.so: the LogicLayer kernel family for AMD
 * MI355X (gfx950), hand-written HIP.
 *
 * Conventions
 * -----------
 * - Every pointer is a DEVICE pointer on the current HIP device unless stated otherwise.
 *   The library never allocates, frees or synchronises (dl_logic_eval_fused_groupbitsum_noalloc
 *   owns one static device array, see there): the caller owns all buffers
 *   (inputs are read-only, outputs are fully overwritten) and orders work through the
 *   `stream` argument (a hipStream_t passed as void*; NULL = the null stream).
 * - All matrices are feature-major and batch-contiguous: element (row f, column r) of an
 *   [F, R] matrix lives at f*R + r.
 * - Index tables `a`, `b` hold values in [0, in_dim); `start`/`idx` are the CSR reverse
 *   index the reference builds at difflogic/difflogic.py:60-69.  The kernels trust them.
 * - Every function returns a dl_status (0 = success).  Nothing here calls exit().
 * - Functions are re-entrant; the only state is a per-thread record of the last refused
 *   launch's HIP error (dl_last_hip_error).  Kernels are launched with hipLaunchKernel and its
 *   return value is what is reported; the runtime's per-thread last error is not touched.
 *
 * Each entry point replaces one function of the reference's extension module
 * `difflogic_cuda` (difflogic/cuda/difflogic.cpp:45-84); the comment above each declaration
 * names it.
 */
#ifndef DIFFLOGIC_HIP_H
#define DIFFLOGIC_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum dl_status {
    DL_OK = 0,
    DL_ERR_INVALID_ARGUMENT = 1, /* null pointer, negative size, misaligned buffer            */
    DL_ERR_BIT_COUNT = 2,        /* bit_count not in {8, 16, 32, 64}                          */
    DL_ERR_NOT_DIVISIBLE = 3,    /* groupbitsum: in_dim not divisible by k                    */
    DL_ERR_DTYPE = 4,            /* dtype not one of dl_dtype                                 */
    DL_ERR_LAUNCH = 5,           /* the HIP runtime refused the launch (see dl_last_hip_error) */
    DL_ERR_TOO_LARGE = 6,        /* a size exceeds what the entry point supports              */
    DL_ERR_SCRATCH_LIMIT = 7,    /* the call needs more than DL_STATIC_SCRATCH_BYTES of scratch */
    DL_ERR_CAPTURING = 8         /* a first call per device that must not run under graph capture  */
} dl_status;

/* DL_F16_W32 / DL_F64_W32: activations and their gradients (x, y, grad_y, grad_x) in half / double, everything of
 * shape [out, 16] (gate weights, logits, probabilities, grad_w, grad_logits) in fp32: a layer with fp32 weights on
 * half / double inputs (the reference's --training-bit-count 16 / 64, experiments/main.py:19-23,286, casts the
 * probabilities instead, difflogic/difflogic.py:123-126).  Accepted by dl_logic_forward, dl_logic_forward_logits,
 * dl_logic_forward_chained, dl_logic_backward_w, dl_logic_backward_logits, dl_logic_backward_w_chained,
 * dl_logic_backward_x, dl_logic_backward_chained and dl_logic_backward_chained_workspace_bytes; every other
 * entry point answers DL_ERR_DTYPE. */
typedef enum dl_dtype { DL_F16 = 0, DL_F32 = 1, DL_F64 = 2, DL_F16_W32 = 3, DL_F64_W32 = 4 } dl_dtype;

/* Library version (major*10000 + minor*100 + patch) and a static message per status. */
int dl_version(void);
const char *dl_status_string(int status);
/* HIP's description of the error behind the calling thread's last DL_ERR_LAUNCH. */
const char *dl_last_hip_error(void);

/* ---- training mode -------------------------------------------------------------------- */

/* Replaces `forward` = logic_layer_cuda_forward (difflogic/cuda/difflogic.cpp:46-51,
 * difflogic/cuda/difflogic_kernel.cu:259-297).
 *   x [in_dim, batch], w [out_dim, 16], y [out_dim, batch] of `dtype`; a, b [out_dim] int64.
 *   y[n,r] = sum_i w[n,i] * f_i(x[a[n],r], x[b[n],r]),  f_i = real-valued gate i. */
int dl_logic_forward(const void *x, const int64_t *a, const int64_t *b, const void *w, void *y,
                     int64_t in_dim, int64_t out_dim, int64_t batch, int dtype, void *stream);

/* Replaces `backward_w` = logic_layer_cuda_backward_w (difflogic.cpp:52-56,
 * difflogic_kernel.cu:300-364), including the host-side sum + 16-way stack.
 *   grad_w[n,i] = sum_r grad_y[n,r] * f_i(x[a[n],r], x[b[n],r]);  grad_w [out_dim, 16].
 * Deterministic: fixed-order in-wave and LDS reductions, no atomics. */
int dl_logic_backward_w(const void *x, const int64_t *a, const int64_t *b, const void *grad_y,
                        void *grad_w, int64_t in_dim, int64_t out_dim, int64_t batch, int dtype,
                        void *stream);

/* forward / backward_w with the softmax over the 16 gate logits folded in, i.e. the pair
 * `softmax(weights)` + `forward` of difflogic/difflogic.py:123-126 and `backward_w` + the softmax
 * backward that autograd chains after it.  No counterpart in the reference's extension.
 *   dl_logic_forward_logits : logits [out_dim,16] -> y [out_dim,batch] and probs [out_dim,16]
 *                             (= softmax(logits), kept for the backward pass; batch >= 1)
 *   dl_logic_backward_logits: grad_logits[n,i] = p_i * (g_i - sum_j p_j g_j) with
 *                             g = dl_logic_backward_w(x, a, b, grad_y), p = probs. */
int dl_logic_forward_logits(const void *x, const int64_t *a, const int64_t *b, const void *logits,
                            void *y, void *probs, int64_t in_dim, int64_t out_dim, int64_t batch,
                            int dtype, void *stream);
int dl_logic_backward_logits(const void *x, const int64_t *a, const int64_t *b, const void *grad_y,
                             const void *probs, void *grad_logits, int64_t in_dim, int64_t out_dim,
                             int64_t batch, int dtype, void *stream);

/* forward / backward_w walked along an evaluation schedule of the layer's wiring (built with
 * dl_eval_schedule_build, declared below): consecutive neurons share an input row, which stays in
 * registers, so a neuron costs one gathered row instead of two.  Results are bit-identical to
 * dl_logic_forward(_logits) / dl_logic_backward_w(_logits) in fp32 and fp64 (fp16 outputs can
 * differ in the last bit).  No counterpart in the reference.
 *   verts [steps+1], neuron [steps], flip [steps]: DEVICE copies of the schedule.
 *   probs: forward  - NULL: `w` holds probabilities; else `w` holds logits and probs receives
 *                     softmax(w) (as dl_logic_forward_logits);
 *          backward - NULL: plain grad_w; else the softmax backward is chained
 *                     (as dl_logic_backward_logits).
 * Return DL_ERR_TOO_LARGE where the chained kernels do not apply (batch not a multiple of 16
 * bytes of elements, unaligned buffers; backward_w: rows longer than 256 vectors of 16 bytes);
 * the caller then uses the unchained entry points. */
int dl_logic_forward_chained(const void *x, const int32_t *verts, const int32_t *neuron,
                             const uint8_t *flip, int64_t steps, const void *w, void *y, void *probs,
                             int64_t in_dim, int64_t out_dim, int64_t batch, int dtype, void *stream);
int dl_logic_backward_w_chained(const void *x, const int32_t *verts, const int32_t *neuron,
                                const uint8_t *flip, int64_t steps, const void *grad_y,
                                const void *probs, void *grad_w, int64_t in_dim, int64_t out_dim,
                                int64_t batch, int dtype, void *stream);

/* Replaces `backward_x` = logic_layer_cuda_backward_x (difflogic.cpp:57-62,
 * difflogic_kernel.cu:367-410).
 *   grad_x[c,r] = scale * sum over neurons n reading input c of
 *                 grad_y[n,r] * d y[n,r] / d x[c,r];          grad_x [in_dim, batch].
 *   start [in_dim+1], idx [2*out_dim] int64: the reverse index.  A neuron with
 *   a[n] == b[n] contributes d/da + d/db (autograd semantics of the python implementation).
 *   `scale` folds the reference's GradFactor (difflogic/functional.py:130-138); pass 1.0 for
 *   the reference's backward_x. */
int dl_logic_backward_x(const void *x, const int64_t *a, const int64_t *b, const void *w,
                        const void *grad_y, const int64_t *start, const int64_t *idx, void *grad_x,
                        int64_t in_dim, int64_t out_dim, int64_t batch, double scale, int dtype,
                        void *stream);

/* backward_w and backward_x of one layer in a single pass along the schedule (the pair
 * difflogic/difflogic.py:218,220): every neuron's input rows and grad_y row are read once and
 * serve grad_w and both grad_x contributions.  No counterpart in the reference.
 *   dl_backward_schedule_build()  HOST pointers.  From a schedule (verts [steps+1], neuron [steps])
 *       writes dst [steps+1]: the grad_x row that schedule position p completes (-1: none;
 *       >= in_dim: row dst - in_dim of the overflow buffer), and the fix-up list for inputs that
 *       occur at several positions or at none: fix_vertex [<= in_dim], fix_start [<= in_dim + 1]
 *       (overflow rows fix_start[i] .. fix_start[i+1]-1 are summed into grad_x[fix_vertex[i]]).
 *       *n_fix receives the list's length; returns the number of overflow rows or a negated
 *       dl_status.
 *   dl_logic_backward_chained()   DEVICE pointers.  w [out,16]: the gate probabilities the forward
 *       pass used.  softmax_backward = 0: grad_w as dl_logic_backward_w; else the gradient with
 *       respect to the logits as dl_logic_backward_logits (w = its probs).  grad_x as
 *       dl_logic_backward_x (same `scale`, same a == b rule) up to summation order.
 *       overflow_rows: what dl_backward_schedule_build returned.  workspace: DEVICE scratch of
 *       dl_logic_backward_chained_workspace_bytes(overflow_rows, out_dim, batch, dtype) bytes,
 *       16-byte aligned (NULL if that is 0): the overflow rows and, for rows longer than 4 KB,
 *       per-segment partial sums of grad_w.  Returns DL_ERR_TOO_LARGE where it does not apply
 *       (batch not a multiple of 16 bytes of elements, unaligned buffers, rows longer than
 *       64 KB); the caller then uses the separate entry points. */
int64_t dl_backward_schedule_build(const int32_t *verts, const int32_t *neuron, int64_t steps,
                                   int64_t in_dim, int32_t *dst, int32_t *fix_vertex,
                                   int32_t *fix_start, int64_t *n_fix);
int dl_logic_backward_chained(const void *x, const int32_t *verts, const int32_t *neuron,
                              const uint8_t *flip, const int32_t *dst, int64_t steps, const void *w,
                              const void *grad_y, int softmax_backward, const int32_t *fix_vertex,
                              const int32_t *fix_start, int64_t n_fix, int64_t overflow_rows,
                              void *grad_w, void *grad_x, void *workspace, int64_t in_dim,
                              int64_t out_dim, int64_t batch, double scale, int dtype, void *stream);
int64_t dl_logic_backward_chained_workspace_bytes(int64_t overflow_rows, int64_t out_dim,
                                                  int64_t batch, int dtype);

/* dl_logic_backward_chained for a layer whose input x is the output of a layer that needs no
 * grad_x itself (a model's first layer): that lower layer's backward_w (difflogic/difflogic.py:220
 * of the layer below) is taken in the same pass.  A finished grad_x row IS the grad_y row of neuron
 * `row` of the lower layer, so its corner sums are formed from the row in registers and the
 * neuron's two input rows, and grad_x is never written or read back.  No counterpart in the
 * reference.  Arguments as dl_logic_backward_chained, except:
 *   x              may be NULL (fp32 / fp64): row v of x is then recomputed as
 *                  dl_logic_forward(x_lower, a_lower, b_lower, w_lower) produced it (bit for bit),
 *                  from the two lower rows that vertex v's backward_w reads anyway, so the activation
 *                  between the two layers need not exist in memory (see dl_logic_forward_chained_lower)
 *   fix_rows       DEVICE [n_fix, batch] scratch (NULL if n_fix == 0) in place of grad_x: the rows
 *                  of the vertices on the fix-up list, the only ones that still pass through memory
 *   x_lower        [in_dim_lower, batch] input of the lower layer; a_lower, b_lower [in_dim] its wiring
 *   w_lower        [in_dim, 16] the lower layer's gate probabilities (needed when x is NULL or
 *                  softmax_backward_lower is set; else may be NULL)
 *   softmax_backward_lower  0: grad_w_lower as dl_logic_backward_w; else with respect to the lower
 *                  layer's logits, as dl_logic_backward_logits
 *   grad_w_lower   [in_dim, 16] out.  Same values as the separate calls (grad_x rounded to dtype in
 *                  between, as when stored).
 * Applies to rows of at most 4 KB; otherwise DL_ERR_TOO_LARGE and the caller uses the separate
 * entry points. */
int dl_logic_backward_chained_lower(const void *x, const int32_t *verts, const int32_t *neuron,
                                    const uint8_t *flip, const int32_t *dst, int64_t steps,
                                    const void *w, const void *grad_y, int softmax_backward,
                                    const int32_t *fix_vertex, const int32_t *fix_start,
                                    int64_t n_fix, int64_t overflow_rows, void *grad_w,
                                    void *fix_rows, void *workspace, const void *x_lower,
                                    const int64_t *a_lower, const int64_t *b_lower,
                                    const void *w_lower, int softmax_backward_lower,
                                    void *grad_w_lower, int64_t in_dim, int64_t out_dim,
                                    int64_t batch, double scale, int dtype, void *stream);

/* ---- GroupSum on the feature-major layout (training mode) ------------------------------- */

/* Replaces the float branch of GroupSum.forward (difflogic/difflogic.py:195-196) for the
 * [out_dim, batch] layout the layer kernels produce, and its autograd backward:
 *   forward : y[r, c] = (1/tau) * sum over the out_dim/k neurons of class c of x[n, r];
 *             x [out_dim, batch] -> y [batch, k].  Deterministic (fixed summation order).
 *             `workspace` is scratch of dl_group_sum_workspace_bytes(...) bytes.
 *   backward: grad_x[n, r] = grad_y[r, class(n)] / tau;  grad_y [batch, k] -> grad_x [out_dim, batch]. */
int64_t dl_group_sum_workspace_bytes(int64_t out_dim, int64_t batch, int64_t k, int dtype);
int dl_group_sum_forward(const void *x, void *y, void *workspace, int64_t out_dim, int64_t batch,
                         int64_t k, double tau, int dtype, void *stream);
int dl_group_sum_backward(const void *grad_y, void *grad_x, int64_t out_dim, int64_t batch, int64_t k,
                          double tau, int dtype, void *stream);

/* The last LogicLayer of a model and the GroupSum that follows it as ONE step (the pair
 * difflogic/difflogic.py:123-126 then :195-196, and their backward passes): the layer's output
 * [out_dim, batch] and the broadcast gradient GroupSum's backward would hand back are never
 * materialised.  No counterpart in the reference.
 *   dl_logic_forward_group_sum : y[r, c] = (1/tau) * sum over the neurons n of class c of
 *       forward(x, a, b, w)[n, r];  y [batch, k].  probs != NULL: w holds logits and probs
 *       receives softmax(w) (as dl_logic_forward_logits); NULL: w holds probabilities.
 *       workspace: dl_group_sum_workspace_bytes(out_dim, batch, k, dtype) bytes.  Deterministic.
 *   dl_logic_backward_*_grouped : as dl_logic_backward_logits (probs == NULL: as
 *       dl_logic_backward_w), dl_logic_backward_x and dl_logic_backward_chained, with
 *       grad_y[n, r] = grad_cls[class(n), r]:  grad_cls [k, batch] is GroupSum's incoming gradient,
 *       transposed and already divided by tau; class(n) = n / (out_dim / k). */
int dl_logic_forward_group_sum(const void *x, const int64_t *a, const int64_t *b, const void *w,
                               void *probs, void *y, void *workspace, int64_t in_dim, int64_t out_dim,
                               int64_t batch, int64_t k, double tau, int dtype, void *stream);
int dl_logic_backward_logits_grouped(const void *x, const int64_t *a, const int64_t *b,
                                     const void *grad_cls, const void *probs, void *grad_w,
                                     int64_t in_dim, int64_t out_dim, int64_t batch, int64_t k,
                                     int dtype, void *stream);
int dl_logic_backward_x_grouped(const void *x, const int64_t *a, const int64_t *b, const void *w,
                                const void *grad_cls, const int64_t *start, const int64_t *idx,
                                void *grad_x, int64_t in_dim, int64_t out_dim, int64_t batch,
                                int64_t k, double scale, int dtype, void *stream);
int dl_logic_backward_chained_grouped(const void *x, const int32_t *verts, const int32_t *neuron,
                                      const uint8_t *flip, const int32_t *dst, int64_t steps,
                                      const void *w, const void *grad_cls, int softmax_backward,
                                      const int32_t *fix_vertex, const int32_t *fix_start,
                                      int64_t n_fix, int64_t overflow_rows, void *grad_w,
                                      void *grad_x, void *workspace, int64_t in_dim, int64_t out_dim,
                                      int64_t batch, int64_t k, double scale, int dtype, void *stream);

/* dl_logic_forward_chained for a layer whose input is the output of the layer below, with that
 * output recomputed row by row instead of read: y = forward(forward(x_lower, a_lower, b_lower,
 * w_lower), a, b, w) bit for bit, but the activation between the two layers is neither written nor
 * read (two calls of difflogic/difflogic.py:123-126 / :209).  Pays when x_lower is small enough to
 * stay in the L2 caches (a model's 784-row input).  No counterpart in the reference.
 *   probs != NULL (then probs_lower != NULL too): w and w_lower hold logits and the two receive
 *   their softmax, as dl_logic_forward_logits; NULL (both): they hold probabilities.
 *   verts, neuron, flip, steps: the evaluation schedule of (a, b) (dl_eval_schedule_build).
 * Applies to rows of at most 2 KB; otherwise DL_ERR_TOO_LARGE.  Only the vertices the schedule
 * visits get their probs_lower row: clear it first if the other rows are read later. */
int dl_logic_forward_chained_lower(const void *x_lower, const int64_t *a_lower, const int64_t *b_lower,
                                   const void *w_lower, void *probs_lower, const int32_t *verts,
                                   const int32_t *neuron, const uint8_t *flip, int64_t steps,
                                   const void *w, void *y, void *probs, int64_t in_dim_lower,
                                   int64_t in_dim, int64_t out_dim, int64_t batch, int dtype,
                                   void *stream);

/* The optimizer step of the reference's training loop (torch.optim.Adam(lr=...).step(),
 * experiments/main.py:169,179) for all of a model's fp32 weight tensors in one launch.  No counterpart
 * in the reference's extension.  Semantics of torch.optim.Adam (amsgrad and maximize off):
 *   step += 1;  g += weight_decay * p;  m += (1 - beta1) * (g - m);  v = beta2 * v + (1 - beta2) * g * g;
 *   p -= lr / (1 - beta1^step) * m / (sqrt(v) / sqrt(1 - beta2^step) + eps)
 *   p, g, m, v : HOST arrays of `count` (<= dl_adam_max_tensors()) DEVICE pointers to contiguous
 *                fp32 tensors of numel[i] elements (numel: HOST array); m, v start as zeros.
 *   state      : DEVICE fp32 [4]; state[0] holds the number of updates done so far (starts at 0) and
 *                is advanced on the device, so a launch captured into a HIP graph stays correct on
 *                replay; state[1..2] are scratch (the bias-correction factors of the update under
 *                way, computed in double); state[3] is unused. */
int dl_adam_max_tensors(void);
int dl_adam_step(int count, float *const *p, const float *const *g, float *const *m, float *const *v,
                 const int64_t *numel, float *state, double lr, double beta1, double beta2, double eps,
                 double weight_decay, void *stream);

/* ---- packed inference mode ------------------------------------------------------------ */

/* The gate ids packed inference evaluates: ids[n] = argmax_i w[n, i] as uint8, i.e.
 * `self.weights.argmax(-1).to(torch.uint8)` of difflogic/difflogic.py:146 in one kernel (the first
 * maximal value wins; a NaN counts as maximal, as in torch).  w [out_dim, 16] of `dtype`. */
int dl_gate_ids(const void *w, uint8_t *ids, int64_t out_dim, int dtype, void *stream);

/* Constant folding over the gate ids of one layer, for packed inference (no counterpart in the
 * reference, whose generated C leaves it to the compiler: difflogic/compiled_model.py:97-128 emits
 * one statement per gate).  A neuron with a constant gate (ids 0, 15), or one whose inputs make it
 * constant, outputs the same word for every sample; a gate reading it is replaced by the gate it
 * amounts to with that input fixed, which ignores the input (so the packed kernels fetch nothing
 * for it).  The evaluated function is unchanged, bit for bit.
 *   a, b [out_dim] the layer's wiring; w [out_dim] its gate ids;
 *   state_in [in_dim] or NULL: 0 = the input row varies, 1 = all zeros, 2 = all ones;
 *   w_out [out_dim]: the gate ids to evaluate; state_out [out_dim]: the constants among the outputs. */
int dl_fold_gate_constants(const int64_t *a, const int64_t *b, const uint8_t *w, const uint8_t *state_in,
                           uint8_t *w_out, uint8_t *state_out, int64_t out_dim, void *stream);

/* dl_gate_ids and dl_fold_gate_constants of one layer in one kernel (what a layer in eval mode hands to the packed
 * path): ids[n] = the argmax gate of neuron n with the constants among its input rows folded in, state_out[n] =
 * whether the neuron is constant itself.  w [out_dim, 16] of `dtype`; a, b, state_in, state_out as above. */
int dl_gate_ids_folded(const void *w, int dtype, const int64_t *a, const int64_t *b, const uint8_t *state_in,
                       uint8_t *ids, uint8_t *state_out, int64_t out_dim, void *stream);

/* Which input rows a layer looks at, for packed inference across fused groups (no counterpart in the
 * reference): live_in[r] is set to 1 where some neuron n with live_out[n] != 0 (live_out NULL: every
 * neuron) reads row r through an input its gate does not ignore.  live_in [in_dim] is cleared by the
 * caller beforehand.  Applied from the last layer downwards it yields, per layer, the output rows
 * that have to exist; dl_logic_eval_chained takes that vector as out_live. */
int dl_mark_live_inputs(const int64_t *a, const int64_t *b, const uint8_t *w, const uint8_t *live_out,
                        uint8_t *live_in, int64_t out_dim, void *stream);

/* Replaces `eval` = logic_layer_cuda_eval (difflogic.cpp:63-68, difflogic_kernel.cu:503-541).
 *   x [in_dim, words], y [out_dim, words] of signed integers of `bit_count` bits;
 *   w [out_dim] uint8 gate ids (4-bit truth tables, difflogic_kernel.cu:418-435).
 *   y[n,c] = gate_{w[n]}(x[a[n],c], x[b[n],c]) bitwise. */
int dl_logic_eval(const void *x, const int64_t *a, const int64_t *b, const uint8_t *w, void *y,
                  int64_t in_dim, int64_t out_dim, int64_t words, int bit_count, void *stream);

/* Replaces `tensor_packbits_cuda` (difflogic.cpp:69-74, difflogic_kernel.cu:583-625).
 *   t [features, batch] bool bytes -> out [features, ceil(batch/bit_count)] words;
 *   bit i of word c = sample bit_count*c + i, tail bits zero.
 *   *pad_len (HOST pointer, may be NULL) receives (bit_count - batch % bit_count) % bit_count. */
int dl_tensor_packbits(const uint8_t *t, void *out, int64_t features, int64_t batch, int bit_count,
                       int64_t *pad_len, void *stream);

/* Fuses the two steps of the reference's PackBitsTensor constructor
 * (difflogic/packbitstensor.py:15-16: `t.T.contiguous()` followed by tensor_packbits_cuda):
 *   x [batch, features] bool bytes, SAMPLE-major -> out [features, ceil(batch/bit_count)] words,
 *   same bit order and padding as dl_tensor_packbits. */
int dl_tensor_packbits_batch_major(const uint8_t *x, void *out, int64_t batch, int64_t features,
                                   int bit_count, int64_t *pad_len, void *stream);

/* The same packing (difflogic/packbitstensor.py:15-16) into rows of a length the caller chooses:
 *   out [features, out_row_bytes] bytes, 8 * out_row_bytes >= batch; sample s is bit s % 8 of byte
 *   s / 8 of its feature's row (the memory image of little-endian words of any of the four widths),
 *   every bit past the batch is zero.  PackBitsTensor uses it to keep rows a multiple of 16 bytes
 *   whatever the batch size and word width, so that the gate kernels always run on whole vectors. */
int dl_tensor_packbits_batch_major_rows(const uint8_t *x, void *out, int64_t batch, int64_t features,
                                        int64_t out_row_bytes, void *stream);

/* Replaces `groupbitsum` (difflogic.cpp:75-83, difflogic_kernel.cu:666-700), including the
 * final transpose.
 *   b [in_dim, words] words -> out [words*bit_count - pad_len, k] int32 (sample-major):
 *   out[s, c] = number of set sample-s bits over neurons c*in_dim/k ... (c+1)*in_dim/k - 1. */
int dl_groupbitsum(const void *b, int32_t *out, int64_t in_dim, int64_t words, int bit_count,
                   int64_t pad_len, int64_t k, void *stream);

/* Fused evaluation of `depth` (1..4) consecutive layers: same result as `depth` calls of
 * dl_logic_eval (the loop difflogic/difflogic.py:147 runs once per layer), but the intermediate
 * activations are never written: every output neuron is evaluated as a depth-`depth` tree of gates
 * over 2^depth gathered rows of x.  No counterpart in the reference.
 *   a, b, w   HOST arrays of `depth` DEVICE pointers, [0] = the group's first layer
 *   dims      HOST array {in_dim, width of layer 0, ..., width of layer depth-1}
 *   x [in_dim, words] -> y [dims[depth], words]
 *   workspace DEVICE scratch of dl_logic_eval_fused_workspace_bytes(depth, dims[depth]) bytes,
 *             8-byte aligned (holds the flattened per-neuron wiring; rebuilt by every call).
 * Rows must be whole 64-bit words (words*bit_count % 64 == 0, 8-byte aligned buffers); otherwise
 * DL_ERR_TOO_LARGE is returned and the caller evaluates layer by layer. */
int64_t dl_logic_eval_fused_workspace_bytes(int depth, int64_t out_dim);
int dl_logic_eval_fused(const void *x, int depth, const int64_t *const *a, const int64_t *const *b,
                        const uint8_t *const *w, const int64_t *dims, void *y, int64_t words,
                        int bit_count, void *workspace, void *stream);

/* Same result as dl_logic_eval_fused, computed along an evaluation schedule of the group's top
 * layer: its neurons are ordered so that consecutive ones share an input, whose value (a subtree
 * of depth-1 layers over 2^(depth-1) gathered rows) stays in registers; a neuron then costs
 * 2^(depth-1) gathers instead of 2^depth.  No counterpart in the reference.  The schedule
 * depends only on the top layer's wiring; build it once per layer.
 *   dl_eval_schedule_chunk()      steps one wave walks at a time (the step count is a multiple)
 *   dl_eval_schedule_capacity()   upper bound of steps for out_dim neurons
 *   dl_eval_schedule_build()      HOST pointers in and out.  a, b [out_dim] (the top layer's wiring)
 *                                 are validated against in_dim.  Writes verts [steps + 1],
 *                                 neuron [steps] (-1 = no output at this step), flip [steps];
 *                                 returns the number of steps, or a negated dl_status.
 *   dl_logic_eval_chained()       as dl_logic_eval_fused plus the DEVICE schedule arrays; workspace
 *                                 of dl_logic_eval_chained_workspace_bytes(depth, dims[depth-1],
 *                                 steps) bytes, 64-byte aligned: the flattened subtrees and one
 *                                 record per step, both rebuilt by every call.
 *                                 out_live [dims[depth]] or NULL: output rows with out_live[n] == 0
 *                                 will not be read by the caller and MAY be left unwritten (see
 *                                 dl_mark_live_inputs); NULL: every row is written. */
int dl_eval_schedule_chunk(void);
int64_t dl_eval_schedule_capacity(int64_t out_dim, int chunk);
int64_t dl_eval_schedule_build(const int64_t *a, const int64_t *b, int64_t in_dim, int64_t out_dim,
                               int chunk, int32_t *verts, int32_t *neuron, uint8_t *flip);
int64_t dl_logic_eval_chained_workspace_bytes(int depth, int64_t sub_dim, int64_t steps);
int dl_logic_eval_chained(const void *x, int depth, const int64_t *const *a, const int64_t *const *b,
                          const uint8_t *const *w, const int64_t *dims, const int32_t *verts,
                          const int32_t *neuron, const uint8_t *flip, int64_t steps,
                          const uint8_t *out_live, void *y, int64_t words, int bit_count, void *workspace,
                          void *stream);

/* The net's last `depth` (1 or 2) layers fused with `groupbitsum` (the sequence
 * difflogic/difflogic.py:147 then difflogic/packbitstensor.py:22): the last layer's output words
 * are counted as they are produced and never written.  Arguments as dl_logic_eval_fused, result
 * as dl_groupbitsum: out [words*bit_count - pad_len, k] int32.  Also needs k <= 65535.
 *   workspace DEVICE scratch of dl_logic_eval_fused_groupbitsum_workspace_bytes(...) bytes,
 *             16-byte aligned: the flattened wiring plus the bit-sliced partial counters that the
 *             first of the two passes hands to the second.
 *   order     NULL, or DEVICE int32 [out_dim]: the order in which the neurons are walked, a
 *             permutation that maps every class onto itself (trusted).  The result does not
 *             depend on it; dl_count_order_build (HOST pointers: the wiring of the top layer and,
 *             for depth 2, of the layer below it, else NULL; rows = dims[0], mid_dim = dims[1];
 *             group = dl_count_group()) returns one that puts neurons reading the same input
 *             rows next to each other, so that a workgroup fetches a shared row once: about a
 *             tenth fewer fetched bytes for the reference's wirings. */
int dl_count_group(void);
int dl_count_order_build(const int64_t *a_top, const int64_t *b_top, const int64_t *a_low,
                         const int64_t *b_low, int64_t rows, int64_t mid_dim, int64_t out_dim,
                         int64_t k, int group, int32_t *order);
int64_t dl_logic_eval_fused_groupbitsum_workspace_bytes(int depth, int64_t out_dim, int64_t words,
                                                        int bit_count, int64_t k);
int dl_logic_eval_fused_groupbitsum(const void *x, int depth, const int64_t *const *a,
                                    const int64_t *const *b, const uint8_t *const *w,
                                    const int64_t *dims, int32_t *out, int64_t words, int bit_count,
                                    int64_t pad_len, int64_t k, const int32_t *order, void *workspace,
                                    void *stream);

/* dl_logic_eval_fused_groupbitsum with the top layer walked along its evaluation schedule (as
 * dl_logic_eval_chained walks it): consecutive neurons share an input vertex whose value stays in
 * registers, so a neuron of a depth-2 group costs two gathered rows of x instead of four (depth 1:
 * one instead of two).  Same result as dl_logic_eval_fused_groupbitsum.  No counterpart in the
 * reference.
 *   verts, neuron, flip, steps   DEVICE copies of the top layer's schedule (dl_eval_schedule_build)
 *   dl_count_chain_block()         outputs a workgroup parks in LDS per block
 *   dl_count_chain_padded_steps()  HOST: steps rounded up to whole workgroups
 *   dl_count_chain_plan_build()    HOST pointers.  From the schedule's neuron [steps], out_dim and k
 *       writes slot [padded] and runs [padded / dl_count_chain_block() * k]: where every workgroup parks the outputs
 *       of a block so that they are sorted by class, and each class's run of slots; and *blocks:
 *       how many blocks of steps a workgroup walks (16 at most; fewer where a workgroup would
 *       otherwise count more than 255 neurons of one class).  Returns padded, or a negated
 *       dl_status: -DL_ERR_TOO_LARGE for k > 32 (the caller then uses
 *       dl_logic_eval_fused_groupbitsum).
 *   slot, runs, padded_steps, blocks   that plan (slot, runs: DEVICE copies; runs 4-byte aligned:
 *       the kernel reads its entries, whose number is even, two at a time)
 *   workspace DEVICE scratch of dl_logic_eval_chained_groupbitsum_workspace_bytes(...) bytes,
 *             16-byte aligned: one 16-byte record per step (composed per call from the schedule
 *             and the current gate ids), the bit-sliced partial counters, and the plan as
 *             thinned for this call (neurons of the top layer whose gate is constant, 0 or 15,
 *             are neither parked nor counted; what the ones add is put into the result at the end).
 * depth is 1 or 2; a, b are read for the layer below the top one only (a[0], b[0] at depth 2).
 * DL_ERR_TOO_LARGE: rows are not whole 64-bit words or k > 32. */
int dl_count_chain_block(void);
int64_t dl_count_chain_padded_steps(int64_t steps);
int64_t dl_count_chain_plan_build(const int32_t *neuron, int64_t steps, int64_t out_dim, int64_t k,
                                  uint8_t *slot, uint16_t *runs, int *blocks);
int64_t dl_logic_eval_chained_groupbitsum_workspace_bytes(int64_t padded_steps, int blocks,
                                                          int64_t words, int bit_count, int64_t k);
int dl_logic_eval_chained_groupbitsum(const void *x, int depth, const int64_t *const *a,
                                      const int64_t *const *b, const uint8_t *const *w,
                                      const int64_t *dims, const int32_t *verts,
                                      const int32_t *neuron, const uint8_t *flip, int64_t steps,
                                      const uint8_t *slot, const uint16_t *runs,
                                      int64_t padded_steps, int blocks, int32_t *out,
                                      int64_t words, int bit_count, int64_t pad_len, int64_t k,
                                      void *workspace, void *stream);

/* A whole narrow net and its `groupbitsum` in one kernel that keeps the activations in LDS (the
 * per-layer loop difflogic/difflogic.py:147 over every layer of the model, then
 * difflogic/packbitstensor.py:22): a workgroup carries a few 64-bit word columns of the packed
 * input through all `depth` layers and counts the last layer's outputs per class; memory sees
 * the packed input once and the counts once.  No counterpart in the reference.  Arguments as
 * dl_logic_eval_fused_groupbitsum, with depth up to 16; result identical to dl_groupbitsum after
 * `depth` calls of dl_logic_eval.
 *   Applies when dims[0..depth] <= dl_logic_net_lds_max_width() and rows are whole 64-bit words
 *   (8-byte aligned x); otherwise DL_ERR_TOO_LARGE is returned and the caller uses the streaming
 *   entry points.
 *   workspace DEVICE scratch of dl_logic_net_lds_workspace_bytes(depth, dims) bytes, 4-byte
 *             aligned: the per-gate records and row ids, rebuilt by every call.
 *   dl_logic_net_lds_groupbitsum_scheduled() additionally takes, per hidden layer l < depth - 1, the
 *   DEVICE copies of that layer's evaluation schedule (HOST arrays verts, neuron, flip of depth - 1
 *   DEVICE pointers and HOST steps [depth - 1]; a NULL entry leaves the layer as it is): such a
 *   layer is walked along its trails inside the kernel, which nearly halves its LDS row reads.
 *   Same result; same workspace size.
 *   dl_logic_net_lds_groupbitsum_bool() takes the bool matrix x [batch, dims[0]] itself (sample-major,
 *   one byte per value, any non-zero byte true: what PackBitsTensor.__init__ receives,
 *   difflogic/packbitstensor.py:6-16) and packs it on the way into LDS, so the pack kernel and the packed
 *   input do not exist; out [batch, k].  Applies when dims[0] is a multiple of 16, x is 16-byte aligned
 *   and the input fits the LDS buffer next to the widest hidden layer (dims[0] + max hidden width <=
 *   dl_logic_net_lds_max_width()); otherwise DL_ERR_TOO_LARGE. */
int64_t dl_logic_net_lds_max_width(void);
int64_t dl_logic_net_lds_workspace_bytes(int depth, const int64_t *dims);
int dl_logic_net_lds_groupbitsum(const void *x, int depth, const int64_t *const *a,
                                 const int64_t *const *b, const uint8_t *const *w,
                                 const int64_t *dims, int32_t *out, int64_t words, int bit_count,
                                 int64_t pad_len, int64_t k, void *workspace, void *stream);
int dl_logic_net_lds_groupbitsum_scheduled(const void *x, int depth, const int64_t *const *a,
                                           const int64_t *const *b, const uint8_t *const *w,
                                           const int64_t *dims, const int32_t *const *verts,
                                           const int32_t *const *neuron, const uint8_t *const *flip,
                                           const int64_t *steps, int32_t *out, int64_t words,
                                           int bit_count, int64_t pad_len, int64_t k, void *workspace,
                                           void *stream);
int dl_logic_net_lds_groupbitsum_bool(const uint8_t *x, int64_t batch, int depth,
                                      const int64_t *const *a, const int64_t *const *b,
                                      const uint8_t *const *w, const int64_t *dims,
                                      const int32_t *const *verts, const int32_t *const *neuron,
                                      const uint8_t *const *flip, const int64_t *steps, int32_t *out,
                                      int64_t k, void *workspace, void *stream);

/* dl_logic_net_lds_groupbitsum / _bool with the net thinned for this call: what no gate looks at is neither
 * evaluated nor stored (the reference evaluates every gate of every layer, difflogic/difflogic.py:147; its
 * generated C leaves the same pruning to gcc).  Before the net runs, one small kernel folds constants through the
 * gate ids `w` (a gate that reads a constant neuron becomes the one-input gate it amounts to) and marks, from the
 * last layer downwards, the neurons that some gate above still looks at; the net kernel then evaluates, per hidden
 * layer, the marked neurons only (renumbered in their order, neuron by neuron: two row reads per gate, no
 * schedules), per class the non-constant neurons of the last layer, and adds the constant ones of a class to every
 * sample's count.  Same result as the other entry points, bit for bit; pays where well below all of the neurons are
 * looked at (uniformly drawn ids: about 55 %).
 *   bool_input != 0: x is the bool matrix [batch, dims[0]] as for dl_logic_net_lds_groupbitsum_bool (words,
 *   bit_count, pad_len unused); else packed words as for dl_logic_net_lds_groupbitsum (batch unused).
 *   folded != 0: the gate ids `w` have the constants folded in already (dl_gate_ids_folded layer by layer, or
 *   dl_fold_gate_constants): the folding kernels are left out.  (Ids that are not folded give the same counts
 *   passed this way; a constant neuron that a gate still looks at is then kept and evaluated like any other.)
 *   workspace, limits and status codes as for those. */
int dl_logic_net_lds_groupbitsum_thinned(const void *x, int bool_input, int64_t batch, int depth,
                                         const int64_t *const *a, const int64_t *const *b, const uint8_t *const *w,
                                         int folded, const int64_t *dims, int32_t *out, int64_t words, int bit_count,
                                         int64_t pad_len, int64_t k, void *workspace, void *stream);

/* dl_logic_eval_fused_groupbitsum without a workspace argument, for callers that cannot allocate
 * device memory: code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  It has no counterpart in the reference (whose functions allocate their outputs and
 * scratch through torch, difflogic/cuda/difflogic_kernel.cu:316,518,615,688).  The workspace is a
 * static device array of DL_STATIC_SCRATCH_BYTES inside the library; every GPU the library runs
 * on holds its own copy until the process ends.  The call allocates and frees nothing and runs
 * the same kernels as dl_logic_eval_fused_groupbitsum, with the same arguments, results and
 * status codes, plus:
 *   DL_ERR_SCRATCH_LIMIT  dl_logic_eval_fused_groupbitsum_workspace_bytes(depth, dims[depth],
 *                         words, bit_count, k) exceeds DL_STATIC_SCRATCH_BYTES (split the batch);
 *   DL_ERR_TOO_LARGE      rows are not whole 64-bit words (no per-layer fallback exists here).
 *   DL_ERR_CAPTURING      the first call on a device, which looks the array's address up with a
 *                         runtime call, was made while `stream` is being captured into a graph
 *                         (make one call on the device before capturing).
 * The array takes DL_STATIC_SCRATCH_BYTES of device memory in every process that loads the
 * library, on every GPU it uses, whether or not this entry point is ever called.
 * All calls on one GPU share that GPU's array: calls that overlap in time on one GPU (different
 * streams or threads) race; calls ordered on one stream do not.  Nothing in the array needs to be
 * cleared between calls. */
#define DL_STATIC_SCRATCH_BYTES (64u << 20)
int dl_logic_eval_fused_groupbitsum_noalloc(const void *x, int depth, const int64_t *const *a,
                                            const int64_t *const *b, const uint8_t *const *w,
                                            const int64_t *dims, int32_t *out, int64_t words,
                                            int bit_count, int64_t pad_len, int64_t k,
                                            const int32_t *order, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* DIFFLOGIC_HIP_H */
