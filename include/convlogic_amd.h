/* convlogic_amd -- C ABI of the MI355X (gfx950) logic-layer kernels.
 *
 * Every entry point is a plain `extern "C"` function taking raw DEVICE pointers,
 * sizes and a HIP stream (passed as void*, may be NULL for the default stream).
 * Nothing here allocates, frees or synchronises: outputs and scratch buffers are
 * provided by the caller, kernels are enqueued on `stream` and the call returns.
 *
 * Return value: 0 on success, a negative CLG_E* code on a rejected argument or a
 * failed launch; clg_last_error() then returns a human readable message for the
 * calling thread.  Bad arguments are rejected on the host before any launch, and so are
 * sizes beyond what a kernel indexes: more than 65535 logic kernels per fused block in the
 * gradients and most forward kernels, in_dim / out_dim of 2^31 and above, element counts of
 * 2^31 and above where an entry point says so in its message.
 *
 * Each declaration cites the function of the reference's native extension modules
 * (`difflogic_cuda`, `convlogic_cuda`; paths relative to the reference checkout) that
 * it stands in for.
 *
 * Conventions
 *   dtype           CLG_F32 or CLG_F64 (all float tensors of a call share it); CLG_F16 where an entry point says so
 *   gate weights w  [..., 16] probabilities per gate (softmax or one-hot), gate ids
 *                   as in src/difflogic/functional.py:7-24
 *   selection       int32 [C, 8], tap = ch << 16 | row << 8 | col
 *                   (src/convlogic/convlogic_layer.py:450-452)
 *   all tensors are dense, row-major, in the shapes written beside each pointer.
 */
#ifndef CONVLOGIC_AMD_H
#define CONVLOGIC_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CLG_F32 0
#define CLG_F64 1
#define CLG_F16 2 /* IEEE half as a storage format of clg_fc_forward / _backward_w / _backward_x (arithmetic in float32) */

#define CLG_OK 0
#define CLG_EINVAL (-1)  /* rejected argument (shape, dtype, null pointer, limit) */
#define CLG_ELAUNCH (-2) /* hipLaunch / HIP runtime error */

/* Message describing the last error on the calling thread ("" if none). */
const char *clg_last_error(void);
/* ABI version of this library (bumped on incompatible changes). */
int clg_abi_version(void);

/* The CLG_* environment variables (tuning and path-forcing knobs) are read once per process; this reads them again
 * after the environment was changed.  Not synchronised with calls on other threads.  No counterpart in the reference. */
void clg_reload_knobs(void);

/* Geometry of a logic convolution (src/convlogic/convlogic_layer.py:94-109,192-193). */
typedef struct clg_conv_geom {
    int32_t n, c_in, h, w;   /* input  [n, c_in, h, w]            */
    int32_t c_out;           /* logic kernels (output channels)   */
    int32_t stride_h, stride_w, pad_h, pad_w, kernel_h, kernel_w;
} clg_conv_geom;

/* ---------------------------------------------------------------------------------
 * fully connected LogicLayer, feature-major like the reference extension
 * ------------------------------------------------------------------------------- */

/* y[j][s] = sum_i w[j][i] * op_i(x[a[j]][s], x[b[j]][s]).
 * Replaces difflogic_cuda.forward -- src/difflogic/cuda/difflogic.cpp:17,
 * logic_layer_cuda_forward src/difflogic/cuda/difflogic_kernel.cu:89-126.  dtype may be CLG_F16 here and in
 * clg_fc_backward_w / clg_fc_backward_x (the reference dispatches these three for half as well, :108,146,249). */
int clg_fc_forward(int dtype, const void *x /*[in_dim,batch]*/, const int64_t *a /*[out_dim]*/,
                   const int64_t *b /*[out_dim]*/, const void *w /*[out_dim,16]*/, void *y /*[out_dim,batch]*/,
                   int64_t in_dim, int64_t out_dim, int64_t batch, void *stream);

/* grad_w[j][i] = sum_s grad_y[j][s] * op_i(x[a[j]][s], x[b[j]][s]) (column 0 is exactly 0).
 * Replaces difflogic_cuda.backward_w -- src/difflogic/cuda/difflogic.cpp:18,
 * logic_layer_cuda_backward_w src/difflogic/cuda/difflogic_kernel.cu:128-173. */
int clg_fc_backward_w(int dtype, const void *x /*[in_dim,batch]*/, const int64_t *a, const int64_t *b,
                      const void *grad_y /*[out_dim,batch]*/, void *grad_w /*[out_dim,16]*/, int64_t in_dim,
                      int64_t out_dim, int64_t batch, void *stream);

/* grad_x[i][s] = sum over neurons reading input i of grad_y * d y / d x_i, gathered through the
 * reverse map (csr_start [in_dim+1], csr_list [2*out_dim]) built as in
 * src/difflogic/difflogic.py:71-87.  No atomics: the result is bitwise reproducible.
 * A neuron whose two inputs are the same feature contributes d/da + d/db (the derivative of the
 * reference's python path).
 * Replaces difflogic_cuda.backward_x -- src/difflogic/cuda/difflogic.cpp:19,
 * logic_layer_cuda_backward_x src/difflogic/cuda/difflogic_kernel.cu:232-269. */
int clg_fc_backward_x(int dtype, const void *x /*[in_dim,batch]*/, const int64_t *a, const int64_t *b,
                      const void *w /*[out_dim,16]*/, const void *grad_y /*[out_dim,batch]*/,
                      const int64_t *csr_start /*[in_dim+1]*/, const int64_t *csr_list /*[2*out_dim]*/,
                      void *grad_x /*[in_dim,batch]*/, int64_t in_dim, int64_t out_dim, int64_t batch,
                      void *stream);

/* clg_fc_backward_w followed by the softmax backward in the same kernel: with w = softmax(logits) the
 * result is the gradient w.r.t. the logits, p_i (g_i - sum_j p_j g_j) per neuron.  Replaces
 * difflogic_cuda.backward_w plus the autograd node of the softmax in LogicLayer.forward_cuda
 * (src/difflogic/difflogic.py:138, :226-228). */
int clg_fc_backward_logits(int dtype, const void *x, const int64_t *a, const int64_t *b, const void *w /*[out_dim,16]*/,
                           const void *grad_y, void *grad_logits /*[out_dim,16]*/, int64_t in_dim, int64_t out_dim,
                           int64_t batch, void *stream);

/* The training step of the module folds each neuron's 16 gate probabilities to the 4 coefficients of
 * y = c_ab*a*b + c_a*a + c_b*b + c_1 once, instead of in every wavefront that touches the neuron:
 *   clg_fc_fold            w_in [out_dim,16] (logits when from_logits != 0, else probabilities) ->
 *                          probs [out_dim,16] (softmax of the logits; may be NULL) and folded [out_dim,4]
 *   clg_fc_forward_folded  clg_fc_forward with folded in place of w
 *   clg_fc_backward_x_folded  clg_fc_backward_x with folded in place of w
 * The two kernels give the values of clg_fc_forward / clg_fc_backward_x on the same probabilities and,
 * when a row of `batch` samples fills fewer than 64 lanes, put 2 or 4 rows into a wavefront.  Replace the
 * softmax of LogicLayer.forward_cuda (src/difflogic/difflogic.py:138) plus difflogic_cuda.forward /
 * backward_x (src/difflogic/cuda/difflogic.cpp:18-19). */
int clg_fc_fold(int dtype, int from_logits, const void *w_in /*[out_dim,16]*/, void *probs /*[out_dim,16] or NULL*/,
                void *folded /*[out_dim,4]*/, int64_t out_dim, void *stream);
/* clg_fc_fold from logits for up to 16 tensors in ONE launch: logits[i] [rows[i], 16] -> probs[i] [rows[i], 16] and
 * folded[i] [rows[i], 4], row by row the values of clg_fc_fold and of the set-up launch of clg_convblock_forward_ex
 * (rows = c_out * 7 there, folded = probs + rows * 16).  For a network that folds all its layers at the start of a
 * training step and hands the results to clg_fc_forward_folded and to clg_convblock_forward_ex (CLG_FWD_FOLDED_IN);
 * logits, probs, folded, rows: host arrays of n entries.  No counterpart in the reference (torch.softmax per layer,
 * src/difflogic/difflogic.py:138, src/convlogic/convlogic_layer.py:321). */
int clg_fold_many(int dtype, int n, const void *const *logits, void *const *probs, void *const *folded, const int64_t *rows,
                  void *stream);
int clg_fc_forward_folded(int dtype, const void *x, const int64_t *a, const int64_t *b, const void *folded /*[out_dim,4]*/,
                          void *y, int64_t in_dim, int64_t out_dim, int64_t batch, void *stream);
int clg_fc_backward_x_folded(int dtype, const void *x, const int64_t *a, const int64_t *b, const void *folded,
                             const void *grad_y, const int64_t *csr_start, const int64_t *csr_list, void *grad_x,
                             int64_t in_dim, int64_t out_dim, int64_t batch, void *stream);

/* Both gradients of a layer in which every input feature is read by exactly one neuron operand (the caller
 * guarantees it; 2*out_dim == in_dim is checked): the neuron that reads a feature writes its grad_x row, so
 * the pass over the CSR map is not needed.  grad_w holds the gradient w.r.t. the probabilities, or w.r.t. the
 * logits when probs [out_dim,16] = softmax(logits) is given (NULL otherwise).  Same values as
 * clg_fc_backward_x_folded + clg_fc_backward_w / clg_fc_backward_logits.  Replaces difflogic_cuda.backward_x
 * and backward_w (src/difflogic/cuda/difflogic.cpp:18-19) for the halving layers of the reference's models
 * (src/convlogic/model.py:49-55, :102-103). */
int clg_fc_backward_sole(int dtype, const void *x, const int64_t *a, const int64_t *b, const void *folded /*[out_dim,4]*/,
                         const void *probs /*[out_dim,16] or NULL*/, const void *grad_y, void *grad_x, void *grad_w,
                         int64_t in_dim, int64_t out_dim, int64_t batch, void *stream);
/* The same when the layer's output goes straight into a GroupSum (the last two modules of the reference's models,
 * src/convlogic/model.py:55-57): grad_out [batch, k] is the gradient of the GroupSum's OUTPUT, and the gradient of neuron
 * j's row, grad_out[b][j / (out_dim / k)] * (1 / tau), is formed inside the kernel -- the values clg_group_sum_backward
 * would write and this call read back, bit for bit, without that launch and without the [out_dim, batch] tensor. */
int clg_fc_backward_sole_classes(int dtype, const void *x, const int64_t *a, const int64_t *b, const void *folded /*[out_dim,4]*/,
                                 const void *probs /*[out_dim,16] or NULL*/, const void *grad_out /*[batch,k]*/, void *grad_x,
                                 void *grad_w, int64_t in_dim, int64_t out_dim, int64_t batch, int64_t k, double tau, void *stream);

/* clg_fc_fold (from logits) + clg_fc_forward_folded in one launch: y from the LOGITS [out_dim, 16]; their softmax goes to
 * probs [out_dim, 16] and its 4 folded coefficients per neuron to folded [out_dim, 4] for the backward entry points
 * (the 16 lanes of a lane row hold a neuron's logits; sums are DPP trees, so probs agree with clg_fc_fold to rounding).
 * Replaces torch.softmax(self.weights) + difflogic_cuda.forward of LogicLayer.forward_cuda
 * (src/difflogic/difflogic.py:130-141) in the module's training path. */
int clg_fc_forward_logits(int dtype, const void *x, const int64_t *a, const int64_t *b, const void *logits,
                          void *probs /*[out_dim,16]*/, void *folded /*[out_dim,4]*/, void *y, int64_t in_dim, int64_t out_dim,
                          int64_t batch, void *stream);

/* Both gradients of a layer with ANY wiring in one pass, for batches that one pass of a wavefront row covers
 * (clg_fc_backward_fused_fits() != 0: batch <= 256 for float32 batches divisible by 4, 128 for float64 batches divisible
 * by 2, 64 otherwise): the walk of clg_fc_backward_x_folded also forms each neuron's weight-gradient sums on the visit
 * through the neuron's first operand.  grad_x and grad_w as clg_fc_backward_x_folded + clg_fc_backward_w /
 * clg_fc_backward_logits (probs given), bit for bit.  Replaces difflogic_cuda.backward_x + backward_w
 * (src/difflogic/cuda/difflogic_kernel.cu:153-269) in the module's training path. */
int clg_fc_backward_fused_fits(int dtype, int64_t batch);
int clg_fc_backward_fused(int dtype, const void *x, const int64_t *a, const int64_t *b, const void *folded /*[out_dim,4]*/,
                          const void *probs /*[out_dim,16] or NULL*/, const void *grad_y, const int64_t *csr_start,
                          const int64_t *csr_list, void *grad_x, void *grad_w, int64_t in_dim, int64_t out_dim, int64_t batch,
                          void *stream);
/* The same with flags, for a layer called on [batch, features] tensors (src/difflogic/difflogic.py:125-147, :214-230 make a
 * transposed copy of x, of grad_y and of grad_x there):
 *   CLG_FC_GX_SAMPLE_MAJOR  grad_x is written sample-major, [batch, in_dim], straight from the kernel; same values bit for bit
 *   CLG_FC_GY_SAMPLE_MAJOR  grad_y is [batch, out_dim]; its feature-major copy is made into scratch (out_dim * batch elements)
 *                           by the same call */
#define CLG_FC_GX_SAMPLE_MAJOR 1
#define CLG_FC_GY_SAMPLE_MAJOR 2
int clg_fc_backward_fused_ex(int dtype, const void *x, const int64_t *a, const int64_t *b, const void *folded /*[out_dim,4]*/,
                             const void *probs /*[out_dim,16] or NULL*/, const void *grad_y, const int64_t *csr_start,
                             const int64_t *csr_list, void *grad_x, void *grad_w, int64_t in_dim, int64_t out_dim, int64_t batch,
                             int flags, void *scratch /*or NULL*/, void *stream);
/* clg_fc_forward_logits with flags: CLG_FC_X_SAMPLE_MAJOR takes x as [batch, in_dim] and leaves its feature-major copy
 * [in_dim, batch] in x_fm (what the backward entry points read) -- the x.transpose(0, 1).contiguous() of
 * LogicLayer.forward_cuda (src/difflogic/difflogic.py:130-133) and the forward in one call. */
#define CLG_FC_X_SAMPLE_MAJOR 1
int clg_fc_forward_logits_ex(int dtype, const void *x, const int64_t *a, const int64_t *b, const void *logits,
                             void *probs /*[out_dim,16]*/, void *folded /*[out_dim,4]*/, void *y, int64_t in_dim, int64_t out_dim,
                             int64_t batch, int flags, void *x_fm /*[in_dim,batch] or NULL*/, void *stream);

/* GroupSum on feature-major activations x [features, batch] (what the last LogicLayer produces): out[b][g] =
 * (sum of the features/k rows of class g) * (1 / tau), the reciprocal rounded to dtype as torch's division of a
 * device tensor by a scalar does; fixed summation order (reproducible).
 * scratch: clg_group_sum_scratch_bytes().  Replaces x.reshape(..., k, F/k).sum(-1) / tau of
 * src/difflogic/difflogic.py:203-208 without the transposed copy. */
int64_t clg_group_sum_scratch_bytes(int dtype, int64_t features, int64_t batch, int64_t k);
int clg_group_sum(int dtype, const void *x, void *out /*[batch,k]*/, void *scratch, int64_t features, int64_t batch,
                  int64_t k, double tau, void *stream);
/* The same sums in ONE launch and without scratch, for classes of 64 to 4096 rows with enough (class, 32 samples) pairs
 * to fill the GPU (clg_group_sum_once_fits() != 0; the last layer of the reference's CIFAR and MNIST models at training
 * batch sizes): a workgroup owns a class and 32 samples.  Fixed summation order, which is not that of clg_group_sum (the
 * values agree to rounding, not bit for bit).  Other sizes: CLG_EINVAL. */
int clg_group_sum_once_fits(int64_t features, int64_t batch, int64_t k);
int clg_group_sum_once(int dtype, const void *x /*[features,batch]*/, void *out /*[batch,k]*/, int64_t features, int64_t batch,
                       int64_t k, double tau, void *stream);
/* clg_group_sum for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc): no scratch argument -- the partial sums go to a buffer of
 * clg_group_sum_static_max_bytes() bytes (1 MiB) that is part of the library image, one copy per GPU, held until the
 * process ends.  Sizes whose partial sums (at most 64 * k * batch elements, fewer for few rows per class) do not fit are
 * rejected with CLG_EINVAL.  The call itself allocates and frees nothing.  Every call on a GPU uses that GPU's one
 * buffer: calls that overlap on one GPU (different streams or threads) race; calls on one stream are ordered.  Same
 * values as clg_group_sum, bit for bit.  The first call on a device asks the runtime for the buffer's address
 * (hipGetSymbolAddress, not a stream operation): before CAPTURING the entry point into a HIP graph, call
 * clg_group_sum_static_init() -- or the entry point itself -- once on that device outside the capture.  No counterpart in
 * the reference. */
int64_t clg_group_sum_static_max_bytes(void);
int clg_group_sum_static_init(void);
int clg_group_sum_static(int dtype, const void *x /*[features,batch]*/, void *out /*[batch,k]*/, int64_t features,
                         int64_t batch, int64_t k, double tau, void *stream);
/* Its backward: grad_x[f][b] = grad_out[b][f / (features/k)] * (1 / tau). */
int clg_group_sum_backward(int dtype, const void *grad_out /*[batch,k]*/, void *grad_x /*[features,batch]*/,
                           int64_t features, int64_t batch, int64_t k, double tau, void *stream);

/* dst[c][r] = src[r][c] for elements of elem_size 1, 2, 4 or 8 bytes (layout change between the
 * module's [batch, features] tensors and the feature-major kernels; the reference does this with
 * x.transpose(0,1).contiguous(), src/difflogic/difflogic.py:130-131). */
int clg_transpose_2d(int elem_size, const void *src /*[rows,cols]*/, void *dst /*[cols,rows]*/, int64_t rows,
                     int64_t cols, void *stream);

/* ---------------------------------------------------------------------------------
 * packed-bit inference (PackBitsTensor)
 * ------------------------------------------------------------------------------- */

/* words[f][c] bit i = t[f][bit_count*c + i] (LSB first, zero padded); bit_count in {8,16,32,64};
 * words holds ceil(batch/bit_count) integers of bit_count bits per feature.
 * Replaces difflogic_cuda.tensor_packbits_cuda -- src/difflogic/cuda/difflogic.cpp:21,
 * src/difflogic/cuda/difflogic_kernel.cu:368-413. */
int clg_pack_bits(const uint8_t *t /*bool [features,batch]*/, void *words /*[features,ceil(batch/bit_count)]*/,
                  int64_t features, int64_t batch, int bit_count, void *stream);

/* Same result from the sample-major tensor t [batch, features] (what PackBitsTensor receives),
 * without materialising the transposed copy of src/difflogic/packbitstensor.py:18. */
int clg_pack_bits_sample_major(const uint8_t *t /*bool [batch,features]*/, void *words, int64_t features,
                               int64_t batch, int bit_count, void *stream);

/* y[j] = g_j(x[a[j]], x[b[j]]) bitwise on rows of `words` integers of elem_size bytes;
 * gate[j] in 0..15.  x and y must not overlap.
 * Replaces difflogic_cuda.eval -- src/difflogic/cuda/difflogic.cpp:20,
 * logic_layer_cuda_eval src/difflogic/cuda/difflogic_kernel.cu:295-330 (gate switch
 * src/common/cuda_utils.cuh:162-199). */
int clg_fc_eval_packed(int elem_size, const void *x /*[in_dim,words]*/, const int64_t *a, const int64_t *b,
                       const uint8_t *gate /*[out_dim]*/, void *y /*[out_dim,words]*/, int64_t in_dim,
                       int64_t out_dim, int64_t words, void *stream);

/* HOST function (plain host pointers, no GPU work): orders the neurons of a layer along trails of
 * its wiring graph (input rows = vertices, neurons = edges) so that consecutive neurons share an input
 * row.  plan [out_dim] is consumed by clg_fc_eval_packed_planned.  Computed once per wiring, like the
 * reverse map of src/difflogic/difflogic.py:71-87 is for the backward pass; no counterpart in the
 * reference's eval path. */
int clg_fc_eval_plan(const int64_t *a_host /*[out_dim]*/, const int64_t *b_host /*[out_dim]*/, int64_t in_dim,
                     int64_t out_dim, int32_t *plan_host /*[out_dim]*/);

/* gate[r] = index of the first maximum of the 16 logits of row r, for rows = out_dim (LogicLayer) or c_out * 7
 * (fused block); dtype CLG_F32, CLG_F64 or CLG_F16.  Replaces self.weights.argmax(-1).to(torch.uint8) of
 * LogicLayer.forward_cuda_eval (src/difflogic/difflogic.py:161), taken on every packed call as there. */
int clg_gate_argmax(int dtype, const void *logits /*[rows,16]*/, uint8_t *gate /*[rows]*/, int64_t rows, void *stream);

/* Same result as clg_fc_eval_packed, evaluated in plan order: the shared input row of consecutive
 * neurons stays in registers, so every input row is fetched about once instead of twice.  plan is
 * the DEVICE copy of clg_fc_eval_plan's output for the same (a, b).
 * Replaces difflogic_cuda.eval -- src/difflogic/cuda/difflogic_kernel.cu:295-330. */
int clg_fc_eval_packed_planned(int elem_size, const void *x /*[in_dim,words]*/, const int64_t *a, const int64_t *b,
                               const uint8_t *gate /*[out_dim]*/, const int32_t *plan /*[out_dim]*/,
                               void *y /*[out_dim,words]*/, int64_t in_dim, int64_t out_dim, int64_t words, void *stream);

/* clg_gate_argmax + clg_fc_eval_packed_planned in ONE launch: the kernel takes the arg-max of the 16 float32 logits of a
 * neuron itself (first maximum, a NaN counts as the maximum: the same gate ids, tested), so a packed layer call is a
 * single launch.  Needs rows the walk kernel takes -- clg_fc_eval_walk_fits(): whole 16-byte vectors, at least 1 KiB, x
 * and y 16-byte aligned -- and is rejected with CLG_EINVAL otherwise (use the two calls then).
 * Replaces `self.weights.argmax(-1).to(torch.uint8)` + difflogic_cuda.eval of LogicLayer.forward_cuda_eval
 * (src/difflogic/difflogic.py:149-164; src/difflogic/cuda/difflogic_kernel.cu:295-330). */
int clg_fc_eval_walk_fits(int elem_size, const void *x, const void *y, int64_t words);
int clg_fc_eval_packed_planned_logits(int elem_size, const void *x /*[in_dim,words]*/, const int64_t *a, const int64_t *b,
                                      const float *logits /*[out_dim,16]*/, const int32_t *plan /*[out_dim]*/,
                                      void *y /*[out_dim,words]*/, int64_t in_dim, int64_t out_dim, int64_t words, void *stream);

/* out[s][g] = number of features of class g (features/k consecutive rows) whose sample-s bit is set,
 * for s < words*8*elem_size - pad_len.  features must be divisible by k.
 * Replaces difflogic_cuda.groupbitsum -- src/difflogic/cuda/difflogic.cpp:22-33,
 * src/difflogic/cuda/difflogic_kernel.cu:450-482 (which returns the same [samples,k] layout). */
int clg_group_bit_sum(int elem_size, const void *x /*[features,words]*/, int32_t *out /*[samples,k]*/,
                      int64_t features, int64_t words, int64_t pad_len, int64_t k, void *stream);

/* ---------------------------------------------------------------------------------
 * split conv-logic layers (ConvLogicLayer(complete=False), TreeLogicLayer)
 * ------------------------------------------------------------------------------- */

/* y[n][c][oy][ox][p] = gate(w[c][p], tap 2p, tap 2p+1), taps outside the image read 0.
 * Replaces convlogic_cuda.convlogic_forward -- src/convlogic/cuda/convlogic.cpp:31,
 * src/convlogic/cuda/convlogic_kernel.cu:67-106. */
int clg_conv4_forward(int dtype, const clg_conv_geom *g, const void *x, const void *w /*[c_out,4,16]*/,
                      const int32_t *selection, void *y /*[n,c_out,ho,wo,4]*/, void *stream);

/* Deterministic (no float atomics) input gradient; grad_x is fully written.
 * Replaces convlogic_cuda.convlogic_backward_x -- src/convlogic/cuda/convlogic.cpp:32,
 * src/convlogic/cuda/convlogic_kernel.cu:321-359. */
int clg_conv4_backward_x(int dtype, const clg_conv_geom *g, const void *grad_y /*[n,c_out,ho,wo,4]*/,
                         const void *x, const void *w, const int32_t *selection, void *grad_x, void *stream);

/* grad_w [c_out,4,16] w.r.t. the gate probabilities.  scratch: clg_conv4_backward_w_scratch_bytes().
 * Replaces convlogic_cuda.convlogic_backward_weight -- src/convlogic/cuda/convlogic.cpp:33,
 * src/convlogic/cuda/convlogic_kernel.cu:197-248. */
int clg_conv4_backward_w(int dtype, const clg_conv_geom *g, const void *grad_y, const void *x,
                         const int32_t *selection, void *grad_w, void *scratch, void *stream);
int64_t clg_conv4_backward_w_scratch_bytes(int dtype, const clg_conv_geom *g);

/* One pairwise tree level: y[r][c][..][p] = gate(w[c][p], x[..][2p], x[..][2p+1]);
 * x [n,c,h,w,2*xo] -> y [n,c,h,w,xo].  `positions` = h*w.
 * Replaces convlogic_cuda.treelogic_forward -- src/convlogic/cuda/convlogic.cpp:35,
 * src/convlogic/cuda/treelogic_kernel.cu:46-85. */
int clg_tree_forward(int dtype, const void *x, const void *w /*[c,xo,16]*/, void *y, int64_t n, int64_t c,
                     int64_t positions, int64_t xo, void *stream);
/* Replaces convlogic_cuda.treelogic_backward_x -- src/convlogic/cuda/convlogic.cpp:36,
 * src/convlogic/cuda/treelogic_kernel.cu:252-285. */
int clg_tree_backward_x(int dtype, const void *grad_y, const void *x, const void *w, void *grad_x, int64_t n,
                        int64_t c, int64_t positions, int64_t xo, void *stream);
/* grad_w [c,xo,16].  scratch: clg_tree_backward_w_scratch_bytes().
 * Replaces convlogic_cuda.treelogic_backward_weight -- src/convlogic/cuda/convlogic.cpp:37,
 * src/convlogic/cuda/treelogic_kernel.cu:160-206 (without its xo <= 4 limit). */
int clg_tree_backward_w(int dtype, const void *grad_y, const void *x, void *grad_w, void *scratch, int64_t n,
                        int64_t c, int64_t positions, int64_t xo, void *stream);
int64_t clg_tree_backward_w_scratch_bytes(int dtype, int64_t n, int64_t c, int64_t positions, int64_t xo);

/* ---------------------------------------------------------------------------------
 * fused block: tap gather -> 4 leaf gates -> 2 gates -> root gate -> 2x2/2 max pool
 * (ConvLogicLayer(complete=True)); conv output height and width must be even.
 * ------------------------------------------------------------------------------- */

/* y [n,c_out,ho/2,wo/2]; argmax [n,c_out,ho/2,wo/2] holds dy*2+dx of the first maximum in window
 * order (0,0),(0,1),(1,0),(1,1) -- the position the reference stores as in_y*wo+in_x.
 * Nothing but y and one byte per pooled output is written.
 * Replaces convlogic_cuda.full_convlogic_forward -- src/convlogic/cuda/convlogic.cpp:39,
 * src/convlogic/cuda/full_convlogic_kernel.cu:147-231. */
int clg_convblock_forward(int dtype, const clg_conv_geom *g, const void *x, const void *w /*[c_out,7,16]*/,
                          const int32_t *selection, void *y, uint8_t *argmax, void *stream);

/* clg_convblock_forward with a caller-provided workspace of clg_convblock_forward_scratch_bytes() bytes
 * (0 for shapes that do not use one; scratch may then be NULL).  With a workspace, layers whose input
 * channels do not fit LDS read their taps from a zero-padded copy of x made in it instead of staging
 * channel subsets.  Same results as clg_convblock_forward; no counterpart in the reference (its forward,
 * src/convlogic/cuda/full_convlogic_kernel.cu:147-231, allocates its intermediates itself). */
int64_t clg_convblock_forward_scratch_bytes(int dtype, const clg_conv_geom *g);
int clg_convblock_forward_ws(int dtype, const clg_conv_geom *g, const void *x, const void *w, const int32_t *selection,
                             void *y, uint8_t *argmax, void *scratch, void *stream);

/* Packed-bit inference of the block: 64 samples per uint64 word, images word-group major
 * x [n, c_in, h, w] with n = ceil(samples / 64) groups (bit s of group g = sample 64 g + s),
 * gates uint8 [c_out, 7] = arg-max gate id of every tree node (0..3 leaves, 4..5 middle, 6 root),
 * y [n, c_out, ho/2, wo/2]; the 2x2 max pool of {0,1} values is the OR of the four positions.
 * The reference has no packed conv path (its packed kernels cover LogicLayer only,
 * src/difflogic/cuda/difflogic_kernel.cu:271-330); the result equals the eval-mode float block
 * (src/convlogic/convlogic_layer.py:231-316 with one-hot weights, :321-325) on binary inputs. */
int clg_convblock_eval_packed(const clg_conv_geom *g, const uint64_t *x, const uint8_t *gates,
                              const int32_t *selection, uint64_t *y, void *stream);

/* clg_convblock_eval_packed with a workspace, as clg_convblock_forward_ws. */
int64_t clg_convblock_eval_packed_scratch_bytes(const clg_conv_geom *g);
int clg_convblock_eval_packed_ws(const clg_conv_geom *g, const uint64_t *x, const uint8_t *gates,
                                 const int32_t *selection, uint64_t *y, void *scratch, void *stream);

/* Intermediates of the block for the return_intermediate / return_indices debug outputs:
 * x2 [n,c_out,ho,wo,4] (leaf gates), x3 [n,c_out,ho,wo,2]; either may be NULL.
 * (second and third result of full_convlogic_forward, full_convlogic_kernel.cu:172,194,230). */
int clg_convblock_intermediates(int dtype, const clg_conv_geom *g, const void *x, const void *w,
                                const int32_t *selection, void *x2, void *x3, void *stream);

/* Input gradient through the stored argmax position; deterministic, grad_x fully written.
 * scratch: clg_convblock_backward_x_scratch_bytes() bytes (folded gate coefficients).
 * Replaces convlogic_cuda.full_convlogic_backward_x -- src/convlogic/cuda/convlogic.cpp:40-41,
 * src/convlogic/cuda/full_convlogic_kernel.cu:365-461. */
int clg_convblock_backward_x(int dtype, const clg_conv_geom *g, const void *grad_y, const void *x, const void *w,
                             const int32_t *selection, const uint8_t *argmax, void *grad_x, void *scratch,
                             void *stream);
int64_t clg_convblock_backward_x_scratch_bytes(int dtype, const clg_conv_geom *g);

/* grad_w [c_out,7,16] w.r.t. the gate probabilities.  scratch: clg_convblock_backward_w_scratch_bytes().
 * Replaces convlogic_cuda.full_convlogic_backward_weight -- src/convlogic/cuda/convlogic.cpp:42-43,
 * src/convlogic/cuda/full_convlogic_kernel.cu:616-701. */
int clg_convblock_backward_w(int dtype, const clg_conv_geom *g, const void *grad_y, const void *x, const void *w,
                             const int32_t *selection, const uint8_t *argmax, void *grad_w, void *scratch,
                             void *stream);
int64_t clg_convblock_backward_w_scratch_bytes(int dtype, const clg_conv_geom *g);

/* Both gradients of the fused block in one call: clg_convblock_backward_x followed by
 * clg_convblock_backward_w on the same stream, sharing one scratch buffer of
 * clg_convblock_backward_scratch_bytes() bytes.
 * Replaces the pair full_convlogic_backward_x + full_convlogic_backward_weight as
 * FullConvLogicFunction.backward calls them -- src/convlogic/convlogic_layer.py:71-82. */
int clg_convblock_backward(int dtype, const clg_conv_geom *g, const void *grad_y, const void *x, const void *w,
                           const int32_t *selection, const uint8_t *argmax, void *grad_x, void *grad_w, void *scratch,
                           void *stream);
int64_t clg_convblock_backward_scratch_bytes(int dtype, const clg_conv_geom *g);

/* Both gradients of the block for a training step that owns the softmax: grad_x as clg_convblock_backward_x
 * (skipped when grad_x is NULL, e.g. for the first layer) and the gradient w.r.t. the LOGITS, i.e.
 * clg_convblock_backward_w followed by the softmax backward with w = softmax(logits), fused into the
 * final reduction.  scratch: clg_convblock_backward_scratch_bytes().  Replaces full_convlogic_backward_x +
 * full_convlogic_backward_weight (src/convlogic/convlogic_layer.py:71-82) plus the autograd node of the
 * softmax in ConvLogicLayer.forward_cuda (src/convlogic/convlogic_layer.py:321-323). */
int clg_convblock_backward_logits(int dtype, const clg_conv_geom *g, const void *grad_y, const void *x, const void *w,
                                  const int32_t *selection, const uint8_t *argmax, void *grad_x, void *grad_logits,
                                  void *scratch, void *stream);

/* The complete block with its output (and the output's gradient) laid out feature-major, [c_out, ho/2, wo/2, n] -- the
 * layout the LogicLayer behind nn.Flatten reads, so that neither direction needs a transposed copy.  For the shapes of
 * clg_convblock_fm_supported() != 0 (4x4 images, 3x3 kernel, stride 1, padding 1, n >= 32: the last block of a
 * 32x32-input network); argmax, x and grad_x keep their layouts.  Scratch: clg_convblock_forward_scratch_bytes /
 * clg_convblock_backward_scratch_bytes.  grad_w: gradient w.r.t. the logits when wrt_logits != 0 (w = their softmax),
 * else w.r.t. the probabilities w; grad_x may be NULL.  Same values as clg_convblock_forward_ws /
 * clg_convblock_backward(_logits) on the permuted tensors.  Replaces full_convlogic_forward / _backward_x /
 * _backward_weight (src/convlogic/cuda/convlogic.cpp:29-37) plus the copies around
 * x.transpose(0, 1).contiguous() in LogicLayer.forward_cuda (src/difflogic/difflogic.py:130-141). */
int clg_convblock_fm_supported(int dtype, const clg_conv_geom *g);
/* clg_convblock_forward_ws with options.  CLG_FWD_W_LOGITS: w holds the LOGITS [c_out, 7, 16]; their softmax is taken
 * while the gate parameters are set up (no separate softmax launch) and written to probs_out [c_out, 7, 16] for the
 * backward entry points -- replaces torch.softmax(self.weights) + full_convlogic_forward of ConvLogicLayer.forward_cuda
 * (src/convlogic/convlogic_layer.py:318-329).  CLG_FWD_Y_FEATURE_MAJOR: y laid out as for clg_convblock_forward_fm. */
#define CLG_FWD_W_LOGITS 1
#define CLG_FWD_Y_FEATURE_MAJOR 2
#define CLG_FWD_FOLDED_OUT 4 /* probs_out holds [c_out, 7, 16] probabilities FOLLOWED BY [c_out, 7, 4] folded coefficients
                              * (ab, a, b, 1 per gate) for clg_convblock_backward_planned; without CLG_FWD_W_LOGITS the
                              * probability part is left untouched (w already holds them) */
#define CLG_FWD_FOLDED_IN 8  /* with the two flags above: probs_out ALREADY holds the probabilities and the folded coefficients of
                              * w's logits (clg_fold_many at the start of the step): no softmax or fold launch in this call */
int clg_convblock_forward_ex(int dtype, const clg_conv_geom *g, const void *x, const void *w, const int32_t *selection, void *y,
                             uint8_t *argmax, void *probs_out, int flags, void *scratch, void *stream);
/* The same for packed words: y laid out [c_out, ho/2, wo/2, groups], which IS the feature-major [features, words] layout
 * of clg_fc_eval_packed (feature = (c, y, x) in nn.Flatten order), so PackBitsTensor.flatten needs no transpose. */
int clg_convblock_eval_packed_fm_supported(const clg_conv_geom *g);
int clg_convblock_eval_packed_fm(const clg_conv_geom *g, const uint64_t *x, const uint8_t *gates, const int32_t *selection,
                                 uint64_t *y /*[c_out,ho/2,wo/2,groups]*/, void *stream);
int clg_convblock_forward_fm(int dtype, const clg_conv_geom *g, const void *x, const void *w, const int32_t *selection,
                             void *y /*[c_out,ho/2,wo/2,n]*/, uint8_t *argmax, void *scratch, void *stream);
int clg_convblock_backward_fm(int dtype, const clg_conv_geom *g, const void *grad_y /*[c_out,ho/2,wo/2,n]*/, const void *x,
                              const void *w, const int32_t *selection, const uint8_t *argmax, void *grad_x, void *grad_w,
                              int wrt_logits, void *scratch, void *stream);

/* Per-layer plan of the block's backward pass: everything its kernels need that depends only on `selection` and the
 * geometry (the reverse map input channel -> kernels and taps in increasing kernel order and the tap offsets of the chosen
 * kernels' image layout), built ONCE per layer and batch shape instead of in every
 * backward call -- the counterpart of the reverse map that LogicLayer builds at construction
 * (src/difflogic/difflogic.py:71-87).  plan: clg_convblock_plan_bytes() bytes of device memory that the caller keeps;
 * *signature identifies what it was made for and is handed back to clg_convblock_backward_planned, which rejects a plan
 * made for another geometry, element type or kernel choice (the CLG_* knobs are part of the choice).  The backward calls
 * only read a plan. */
int64_t clg_convblock_plan_bytes(int dtype, const clg_conv_geom *g);
int clg_convblock_plan(int dtype, const clg_conv_geom *g, const int32_t *selection, void *plan, int64_t *signature, void *stream);
#define CLG_BWD_WRT_LOGITS 1       /* w = softmax(logits): grad_w is the gradient w.r.t. the logits */
#define CLG_BWD_GY_FEATURE_MAJOR 2 /* grad_y laid out [c_out, ho/2, wo/2, n] (shapes of clg_convblock_fm_supported) */
/* clg_convblock_backward / clg_convblock_backward_logits / clg_convblock_backward_fm (chosen by flags) with a plan: no list building per call, and with folded [c_out, 7, 4] (written by clg_convblock_forward_ex with
 * CLG_FWD_FOLDED_OUT for the same w; may be NULL) no set-up launch is left for blocks whose images fit LDS.  grad_x may
 * be NULL.  scratch: clg_convblock_backward_scratch_bytes().  Same values as the unplanned entry points.
 * Replaces full_convlogic_backward_x + full_convlogic_backward_weight (src/convlogic/convlogic_layer.py:71-82). */
int clg_convblock_backward_planned(int dtype, const clg_conv_geom *g, const void *grad_y, const void *x, const void *w,
                                   const void *folded, const int32_t *selection, const uint8_t *argmax, void *plan,
                                   int64_t signature, void *grad_x, void *grad_w, int flags, void *scratch, void *stream);

/* The padded hand-off.  The forward kernels of most shapes stage a zero-padded copy of x (in LDS, or in their scratch), and
 * the input gradient of layers with many channels reads its taps from exactly such a copy, which the backward call
 * otherwise makes in a launch of its own.  clg_convblock_padded_elems(): elements of that copy (n samples of
 * c_in * (h + ph) * (w + pw) + ph * (w + pw) + pw) when both sides have use for it at this shape, else 0.
 * clg_convblock_forward_padded = clg_convblock_forward_ex that also leaves the copy in padded_out;
 * clg_convblock_backward_planned_padded = clg_convblock_backward_planned that reads it (`padded` may be NULL: the plain
 * call) -- same values.  The reference pads x once per weight-gradient call (torch::constant_pad_nd,
 * src/convlogic/cuda/full_convlogic_kernel.cu:635) and bounds-checks every tap elsewhere (:16-33, :241-257); here one
 * padded copy per step serves the forward and both gradients. */
int64_t clg_convblock_padded_elems(int dtype, const clg_conv_geom *g, int have_scratch);
int clg_convblock_forward_padded(int dtype, const clg_conv_geom *g, const void *x, const void *w, const int32_t *selection, void *y,
                                 uint8_t *argmax, void *probs_out, int flags, void *scratch, void *padded_out, void *stream);
int clg_convblock_backward_planned_padded(int dtype, const clg_conv_geom *g, const void *grad_y, const void *x, const void *w,
                                          const void *folded, const void *padded, const int32_t *selection, const uint8_t *argmax,
                                          void *plan, int64_t signature, void *grad_x, void *grad_w, int flags, void *scratch,
                                          void *stream);

/* The fused block on BINARY inputs (every x is 0 or 1: the first block of a network, behind the threshold transform of
 * src/convlogic/data.py:46-50).  float32, stride 1, images at most 32 columns wide, at most 256 pooled cells (a multiple
 * of 4) per plane: clg_convblock_bin_supported.  A kernel's tree is then a 256-entry table over its 8 tap bits, made with
 * the same gate arithmetic as clg_convblock_forward, so y and the pooled position are bit-identical to that entry point.
 *   forward   y [n,c_out,ho/2,wo/2]; taps uint16 [n,c_out,ho/2,wo/2] = (dy*2+dx of the first maximum) << 8 | tap byte
 *             (bit i = tap i of the kernel at that position); ctx: clg_convblock_bin_ctx_bytes() bytes that the caller
 *             keeps for the backward call (bit rows of x, tables, folded coefficients, probabilities, per-channel
 *             kernel lists).  flags: CLG_FWD_W_LOGITS as for clg_convblock_forward_ex.  *not_binary (device-writable
 *             int32, e.g. pinned host memory) is set to 1 when some x is neither 0 nor 1 -- y is then undefined; it is
 *             never cleared.
 *   backward  from grad_y, taps and ctx alone (x is not read): grad_x [n,c_in,h,w] and / or grad_w [c_out,7,16]
 *             (either may be NULL); flags: CLG_BWD_WRT_LOGITS.  scratch: clg_convblock_bin_backward_scratch_bytes().
 *             Deterministic; equal to clg_convblock_backward(_logits) up to float rounding.
 * Replaces full_convlogic_forward / full_convlogic_backward_x / full_convlogic_backward_weight
 * (src/convlogic/cuda/convlogic.cpp:39-43; src/convlogic/cuda/full_convlogic_kernel.cu:10-145,233-363,463-701) for
 * binary inputs. */
int clg_convblock_bin_supported(int dtype, const clg_conv_geom *g);
/* Device address of a flag word in PINNED host memory (hipHostMalloc), for `not_binary`: the host can then read the flag
 * without a copy or a synchronisation.  CLG_EINVAL when `host` is not pinned memory mapped for the current device.  No
 * counterpart in the reference (its kernels do not check their inputs). */
int clg_host_flag_device_pointer(void *host, void **device);
int64_t clg_convblock_bin_ctx_bytes(int dtype, const clg_conv_geom *g);
int clg_convblock_bin_forward(int dtype, const clg_conv_geom *g, const void *x, const void *w, const int32_t *selection, void *y,
                              uint16_t *taps, void *ctx, int flags, int32_t *not_binary, void *stream);
int64_t clg_convblock_bin_backward_scratch_bytes(int dtype, const clg_conv_geom *g);
int clg_convblock_bin_backward(int dtype, const clg_conv_geom *g, const void *grad_y, const uint16_t *taps, const void *ctx,
                               void *grad_x, void *grad_w, int flags, void *scratch, void *stream);

/* ---------------------------------------------------------------------------------
 * input binarisation (the step in front of the first layer)
 * --------------------------------------------------------------------------------- */

/* out[s, l*c0 + c, p] = x[s, c, p] > thresholds[l] ? 1 : 0 for l < levels: the threshold-major channel
 * concatenation of the reference's input transform (torch.cat([(x > t).float() for t in thresholds]),
 * src/convlogic/data.py:46-50), applied to a batch x [n, c0, hw] of float32 images. */
int clg_threshold_images(const float *x, const float *thresholds, float *out /*[n, levels*c0, hw]*/, int64_t n,
                         int64_t c0, int64_t hw, int64_t levels, void *stream);

/* The same comparison written straight into packed words for clg_convblock_eval_packed:
 * words [ceil(n/64), levels*c0, hw], bit s of group g = sample 64 g + s (missing samples of the last
 * group are 0).  Fuses src/convlogic/data.py:46-50 with the packing of
 * src/difflogic/packbitstensor.py:12-21; the float {0,1} tensor is never materialised. */
int clg_threshold_pack_images(const float *x, const float *thresholds, uint64_t *words, int64_t n, int64_t c0,
                              int64_t hw, int64_t levels, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* CONVLOGIC_AMD_H */
