/*
 * C ABI of the gfx950 kernels behind the CoreScheduler op API.
 *
 * Every entry point takes plain device pointers, element counts, scalar
 * hyper-parameters and a HIP stream (passed as void*; NULL is the null
 * stream).  Entry points enqueue work on that stream and return; none of
 * them allocates device memory, synchronises the device or the stream, or
 * touches another stream.  Scratch memory, where a kernel needs it, is a
 * caller-owned `workspace` whose size the matching *_workspace_bytes call
 * reports.
 *
 * Return value: 0 on success, a negative CS_ERR_* for an argument the
 * library rejects before launching anything, a positive hipError_t when the
 * HIP runtime refused a launch.  cs_hip_error_string() names either kind.
 *
 * Each declaration cites the reference task body (file:line under the
 * CoreScheduler tree) whose device work it replaces.  The C++ task bodies
 * of cs::compute::{CrossEntropy,Embedding,LayerNorm,GeLU} and
 * cs::optimizer::AdamW are the intended callers; they turn a non-zero
 * return into CS_ASSERT_TRUE(false, ...).
 */
#ifndef CS_HIP_KERNELS_H_
#define CS_HIP_KERNELS_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* raised when an existing entry point changes its arguments or meaning; new entry points leave it */
#define CS_HIP_ABI_VERSION 1

/* element types */
enum cs_dtype {
  CS_F32 = 0,
  CS_F64 = 1,
  CS_F16 = 2,
  CS_BF16 = 3,
};

/* index types (the reference feeds int64 from its loader and int32 from its
 * tests: src/data/dataloader.cpp:165, test/test_embedding.cpp:72) */
enum cs_itype {
  CS_I32 = 0,
  CS_I64 = 1,
};

/* loss reductions; the values are at::Reduction's (None, Mean, Sum) as
 * stored in CrossEntropy::State::Args::reduction
 * (include/compute/cross_entropy.h:38-42) */
enum cs_reduction {
  CS_REDUCTION_NONE = 0,
  CS_REDUCTION_MEAN = 1,
  CS_REDUCTION_SUM = 2,
};

/* GeLU flavours: at::gelu's `approximate` argument ("none" / "tanh") */
enum cs_gelu_mode {
  CS_GELU_ERF = 0,
  CS_GELU_TANH = 1,
};

enum cs_error {
  CS_OK = 0,
  CS_ERR_INVALID_ARGUMENT = -1, /* null pointer, negative size, bad enum   */
  CS_ERR_UNSUPPORTED = -2,      /* dtype combination that has no kernel     */
  CS_ERR_MISALIGNED = -3,       /* pointer not aligned to its element size  */
  CS_ERR_WORKSPACE = -4,        /* workspace missing or too small           */
  CS_ERR_TOO_LARGE = -5,        /* size beyond what the launch can address  */
  CS_ERR_STATIC_LIMIT = -6,     /* size beyond the library's built-in scratch:
                                   use the entry point that takes a workspace */
};

int cs_hip_abi_version(void);
const char *cs_hip_error_string(int code);

/* Plain device-to-device copy of `bytes` (a multiple of 16, both pointers
 * 16-byte aligned) with the same 16-byte streaming accesses the ops use.  It
 * has no counterpart in the reference: it is the calibration kernel of the
 * benchmark (the bandwidth a trivial HBM-bound kernel reaches on this device,
 * and the scale of the hardware traffic counters). */
int cs_stream_copy(void *dst, const void *src, int64_t bytes, void *stream);

/* The two halves of that calibration, also without counterpart in the
 * reference: a read-only pass (every workgroup leaves one 32-bit word, the xor
 * of what it read, in out[0 .. cs_stream_read_out_words(bytes))) and a
 * write-only pass (dst filled with `value`).  Same rules for bytes and
 * alignment as cs_stream_copy. */
int64_t cs_stream_read_out_words(int64_t bytes);
int cs_stream_read(const void *src, void *out, int64_t bytes, void *stream);
int cs_stream_fill(void *dst, int64_t bytes, uint32_t value, void *stream);
/* cs_stream_fill in a chosen launch shape, for sweeping the write path (the
 * shape cs_stream_fill uses is the best of these): lanes per workgroup (256
 * or 1024), 16-byte vectors per lane (1, 2, 4, 8), lane-strided chunks or
 * (wave_kilobytes != 0) whole kilobytes per wave, nontemporal or
 * (plain_stores != 0) plain stores, one chunk per workgroup
 * (workgroups_per_cu == 0) or that many persistent workgroups per CU.
 * CS_ERR_UNSUPPORTED for a shape that is not built.  No counterpart in the
 * reference: a measurement aid like cs_stream_copy. */
int cs_stream_fill_shape(void *dst, int64_t bytes, uint32_t value, int lanes,
                         int vectors_per_lane, int wave_kilobytes,
                         int plain_stores, int workgroups_per_cu,
                         void *stream);

/* A fourth calibration with the memory traffic of the AdamW step and none of
 * its arithmetic: a0..a3 (`bytes` each) are read, a1..a3 rewritten in place
 * (a_k = (a0 ^ a1 ^ a2 ^ a3) + k per 32-bit word).  7 * bytes move; what this
 * reaches is the ceiling for a kernel that streams four arrays in and three
 * out.  No counterpart in the reference. */
int cs_stream_update4(const void *a0, void *a1, void *a2, void *a3,
                      int64_t bytes, void *stream);

/* ------------------------------------------------------------------------
 * AdamW
 * replaces stepKernel / stepKernelAmsgrad and the step<UpT,T> kernels,
 * src/optimizer/adamw.cu:35-60, :62-90, :93-151.
 *
 * All of w, dw, m, v (and v_max) hold `n` elements of `dtype`; arithmetic is
 * in float (double for CS_F64) in the reference's operation order.  The bias
 * corrections 1/(1-beta^t) are formed on the host in double and narrowed, as
 * adamw.cu:116-117 does.  v_max == NULL selects the plain step, non-NULL the
 * amsgrad step.  `t` is the step count AFTER the increment the caller makes
 * at submit time (src/optimizer/adamw.cpp:112), so the first step has t == 1.
 * ---------------------------------------------------------------------- */
int cs_adamw_step(void *w, const void *dw, void *m, void *v, void *v_max,
                  int64_t n, int dtype, double lr, double beta1, double beta2,
                  double eps, double weight_decay, int64_t t, void *stream);

/* One launch for a whole parameter set (the 148 launches per step of
 * src/module/adamw.cpp:32-38 become one).  The caller fills an array of
 * descriptors, asks the library to lay out a device table for them in HOST
 * memory, copies those bytes to the device itself (any way it likes) and
 * passes the device copy to the step.  Pointers in the table may be
 * refreshed and re-uploaded every step (gradients are re-allocated after
 * zero_grad in the reference: src/compute/embedding.cpp:54). */
typedef struct cs_adamw_tensor {
  void *w;
  const void *dw;
  void *m;
  void *v;
  void *v_max; /* NULL unless amsgrad */
  int64_t n;
} cs_adamw_tensor;

size_t cs_adamw_multi_table_bytes(int64_t n_tensors);
/* Writes the table for `tensors` into host_table (table_bytes long) and the
 * number of workgroup slots the launch needs into *n_slots.  The layout
 * depends on `dtype`; pass the same dtype to cs_adamw_multi_step. */
int cs_adamw_multi_build_table(const cs_adamw_tensor *tensors,
                               int64_t n_tensors, int dtype, void *host_table,
                               size_t table_bytes, int64_t *n_slots);
int cs_adamw_multi_step(const void *device_table, int64_t n_tensors,
                        int64_t n_slots, int dtype, int amsgrad, double lr,
                        double beta1, double beta2, double eps,
                        double weight_decay, int64_t t, void *stream);

/* Global gradient-norm clipping over the same table — Utils::clip_grad_norm_
 * (src/compute/utils.cpp:700-746), which the GPT-2 example leaves as a TODO
 * (example/gpt2/gpt2_single_device.cpp:706).  cs_grad_norm_multi writes
 *   *total_norm = || all gradients ||_p   (p = 2, or +infinity)
 *   *clip_coef  = min(1, max_norm / (total_norm + 1e-6))      (float arithmetic)
 * to device memory with two launches: one partial per workgroup slot, then a
 * sum in slot order in double (the result does not depend on scheduling).
 * The reference then multiplies every gradient in place; that pass is
 * cs_grad_scale_multi.  cs_adamw_multi_step_clipped instead reads the
 * coefficient inside the step and applies it to each gradient as it is
 * loaded (rounded to the gradient's type first, so the update is the one the
 * in-place clip followed by the plain step gives), leaving the gradients as
 * they were: one 4 B/parameter read instead of a read and a write more. */
size_t cs_grad_norm_multi_workspace_bytes(int64_t n_slots);
int cs_grad_norm_multi(const void *device_table, int64_t n_tensors,
                       int64_t n_slots, int dtype, double norm_type,
                       double max_norm, void *workspace, size_t workspace_bytes,
                       float *total_norm, float *clip_coef, void *stream);
int cs_grad_scale_multi(const void *device_table, int64_t n_tensors,
                        int64_t n_slots, int dtype, const float *clip_coef,
                        void *stream);
int cs_adamw_multi_step_clipped(const void *device_table, int64_t n_tensors,
                                int64_t n_slots, int dtype, int amsgrad,
                                double lr, double beta1, double beta2,
                                double eps, double weight_decay, int64_t t,
                                const float *clip_coef, void *stream);

/* ------------------------------------------------------------------------
 * GeLU
 * replaces at::gelu / at::gelu_backward in the task bodies of
 * src/compute/gelu.cpp:39 and :61-62 (erf form; the reference never passes
 * `approximate`).  CS_GELU_TANH is at::gelu(x, "tanh").  x, y, dy, dx hold
 * `n` elements of `dtype`; the arithmetic is fp32 for f16/bf16 storage.
 * ---------------------------------------------------------------------- */
int cs_gelu_forward(const void *x, void *y, int64_t n, int dtype, int mode,
                    void *stream);
int cs_gelu_backward(const void *dy, const void *x, void *dx, int64_t n,
                     int dtype, int mode, void *stream);

/* ------------------------------------------------------------------------
 * LayerNorm over the last dimension
 * forward replaces at::native_layer_norm, src/compute/layer_norm.cpp:163-169
 * and :198-204; backward replaces both at::native_layer_norm_backward calls,
 * :263-266 (dx) and :321-334 / :375-383 (dgamma, dbeta, with += when the
 * gradient already exists).
 *
 * x, y: [rows, C] row-major contiguous.  gamma, beta: [C] (beta may be NULL:
 * the reference's bias=false path).  mean, rstd: [rows] fp32 (fp64 when
 * x_dtype is CS_F64), rstd = 1/sqrt(biased variance + eps).
 * x_dtype: storage of x.  y_dtype: storage of y, either x_dtype or CS_F32
 * (what autocast produces for bf16 x).  param_dtype: storage of gamma/beta,
 * either x_dtype or CS_F32.
 * ---------------------------------------------------------------------- */
int cs_layernorm_forward(const void *x, const void *gamma, const void *beta,
                         void *y, void *mean, void *rstd, int64_t rows,
                         int64_t C, double eps, int x_dtype, int y_dtype,
                         int param_dtype, void *stream);

size_t cs_layernorm_backward_workspace_bytes(int64_t rows, int64_t C);
/* Any of dx, dgamma, dbeta may be NULL (the reference's output masks
 * {1,0,0}, {0,1,1}, {0,1,0}); dgamma/dbeta are stored in param_dtype and,
 * when accumulate != 0, added to what is already there.  dy is stored as
 * dy_dtype (x_dtype or CS_F32), dx as dx_dtype (same choice).  workspace
 * is needed whenever dgamma or dbeta is requested. */
int cs_layernorm_backward(const void *dy, const void *x, const void *mean,
                          const void *rstd, const void *gamma, void *dx,
                          void *dgamma, void *dbeta, void *workspace,
                          size_t workspace_bytes, int64_t rows, int64_t C,
                          int dy_dtype, int x_dtype, int dx_dtype,
                          int param_dtype, int accumulate, void *stream);

/* The residual stream around LayerNorm, in one call (the transformer block
 * of example/gpt2/gpt2_single_device.cpp:457-464 and :467-474):
 *   forward : sum_out = x + residual;  y = LayerNorm(sum_out)
 *             replaces Utils::add (:459) followed by ln2->forward (:460)
 *   backward: dx = LayerNorm_backward(dy) + dresidual
 *             replaces ln2->backward (:468) followed by Utils::add (:469)
 * Results are those of the two separate kernels, bit for bit: the sum is
 * rounded to x_dtype before it is normalised, and dx is rounded to dx_dtype
 * before dresidual is added.  Both adds run inside the LayerNorm kernel, which
 * saves a [rows, C] round trip and a launch: forward for every row width the
 * row-in-registers kernels take (up to 512 16-byte vectors: C <= 4096 for
 * 16-bit x), backward for rows of up to 256 vectors (C <= 2048 at 16 bit);
 * other shapes run an elementwise add launch next to the LayerNorm launch.
 * residual and sum_out are [rows, C] of x_dtype (sum_out may be x or residual
 * itself); dresidual is [rows, C] of dx_dtype (dx may be dresidual itself).
 * All other arguments as in the plain calls. */
int cs_add_layernorm_forward(const void *x, const void *residual,
                             void *sum_out, const void *gamma,
                             const void *beta, void *y, void *mean, void *rstd,
                             int64_t rows, int64_t C, double eps, int x_dtype,
                             int y_dtype, int param_dtype, void *stream);
int cs_layernorm_backward_add(const void *dy, const void *x, const void *mean,
                              const void *rstd, const void *gamma,
                              const void *dresidual, void *dx, void *dgamma,
                              void *dbeta, void *workspace,
                              size_t workspace_bytes, int64_t rows, int64_t C,
                              int dy_dtype, int x_dtype, int dx_dtype,
                              int param_dtype, int accumulate, void *stream);

/* LayerNorm backward as the reference schedules it: the input gradient is a
 * task on the main stream (src/compute/layer_norm.cpp:235-283, kMain), the
 * parameter gradients a task on the assist stream (:285-400, kAssist).  Here
 * the first task reads dy and x once and leaves, next to dx, per-workgroup
 * column sums of dy*xhat and dy ("partial rows", fp32 [partial_rows, 2, C]);
 * the second adds those rows in a fixed order, which is a few hundred KB of
 * work and can run on another stream while the main stream goes on.  The pair
 * gives the bits of cs_layernorm_backward (same kernels, same order).
 *
 * cs_layernorm_backward_partial_rows: rows of the partial buffer for this
 *   shape (the buffer holds partial_rows * 2 * C floats), or 0 when the shape
 *   has no split form (C not a multiple of the 16-byte vector, rows wider than
 *   512 vectors, CS_F64): use cs_layernorm_backward then.
 * cs_layernorm_backward_rows: dx (may be NULL) and the partial rows;
 *   dresidual as in cs_layernorm_backward_add or NULL.  All pointers 16-byte
 *   aligned (CS_ERR_MISALIGNED otherwise).
 * cs_layernorm_backward_finalize: dgamma / dbeta (either may be NULL) from the
 *   partial rows; x_dtype is the one the rows call was given (it fixes the
 *   column order inside a partial row). */
int64_t cs_layernorm_backward_partial_rows(int64_t rows, int64_t C, int x_dtype);
int cs_layernorm_backward_rows(const void *dy, const void *x, const void *mean,
                               const void *rstd, const void *gamma,
                               const void *dresidual, void *dx, void *partials,
                               size_t partials_bytes, int64_t rows, int64_t C,
                               int dy_dtype, int x_dtype, int dx_dtype,
                               int param_dtype, void *stream);
int cs_layernorm_backward_finalize(const void *partials, int64_t partial_rows,
                                   void *dgamma, void *dbeta, int64_t C,
                                   int x_dtype, int param_dtype, int accumulate,
                                   void *stream);

/* cs_layernorm_backward_rows that also does an EARLIER call's
 * cs_layernorm_backward_finalize inside its own launch: a few workgroups ahead
 * of the row work add `pending_partials` (what that earlier rows call left,
 * pending_partial_rows rows of the same C, x_dtype and param_dtype) into
 * pending_dgamma / pending_dbeta and leave.  A training step runs one
 * LayerNorm backward after another (src/compute/layer_norm.cpp:228-233, once
 * per norm, 25 times for GPT-2-small), and the reference already lets the
 * parameter gradients lag the input gradient (its parameter task runs on the
 * assist stream, :302,356): each call carries the previous norm's sums, and
 * only the last norm needs a cs_layernorm_backward_finalize launch of its
 * own.  Results are those of cs_layernorm_backward_finalize, bit for bit.
 * pending_partials must not overlap partials (CS_ERR_INVALID_ARGUMENT) and
 * must have been written by work that precedes this call on the stream;
 * pending_partials == NULL makes this cs_layernorm_backward_rows. */
int cs_layernorm_backward_rows_pending(
    const void *dy, const void *x, const void *mean, const void *rstd,
    const void *gamma, const void *dresidual, void *dx, void *partials,
    size_t partials_bytes, const void *pending_partials,
    int64_t pending_partial_rows, void *pending_dgamma, void *pending_dbeta,
    int pending_accumulate, int64_t rows, int64_t C, int dy_dtype, int x_dtype,
    int dx_dtype, int param_dtype, void *stream);

/* ------------------------------------------------------------------------
 * Embedding
 * forward replaces torch::embedding, src/compute/embedding.cpp:117-121:
 * out[i, :] = weight[indices[i], :], a byte-exact copy.  An index outside
 * [0, num_weights) yields a zero row and never reads out of bounds.
 * ---------------------------------------------------------------------- */
int cs_embedding_forward(const void *weight, const void *indices, void *out,
                         int64_t n_indices, int64_t C, int64_t num_weights,
                         int dtype, int idx_dtype, void *stream);

/* Token + position embedding in one pass: out[b,t,:] = wte[ids[b,t],:] +
 * wpe[t,:], replacing the two gathers, broadcast_to and add of
 * example/gpt2/gpt2_single_device.cpp:541-545.  The sum is formed in fp32
 * and rounded once, which for f16/bf16 equals the reference's add bit for
 * bit. */
int cs_embedding_forward_add(const void *wte, const void *wpe,
                             const void *indices, void *out, int64_t B,
                             int64_t T, int64_t C, int64_t num_weights,
                             int dtype, int idx_dtype, void *stream);

/* backward replaces at::embedding_backward (+ the += of an existing
 * gradient), src/compute/embedding.cpp:147-157: dense dweight[num_weights,C],
 * dweight[k] = sum over {i : indices[i]==k, k != padding_idx} of dout[i],
 * rows never indexed are zero (left untouched when accumulate != 0).
 * Sums are formed in fp32 (fp64 for CS_F64) in ascending order of i, by
 * sorting (index, i) pairs and reducing segments, so results do not depend
 * on scheduling.  padding_idx < 0 means none. */
size_t cs_embedding_backward_workspace_bytes(int64_t n_indices, int64_t C,
                                             int64_t num_weights);
int cs_embedding_backward(const void *dout, const void *indices,
                          void *dweight, void *workspace,
                          size_t workspace_bytes, int64_t n_indices, int64_t C,
                          int64_t num_weights, int64_t padding_idx, int dtype,
                          int idx_dtype, int accumulate, void *stream);

/* cs_embedding_backward with the reference's scale_grad_by_freq option
 * (at::embedding_backward(..., scale_grad_by_freq = true, sparse = false),
 * src/compute/embedding.cpp:147-157): the gradient of a row is the sum over
 * the entries that name it divided by their number, then added to what is
 * there when accumulate != 0.  (The `sparse` option returns a sparse tensor
 * and has no counterpart here.) */
int cs_embedding_backward_scaled(const void *dout, const void *indices,
                                 void *dweight, void *workspace,
                                 size_t workspace_bytes, int64_t n_indices,
                                 int64_t C, int64_t num_weights,
                                 int64_t padding_idx, int dtype, int idx_dtype,
                                 int accumulate, void *stream);

/* Token and position table gradients of out[b,t,:] = wte[ids[b,t],:] +
 * wpe[t,:] from one dout[B,T,C]: dwte as cs_embedding_backward (no padding
 * index), dwpe[t,:] (+)= sum_b dout[b,t,:] in ascending b.  Replaces
 * Utils::sum(dx,0), wpe->backward and wte->backward of
 * example/gpt2/gpt2_single_device.cpp:565-567 with one call.  Workspace as
 * cs_embedding_backward_workspace_bytes(B*T, C, num_weights). */
int cs_embedding_backward_fused(const void *dout, const void *indices,
                                void *dwte, void *dwpe, void *workspace,
                                size_t workspace_bytes, int64_t B, int64_t T,
                                int64_t C, int64_t num_weights, int dtype,
                                int idx_dtype, int accumulate, void *stream);

/* Position-table gradient: dwpe[t,:] (+)= sum_b dout[b,t,:], replacing
 * Utils::sum(dx, 0) followed by wpe->backward with arange positions,
 * example/gpt2/gpt2_single_device.cpp:565-566. */
int cs_embedding_backward_positions(const void *dout, void *dwpe, int64_t B,
                                    int64_t T, int64_t C, int dtype,
                                    int accumulate, void *stream);

/* ------------------------------------------------------------------------
 * Fused classifier: row softmax + cross-entropy loss + dlogits
 * replaces at::log_softmax + at::nll_loss_forward
 * (src/compute/cross_entropy.cpp:57-63) and at::nll_loss_backward +
 * at::_log_softmax_backward_data (:103-109) with one pass over the logits.
 *
 * logits: [N, row_stride] row-major, columns [0, V) are classes, columns
 * [V, row_stride) are padding that is ignored on input.
 * targets: [N] int64; rows whose target equals ignore_index contribute no
 * loss and get zero dlogits.
 * row_loss: [N] fp32, written for every reduction (NULL: not wanted unless
 * reduction is NONE).  loss: one fp32 (MEAN or SUM; ignored for NONE).
 * total_weight: one fp32 = number of rows not ignored (may be NULL).
 * dlogits: [N, row_stride] of dlogits_dtype (logits' dtype or CS_F32), may
 * alias logits when the dtypes match (in-place), may be NULL (loss only).
 * dlogits = (softmax(logits) - onehot(target)) * s, s = dloss / total_weight
 * for MEAN and dloss otherwise; padding columns are written as zero.  The
 * reference has no upstream gradient (it passes ones_like(loss)):
 * dloss = 1 reproduces it.
 * Any row_stride >= V is accepted.  Rows that start on 16-byte boundaries
 * and have at most 57344 columns (16 bit) or 65536 (fp32) are read once;
 * other rows are read twice, the second time from cache.
 * ---------------------------------------------------------------------- */
size_t cs_fused_classifier_workspace_bytes(int64_t N);
int cs_fused_classifier(const void *logits, void *dlogits,
                        const int64_t *targets, float *row_loss, float *loss,
                        float *total_weight, void *workspace,
                        size_t workspace_bytes, int64_t N, int64_t V,
                        int64_t row_stride, int64_t ignore_index,
                        int reduction, float dloss, int dtype,
                        int dlogits_dtype, void *stream);

/* cs_fused_classifier with at::nll_loss's per-class `weight`
 * (state->forward.weight, src/compute/cross_entropy.cpp:52-63 and :97-105):
 * class_weight is [V] fp32; a row's loss and gradient are scaled by the weight
 * of its target, MEAN divides by the sum of those weights over the rows that
 * are not ignored, and total_weight returns that sum.  class_weight == NULL is
 * cs_fused_classifier.  No caller in the reference sets a weight, so this
 * form takes the two-sweep row kernel for every shape. */
int cs_fused_classifier_weighted(const void *logits, void *dlogits,
                                 const int64_t *targets,
                                 const float *class_weight, float *row_loss,
                                 float *loss, float *total_weight,
                                 void *workspace, size_t workspace_bytes,
                                 int64_t N, int64_t V, int64_t row_stride,
                                 int64_t ignore_index, int reduction,
                                 float dloss, int dtype, int dlogits_dtype,
                                 void *stream);

/* The same call split into its three launches, for callers that want to
 * time or capture them apart, or that already know the row count:
 * phases is a bit set of CS_CE_PHASE_COUNT (write the number of rows that are
 * not ignored into the workspace), CS_CE_PHASE_ROWS (the pass over the logits;
 * needs the count in the workspace) and CS_CE_PHASE_REDUCE (row losses ->
 * loss, total_weight).  All three in one call is cs_fused_classifier. */
enum cs_ce_phase {
  CS_CE_PHASE_COUNT = 1,
  CS_CE_PHASE_ROWS = 2,
  CS_CE_PHASE_REDUCE = 4,
};
int cs_fused_classifier_phases(const void *logits, void *dlogits,
                               const int64_t *targets, float *row_loss,
                               float *loss, float *total_weight,
                               void *workspace, size_t workspace_bytes,
                               int64_t N, int64_t V, int64_t row_stride,
                               int64_t ignore_index, int reduction,
                               float dloss, int dtype, int dlogits_dtype,
                               int phases, void *stream);

/* cs_fused_classifier for callers that cannot allocate device memory (code
 * under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc): the same launches and the same results, with the workspace
 * taken from an array of CS_FUSED_CLASSIFIER_STATIC_SCRATCH_BYTES that the
 * library itself holds in device memory on every GPU it runs on, until the
 * process ends.  It has no counterpart in the reference.  It allocates
 * nothing and frees nothing, on the device or through any library.
 * Limit: N <= cs_fused_classifier_static_max_rows() (262,080 rows for the
 * 1 MiB array); more rows return CS_ERR_STATIC_LIMIT and launch nothing.
 * All calls on one GPU share that GPU's array, which keeps what the last
 * call left there (no call needs it cleared): calls that overlap on one GPU,
 * on different streams or from different threads, race on it and must be
 * ordered by the caller.  The first call on a device looks up the array's
 * address on that device (hipGetSymbolAddress), later calls reuse it. */
#define CS_FUSED_CLASSIFIER_STATIC_SCRATCH_BYTES (1 << 20)
int64_t cs_fused_classifier_static_max_rows(void);
int cs_fused_classifier_static(const void *logits, void *dlogits,
                               const int64_t *targets, float *row_loss,
                               float *loss, float *total_weight, int64_t N,
                               int64_t V, int64_t row_stride,
                               int64_t ignore_index, int reduction,
                               float dloss, int dtype, int dlogits_dtype,
                               void *stream);

#ifdef __cplusplus
}
#endif

#endif /* CS_HIP_KERNELS_H_ */
