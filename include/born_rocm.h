/*
 * born_rocm.h — C ABI of the MI355X (gfx950) token-sampling engine for Born.
 *
 * This is the boundary a build-tagged Go package `backend/rocm` binds through cgo
 * (plain pointers and sizes only; no Go pointer is retained after a call returns).
 * Born v0.1.1 has no device backend and no sampler, so each entry point cites the
 * reference interface it stands beside or extends (paths relative to the reference
 * root).  Semantics of every sampling stage: docs/SAMPLING_SPEC.md.
 *
 * Conventions
 *   - every function returns 0 on success or a BORN_ROCM_ERR_* code; the message
 *     for the calling thread's last failure is born_rocm_last_error();
 *   - all device pointers are plain `void*` / typed pointers into HIP device
 *     memory; `stream` is a hipStream_t passed as void* (NULL = the null stream);
 *   - logits are fp32, row-major `[batch, vocab]` with a row stride in elements,
 *     the layout of tensor.RawTensor (internal/tensor/raw.go:78-105, strides
 *     internal/tensor/shape.go:52-63); token ids are int32, as the reference's
 *     label tensors are (internal/nn/cross_entropy.go:73, raw.go:167-174);
 *   - inputs are never modified (the reference's "inputs are immutable unless
 *     uniquely owned" rule, internal/backend/cpu/backend.go:45-51);
 *   - launches are asynchronous on `stream`; outputs are valid after the stream
 *     is synchronised (born_rocm_stream_sync or a born_rocm_d2h on that stream).
 */
#ifndef BORN_ROCM_H
#define BORN_ROCM_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BORN_ROCM_OK               0
#define BORN_ROCM_ERR_ARGUMENT     1   /* programmer error: the Go layer panics "sampler: ..." (internal/backend/cpu/backend.go:36 idiom) */
#define BORN_ROCM_ERR_HIP          2   /* runtime failure: the Go layer returns an error (internal/tensor/raw.go:89-92 idiom) */
#define BORN_ROCM_ERR_UNSUPPORTED  3   /* shape outside what the kernels handle (e.g. vocab too large for LDS) */
#define BORN_ROCM_ERR_DATA         4   /* device-side data error: out-of-range history id / draft token */

/* Sampling configuration.  Mirrors the reference's plain-struct config idiom
 * (AdamConfig, internal/optim/adam.go:59-63): a zero field means "default", filled
 * in by born_rocm_sampler_create the way NewAdam fills its defaults
 * (internal/optim/adam.go:78-91). */
typedef struct born_sampler_config {
    float   temperature;          /* 0 => 1.0 ; must be > 0 otherwise */
    int32_t top_k;                /* <= 0 => disabled */
    float   top_p;                /* 0 => 1.0 (disabled) ; must be > 0 otherwise; >= 1 disables */
    float   repetition_penalty;   /* 0 => 1.0 (identity) ; must be > 0 otherwise */
    int64_t seed;                 /* seed of the built-in uniform stream (used only when `uniforms` is NULL) */
    float   min_p;                /* 0 => disabled ; else in (0, 1): a token stays only if its probability is at
                                     least min_p times the most likely token's (applied before top-k and top-p) */
    float   frequency_penalty;    /* 0 => disabled ; subtracted from a token's logit once per occurrence in the history */
    float   presence_penalty;     /* 0 => disabled ; subtracted once from the logit of every token the history holds
                                     (both after the repetition penalty, before the temperature; finite, either sign).
                                     A handle configured with either keeps a table of max_batch * max_vocab counters. */
} born_sampler_config;

typedef struct born_sampler born_sampler;   /* opaque: config + stream-ordered workspace + draw counter */

/* Thread-local message of the last failure on the calling thread ("" if none). */
const char *born_rocm_last_error(void);

/* Device discovery / selection — extends tensor.Device (internal/tensor/raw.go:10-20), which has no ROCm value. */
int born_rocm_device_count(int32_t *count);
int born_rocm_device_name(int32_t device, char *buf, int64_t buf_len);

/* Device buffers — Born's RawTensor is host-only (internal/tensor/raw.go:42-46,139-141); these give the Go
 * layer its DeviceBuffer handle.  Copies are enqueued on `stream` and are synchronous with respect to the host
 * when the host pointer is pageable. */
int born_rocm_alloc(int64_t bytes, void **dev_ptr);
int born_rocm_free(void *dev_ptr);
int born_rocm_h2d(void *dst_dev, const void *src_host, int64_t bytes, void *stream);
int born_rocm_d2h(void *dst_host, const void *src_dev, int64_t bytes, void *stream);
int born_rocm_stream_sync(void *stream);

/* Sampler handle — the capability object a `SamplerBackend` type assertion would return
 * (idiom: ReLUBackend, internal/nn/activation.go:8-20).  `max_batch`/`max_vocab` size the workspace;
 * calls with larger shapes fail with BORN_ROCM_ERR_ARGUMENT.  One handle = one stream at a time. */
int born_rocm_sampler_create(const born_sampler_config *cfg, int64_t max_batch, int64_t max_vocab,
                             born_sampler **out);
int born_rocm_sampler_destroy(born_sampler *s);
int born_rocm_sampler_get_config(const born_sampler *s, born_sampler_config *out);   /* after defaults were filled */
int born_rocm_sampler_set_config(born_sampler *s, const born_sampler_config *cfg);
/* Device status since the last call of this function: 0, or BORN_ROCM_ERR_DATA if a kernel met an
 * out-of-range history id or draft token.  Synchronises `stream`. */
int born_rocm_sampler_status(born_sampler *s, void *stream);
/* Work counters accumulated by the kernels (diagnostics): rows the single-pass top-k kernel settled from its
 * candidate lists, rows it had to finish by its exact (slower) selection, rows sampled by the general kernel.
 * Synchronises. */
int born_rocm_sampler_counters(born_sampler *s, void *stream, int64_t *topk_rows, int64_t *fallback_rows,
                               int64_t *general_rows);

/* Diagnostics.  0 = choose the kernel from the configuration (default: the single-pass kernel for
 * 1 <= top_k <= 512 and a vocabulary of at most 393216, with penalties that raise a logit (a repetition penalty below
 * 1, a negative frequency or presence penalty) only over a history of at most 1024 tokens; the general kernel otherwise).
 * 1 = always the general kernel.  2 = as 0, but the kernel for top_k 0 and the single-pass kernel for top_k <= 128 run
 * 512 threads per row (two rows to a CU at a time) whatever the batch; by default they do so only for batches of more
 * rows than the device has CUs.
 * All implement the same fixed-point pipeline and must return identical results; tests compare them. */
int born_rocm_sampler_set_path(born_sampler *s, int32_t path);

/* The draw counter of the built-in uniform stream: a call that is given no `uniforms` draws row b's uniform from
 * (cfg.seed, step, b) and then advances `step` by one (born_rocm_sample, born_rocm_sample_rows,
 * born_rocm_linear_sample; calls that are given uniforms leave it alone).  Reading and setting it lets a caller
 * repeat a call with the same draws: the fallback after born_rocm_linear_sample reports an unsettled row sets the
 * counter back to what it was before that call, so that born_rocm_linear + born_rocm_sample draw the very uniforms
 * the fused call used and the generation consumes one step either way.  Host state only: nothing is enqueued.  No
 * counterpart in the reference snapshot (its only generator is the process-global unseeded one,
 * internal/tensor/creation.go:92-93). */
int born_rocm_sampler_get_step(const born_sampler *s, int64_t *step_out);
int born_rocm_sampler_set_step(born_sampler *s, int64_t step);

/* Greedy decode: index of the maximum of each row, lowest index on ties — `argmax`,
 * internal/nn/cross_entropy.go:241-251 (the per-row step of nn.Accuracy, :261-284). */
int born_rocm_argmax(born_sampler *s, const float *logits, int64_t batch, int64_t vocab, int64_t row_stride,
                     int32_t *tokens_out, void *stream);

/* Max-shifted softmax / log-softmax over the last dimension —
 * softmaxFloat32, internal/autodiff/ops/softmax.go:214-238 (ops.Softmax, :268-294);
 * logSoftmax, internal/nn/cross_entropy.go:126-153.  `out` is `[batch, vocab]` contiguous. */
int born_rocm_softmax(born_sampler *s, const float *logits, int64_t batch, int64_t vocab, int64_t row_stride,
                      float *out, void *stream);
int born_rocm_log_softmax(born_sampler *s, const float *logits, int64_t batch, int64_t vocab, int64_t row_stride,
                          float *out, void *stream);

/* One sampling step for `batch` rows: penalties -> temperature -> (min-p) -> top-k -> softmax -> top-p -> draw.
 * No counterpart in the reference snapshot; it consumes the `[batch, vocab]` fp32 output of the last
 * Linear (internal/nn/linear.go:78-107) where the reference's only consumers are CrossEntropy and
 * nn.Accuracy (internal/nn/cross_entropy.go:261-284).
 *   history   int32 [batch, hist_stride] or NULL; hist_len int32 [batch] or NULL (=> hist_stride each)
 *   uniforms  fp32 [batch] in [0,1) or NULL (=> built-in stream from cfg.seed and the handle's draw counter)
 *   tokens_out int32 [batch]; probs_out fp32 [batch] or NULL (probability of the sampled token in the
 *   renormalised nucleus)
 *   The logits buffer must span batch * row_stride elements (the last row included): rows that start 16-byte aligned
 *   with a row_stride that is a multiple of 4 are read in whole 128-bit blocks, so up to 3 floats past `vocab`
 *   (inside the row's pitch) are loaded and ignored when vocab is not a multiple of 4.
 *   nucleus outputs (all three NULL, or all three set with nucleus_cap > 0): the first
 *   min(n, nucleus_cap) survivors of each row in rank order; produced when 1 <= top_k <= 4096
 *   (nucleus_len_out[b] = -1 otherwise). */
int born_rocm_sample(born_sampler *s, const float *logits, int64_t batch, int64_t vocab, int64_t row_stride,
                     const int32_t *history, const int32_t *hist_len, int64_t hist_stride,
                     const float *uniforms, int32_t *tokens_out, float *probs_out,
                     int32_t *nucleus_len_out, int32_t *nucleus_ids_out, float *nucleus_probs_out,
                     int64_t nucleus_cap, void *stream);

/* The same step with a configuration per row (continuous batching: requests with different settings share a
 * batch).  Every member is a device array of `batch` values or NULL (=> the handle's value for every row); the
 * values mean what the fields of born_sampler_config mean after defaults (top_k <= 0 or >= vocab: no top-k cut;
 * top_p = 1: no top-p cut; repetition_penalty = 1, min_p = 0, frequency_penalty = 0, presence_penalty = 0: off).
 * A row whose values are invalid (temperature or repetition penalty not positive and finite, top_p outside (0, 1],
 * min_p outside [0, 1), a frequency or presence penalty that is not finite) gets token 0 and BORN_ROCM_ERR_DATA
 * from born_rocm_sampler_status.  Every row's result equals what born_rocm_sample returns for that row under a
 * handle configured with the row's values.  Per-row frequency or presence penalties use the handle's table of
 * counters (unless row_kinds promises small top-k rows only and hist_stride <= 4096: that kernel counts by itself);
 * a handle not configured with either allocates it on the first such call (which synchronises the stream, so make
 * that call outside a graph capture).  No counterpart in the reference snapshot. */
typedef struct born_sampler_row_configs {
    const float   *temperature;
    const int32_t *top_k;
    const float   *top_p;
    const float   *repetition_penalty;
    const float   *min_p;
    const float   *frequency_penalty;
    const float   *presence_penalty;
    /* Optional promise about the rows of this call, so that kernels no row needs are not launched at all (an idle
     * launch costs about 7 us): 0 = no promise (every kernel is launched), else the OR of the kinds of row that
     * may occur.  A row of a kind that was not promised gets token 0 and BORN_ROCM_ERR_DATA, like an invalid one. */
    uint32_t       row_kinds;
} born_sampler_row_configs;
#define BORN_ROCM_ROWS_SMALL_TOP_K  1u   /* 1 <= top_k <= 512, vocab <= 393216; a penalty that raises a logit only with hist_stride <= 1024 */
#define BORN_ROCM_ROWS_NO_TOP_K     2u   /* top_k disabled (<= 0 or >= vocab) */
#define BORN_ROCM_ROWS_OTHER        4u   /* everything else (top_k > 512, a penalty that raises logits with a top-k cut and a longer history, ...) */

int born_rocm_sample_rows(born_sampler *s, const float *logits, int64_t batch, int64_t vocab, int64_t row_stride,
                          const int32_t *history, const int32_t *hist_len, int64_t hist_stride, const float *uniforms,
                          const born_sampler_row_configs *rows, int32_t *tokens_out, float *probs_out, void *stream);

/* born_rocm_sample for callers that cannot allocate device memory at any time: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference and takes no handle (creating
 * one allocates): the kernels' workspace (the per-row work counters and a status word) is a fixed array inside the
 * library, one copy per device, sized for at most 4096 rows; a larger batch is BORN_ROCM_ERR_UNSUPPORTED.  The call
 * allocates and frees nothing and returns after enqueueing, like born_rocm_sample, and every row's token and
 * probability equal what born_rocm_sample returns under a handle configured with *cfg.
 *   cfg        as for born_rocm_sampler_create (NULL: all defaults)
 *   uniforms   required (the built-in uniform stream counts its draws in a handle)
 *   status_out int32 device word or NULL: the bits born_rocm_sampler_status reports (1 = a history id outside the
 *              vocabulary) are OR-ed into it; the caller zeroes and reads it
 * Not served (BORN_ROCM_ERR_UNSUPPORTED): frequency / presence penalties where the kernel cannot count the
 * occurrences itself (histories beyond 4096 tokens, top_k outside 1..512); nucleus listings and per-row
 * configurations have no static form.  All calls on one device share that device's array: calls that overlap on one
 * device (two streams, two threads) race on it.  The first call on a device looks up the array's address; make that
 * call outside a graph capture. */
int born_rocm_sample_static(const born_sampler_config *cfg, const float *logits, int64_t batch, int64_t vocab,
                            int64_t row_stride, const int32_t *history, const int32_t *hist_len, int64_t hist_stride,
                            const float *uniforms, int32_t *tokens_out, float *probs_out, int32_t *status_out,
                            void *stream);

/* Log-probability of one given token per row: logprobs_out[b] = log_softmax(z_b)[tokens[b]], z_b being row b after
 * the handle's penalties and temperature (steps 1-3 of the sampling pipeline; no min-p / top-k / top-p truncation).
 * With temperature 1 and no history this is minus the per-row term `-logProbs[target]` of CrossEntropyLoss.Forward,
 * internal/nn/cross_entropy.go:37-90 (logSoftmax, :126-153): the mean of the negated outputs is that loss.  Also
 * the log-probability reported next to a sampled token (pass tokens_out of born_rocm_sample and the same history).
 *   tokens int32 [batch] on the device; a token outside [0, vocab) gives NaN and BORN_ROCM_ERR_DATA from
 *   born_rocm_sampler_status (the reference panics "target index out of bounds"). */
int born_rocm_token_logprobs(born_sampler *s, const float *logits, int64_t batch, int64_t vocab, int64_t row_stride,
                             const int32_t *history, const int32_t *hist_len, int64_t hist_stride, const int32_t *tokens,
                             float *logprobs_out, void *stream);

/* The two small steps that keep a decode loop on the device (no counterpart in the reference snapshot, which has
 * neither a generation loop nor an embedding layer):
 *   born_rocm_history_append  history[b][hist_len[b]] = tokens[b]; hist_len[b] += 1 — the sampled tokens join the
 *       histories the next born_rocm_sample call penalises.  A full row (hist_len[b] == hist_stride) is left as it
 *       is, a token outside [0, vocab) is not appended; both give BORN_ROCM_ERR_DATA from born_rocm_sampler_status.
 *   born_rocm_gather_rows     out[i][:] = table[ids[i]][:] (fp32 rows, strides in elements) — the embedding lookup
 *       that turns the sampled tokens into the next step's input rows.  An id outside [0, rows) yields a row of
 *       zeros and BORN_ROCM_ERR_DATA from born_rocm_sampler_status.
 * The handle only lends its status word. */
int born_rocm_history_append(born_sampler *s, int32_t *history, int32_t *hist_len, int64_t hist_stride, const int32_t *tokens,
                             int64_t batch, int64_t vocab, void *stream);
int born_rocm_gather_rows(born_sampler *s, const float *table, int64_t rows, int64_t cols, int64_t row_stride, const int32_t *ids,
                          int64_t n, float *out, int64_t out_stride, void *stream);

/* Speculative-decoding accept/reject with residual max(0, p - q) resampling.
 * No counterpart in the reference snapshot.
 *   target, draft  fp32 [batch, gamma, vocab] contiguous;  draft_tokens int32 [batch, gamma]
 *   u_accept fp32 [batch, gamma];  u_residual fp32 [batch]
 *   n_accepted_out int32 [batch];  next_token_out int32 [batch] (-1 when every draft token was accepted)
 * The first call with a larger batch * gamma than any before it grows the handle's per-position statistics: it
 * synchronises the stream and allocates, and is refused (BORN_ROCM_ERR_UNSUPPORTED) inside a stream capture. */
int born_rocm_spec_verify(born_sampler *s, const float *target, const float *draft, int64_t batch,
                          int64_t gamma, int64_t vocab, const int32_t *draft_tokens, const float *u_accept,
                          const float *u_residual, int32_t *n_accepted_out, int32_t *next_token_out,
                          void *stream);

/* The same step with the bonus draw: `bonus` holds, per sequence, the target's logits one position past the
 * draft (fp32 [vocab], `bonus_stride` elements apart).  A sequence whose draft tokens are all accepted then
 * gets next_token = a draw from softmax(bonus / T) by inverse CDF in ascending id order with u_residual[b]
 * (never -1).  Sequence strides (elements between consecutive sequences) let target and bonus alias one
 * [batch, gamma + 1, vocab] tensor: target_seq_stride = bonus_stride = (gamma + 1) * vocab,
 * bonus = target + gamma * vocab.  No counterpart in the reference snapshot. */
int born_rocm_spec_verify_bonus(born_sampler *s, const float *target, int64_t target_seq_stride, const float *draft,
                                int64_t draft_seq_stride, const float *bonus, int64_t bonus_stride, int64_t batch,
                                int64_t gamma, int64_t vocab, const int32_t *draft_tokens, const float *u_accept,
                                const float *u_residual, int32_t *n_accepted_out, int32_t *next_token_out,
                                void *stream);

/* The logits producer, fp32 on the matrix cores (fp32 operands, fp32 accumulation; the order of the k-sum
 * differs from the reference's sequential loop, so results agree with it to rounding, not bit for bit).
 *
 * born_rocm_linear: out[batch, out_features] = x[batch, in_features] @ weight^T + bias, weight stored
 * [out_features, in_features] row-major as nn.Linear holds it, bias [out_features] or NULL: Linear.Forward,
 * internal/nn/linear.go:78-107 (which transposes the weight, calls MatMul and adds the bias).  For the LM
 * head `out` is the `[batch, vocab]` logits that born_rocm_sample reads, so they never leave the device.
 *
 * born_rocm_matmul: c[m,n] = a[m,k] @ b[k,n], all row-major: tensor.Backend.MatMul,
 * internal/tensor/backend.go:20, CPU form internal/backend/cpu/matmul.go:13-71 (2-D fp32 only).
 *
 * Pitches (x_stride, w_stride, out_stride, lda, ldb, ldc) are in elements between consecutive rows.  Inputs
 * are not modified; `out` / `c` must not overlap them. */
int born_rocm_linear(const float *x, int64_t batch, int64_t in_features, int64_t x_stride, const float *weight,
                     int64_t out_features, int64_t w_stride, const float *bias, float *out, int64_t out_stride,
                     void *stream);
/* (born_rocm_matmul, born_rocm_linear and the fused heads below: a product of few output tiles and a long k is computed in slices of k that are added in a fixed order;
 * the first such call on a stream allocates the library's workspace for that stream, 8 or 64 MiB kept until the process
 * ends - outside a stream capture; a call under capture that finds no workspace computes the product unsplit.) */
int born_rocm_matmul(const float *a, const float *b, float *c, int64_t m, int64_t k, int64_t n, int64_t lda,
                     int64_t ldb, int64_t ldc, void *stream);

/* Greedy decode fused into the LM head: tokens_out[b] = argmax_j (x[b] @ weight[j]^T + bias[j]) without the
 * [batch, out_features] logits ever being written: every tile of the product keeps its rows' largest value and
 * the tiles are merged by a 64-bit atomic max.  Same arithmetic as born_rocm_linear followed by
 * born_rocm_argmax and the same token ids, including the reference's tie rule (`argmax`,
 * internal/nn/cross_entropy.go:241-251; Linear.Forward, internal/nn/linear.go:78-107).  The handle provides the
 * per-row workspace (batch <= its max_batch); one call at a time per handle. */
int born_rocm_linear_argmax(born_sampler *s, const float *x, int64_t batch, int64_t in_features, int64_t x_stride,
                            const float *weight, int64_t out_features, int64_t w_stride, const float *bias,
                            int32_t *tokens_out, void *stream);

/* The LM head and the sampling step in one call: tokens_out[b] is what born_rocm_sample draws from the logits
 * born_rocm_linear would produce, bit for bit, and those [batch, out_features] logits are never written to memory —
 * Linear.Forward (internal/nn/linear.go:78-107) with the reference's only logits consumers replaced by a sampler that
 * lives in the GEMM's epilogue.  The handle's configuration must be one the single-pass sampler serves: 1 <= top_k <=
 * 128, out_features <= 393216, repetition penalty >= 1, no frequency / presence penalty (else
 * BORN_ROCM_ERR_UNSUPPORTED).  How: the product over a strided sample of at most 1024 weight rows gives every row a
 * threshold that about 1500 of its logits reach; the full product's epilogue lists the logits at or above
 * it (value and column); the sampling step runs over the list and proves that nothing outside it can belong to the
 * row's top_k.  A row it cannot settle (a list of more than 4096, fewer than top_k candidates above the bound, a
 * history of more than 1024 tokens with a penalty) gets token -1 and born_rocm_sampler_status returns
 * BORN_ROCM_ERR_DATA: the caller then runs born_rocm_linear + born_rocm_sample for that call.  With uniforms == NULL
 * the fused call has advanced the handle's draw counter whether or not every row settled: a caller that falls back
 * first sets the counter to its value before the fused call (born_rocm_sampler_get_step / _set_step), so that the
 * unfused pair draws the same uniforms and the tokens stay those of a run that never used the fused call.  The first
 * call on a handle allocates about 36 KiB of workspace per row of max_batch (outside a stream capture). */
int born_rocm_linear_sample(born_sampler *s, const float *x, int64_t batch, int64_t in_features, int64_t x_stride,
                            const float *weight, int64_t out_features, int64_t w_stride, const float *bias,
                            const int32_t *history, const int32_t *hist_len, int64_t hist_stride, const float *uniforms,
                            int32_t *tokens_out, float *probs_out, void *stream);

/* The element-wise and shape operations of tensor.Backend (internal/tensor/backend.go:12-33) on fp32 device
 * memory.  Operands are row-major and contiguous; shapes are given as arrays of `ndim` extents (0 <= ndim <= 8,
 * every extent > 0).  `out` is contiguous in the result's shape and must not overlap an operand.
 *
 * born_rocm_add / sub / mul / div: NumPy-style broadcasting — Add/Sub/Mul/Div,
 * internal/backend/cpu/backend.go:32-134; the result shape is that of tensor.BroadcastShapes,
 * internal/tensor/shape.go:83-118, which born_rocm_broadcast_shape evaluates on the host (out_shape receives
 * max(a_ndim, b_ndim) extents).  Incompatible shapes return BORN_ROCM_ERR_ARGUMENT with the reference's
 * message ("add: shapes not compatible for broadcasting: [2 3] vs [4] (dimension 1: 3 vs 4)").  Each result
 * element is one IEEE fp32 operation, so results equal the CPU backend's bit for bit.
 *
 * born_rocm_transpose: out = in with its dimensions permuted, result extent i = shape[axes[i]]; axes == NULL
 * reverses all dimensions — Transpose, internal/backend/cpu/backend.go:164-209 (same validation messages).
 *
 * born_rocm_reshape: same elements in row-major order under a new shape; like the reference (which copies,
 * internal/backend/cpu/backend.go:137-161) it fills `out`, or does nothing when out == in. */
int born_rocm_broadcast_shape(const int64_t *a_shape, int32_t a_ndim, const int64_t *b_shape, int32_t b_ndim,
                              int64_t *out_shape);
int born_rocm_add(const float *a, const int64_t *a_shape, int32_t a_ndim, const float *b, const int64_t *b_shape,
                  int32_t b_ndim, float *out, void *stream);
int born_rocm_sub(const float *a, const int64_t *a_shape, int32_t a_ndim, const float *b, const int64_t *b_shape,
                  int32_t b_ndim, float *out, void *stream);
int born_rocm_mul(const float *a, const int64_t *a_shape, int32_t a_ndim, const float *b, const int64_t *b_shape,
                  int32_t b_ndim, float *out, void *stream);
int born_rocm_div(const float *a, const int64_t *a_shape, int32_t a_ndim, const float *b, const int64_t *b_shape,
                  int32_t b_ndim, float *out, void *stream);
int born_rocm_transpose(const float *in, const int64_t *shape, int32_t ndim, const int32_t *axes, float *out,
                        void *stream);
int born_rocm_reshape(const float *in, const int64_t *shape, int32_t ndim, const int64_t *new_shape, int32_t new_ndim,
                      float *out, void *stream);

/* born_rocm_conv2d: input [N, C, H, W] * kernel [CO, C, KH, KW], zero padding -> out [N, CO, HO, WO] with
 * HO = (H + 2 padding - KH) / stride + 1 (WO alike) — Conv2D, internal/backend/cpu/conv2d.go:35-203.  Each output
 * sums its C * KH * KW products in the reference's order with one fp32 accumulator, so results equal the CPU
 * backend's bit for bit.  born_rocm_maxpool2d: windows of kernel_size x kernel_size, no padding — MaxPool2D,
 * internal/backend/cpu/maxpool2d.go:26-113 (the running maximum starts at -1e38, as there).  input_shape /
 * kernel_shape are 4 extents; out_shape (4 extents) may be NULL.  Same validation messages as the reference. */
int born_rocm_conv2d(const float *input, const int64_t *input_shape, const float *kernel, const int64_t *kernel_shape,
                     int32_t stride, int32_t padding, float *out, int64_t *out_shape, void *stream);
int born_rocm_maxpool2d(const float *input, const int64_t *input_shape, int32_t kernel_size, int32_t stride, float *out,
                        int64_t *out_shape, void *stream);

/* Element-wise exponential, out[i] = float32(exp(float64(x[i]))) — ops.Exp, internal/autodiff/ops/log.go:159-185
 * (a helper without a backward operation; its fp32 branch).  x and out are device arrays of n fp32 values (any shape,
 * flat); they may be the same buffer.  n = 0 is a no-op. */
int born_rocm_exp(const float *x, float *out, int64_t n, void *stream);

/* Building blocks exported for parity tests (device-side evaluation of the specified fp32 exponential and of
 * the built-in uniform stream). */
int born_rocm_expneg(const float *d_in, float *e_out, int64_t n, void *stream);
int born_rocm_uniforms(int64_t seed, int64_t step, float *u_out, int64_t n, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* BORN_ROCM_H */
