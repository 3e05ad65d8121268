/* C ABI of the MI355X (gfx950) transducer-loss kernels.
 *
 * The reference exposes this path as a pybind11 function that takes torch
 * tensors (optimized_transducer/python/csrc/optimized_transducer.cc:12-19) and
 * keeps its CUDA launchers private to one translation unit
 * (optimized_transducer/csrc/cuda.cu).  This header is the same set of steps
 * with plain pointers and sizes, so that any host language can bind it; the
 * torch extension `_optimized_transducer` of this repository is one such
 * binding and adds nothing but argument checks and allocation.
 *
 * Conventions
 *   - every pointer is DEVICE memory on the current HIP device unless stated;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *     work is enqueued, nothing here synchronises;
 *   - packed layout (reference README.md:133-136): utterance b owns rows
 *     [row_splits[b], row_splits[b+1]) of every per-row array; inside it cell
 *     (t, u), 0 <= t < T_b, 0 <= u <= U_b, is row row_splits[b] + t*(U_b+1) + u;
 *   - return value: 0 on success, a positive hipError_t from the launch, or a
 *     negative OT_E_* code for arguments the kernels cannot run with.
 */
#ifndef OT_TRANSDUCER_H_
#define OT_TRANSDUCER_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define OT_E_BAD_ARG (-1)       /* null pointer / non-positive size            */
#define OT_E_TOO_LONG (-2)      /* a length exceeds what the kernels address   */
#define OT_E_MISALIGNED (-3)    /* logits / grad not 4-byte aligned            */
#define OT_E_TOO_LARGE (-4)     /* batch exceeds OT_STATIC_WORKSPACE_BYTES     */

/* Lattice columns (u = 0..U) one workgroup sweeps at a time, one thread per
 * column; an utterance with more columns is swept in tiles of this width, one
 * after the other, like the reference's CPU path loops over any U
 * (cpu.cc:162-244; its CUDA path stops at 1024 columns, cuda.cu:10, cuda.cu:202). */
#define OT_LATTICE_TILE 1024
/* Largest max_u1 = max_b(U_b)+1 accepted.  What really bounds an utterance is
 * that its cells are addressed with 32-bit byte offsets:
 * (T_b + 1300) * (U_b + 1) < 2^28. */
#define OT_MAX_U1 (1 << 18)

/* Batch facts gathered on the device by ot_row_splits; the host-side argument
 * checks of the reference (transducer-loss.cc:49-66) need exactly these and
 * obtain them with three blocking .item() calls.  32 bytes. */
typedef struct ot_batch_status {
  int64_t sum_tu;          /* sum_b T_b * (U_b + 1), exact in 64 bits          */
  int32_t targets_max;     /* max over the whole (N, targets_cols) array       */
  int32_t targets_min;     /* min over the same array if that is >= 0; else
                              min over the entries that are read, u < U_b
                              (INT32_MAX if none): negative exactly when an
                              entry that is read is negative                   */
  int32_t target_len_max;  /* max_b U_b                                        */
  int32_t target_len_min;  /* min_b U_b                                        */
  int32_t logit_len_max;   /* max_b T_b                                        */
  int32_t logit_len_min;   /* min_b T_b                                        */
} ot_batch_status;

/* Row offsets + batch facts in one launch.
 * Replaces the ATen sequence sizes = T*(U+1); cumsum(int32); cat(zero) at
 * cuda.cu:411-414 and the reductions at transducer-loss.cc:49,53,62.
 * row_splits: (N+1,) int32, row_splits[0] = 0, int32 wrap-around like the
 * reference; status: one ot_batch_status.  targets may be NULL when
 * targets_cols == 0.  row_splits_mirror (may be NULL) receives a second copy
 * of row_splits; it and `status` may be device-visible pinned host memory, so
 * that the host can read both after waiting for an event on `stream`. */
int ot_row_splits(const int32_t *logit_lengths, const int32_t *target_lengths,
                  const int32_t *targets, int32_t N, int32_t targets_cols,
                  int32_t *row_splits, int32_t *row_splits_mirror,
                  ot_batch_status *status, void *stream);

/* Row -> utterance map, (rows,) int32.  Replaces RowSplitsToRowIds /
 * mgpu::load_balance_search (cuda.cu:40-59).  The kernels below do not need
 * it (they decode rows from row_splits); it exists for callers and tests. */
int ot_row_ids(const int32_t *row_splits, int32_t N, int64_t rows,
               int32_t *row_ids, void *stream);

/* Per-row denominators and blank/symbol log-probabilities.
 * from_log_softmax == 0: den[r] = logsumexp(logits[r, :]) (the ATen call at
 *   cuda.cu:427), lp[r] = {logits[r,blank]-den[r], logits[r,target_u]-den[r]}
 *   (ComputeLogProbs, cuda.cu:71-97 / kernels.cu:30-60); one fused kernel that
 *   reads each row once.
 * from_log_softmax != 0: den is not touched (may be NULL) and lp holds the two
 *   gathered values as they are (ComputeLogProbsForLogSoftmax, cuda.cu:111-133).
 * lp is (rows, 2) float; lp[r][1] at u == U_b, which the reference leaves
 * uninitialised, is written as -inf.  Rows beyond row_splits[N] (only possible
 * when the caller's sizes are inconsistent) get den only. */
int ot_log_probs(const float *logits, const int32_t *targets,
                 const int32_t *target_lengths, const int32_t *row_splits,
                 int32_t N, int32_t targets_cols, int64_t rows, int32_t V,
                 int32_t blank, int32_t from_log_softmax, float *den, float *lp,
                 void *stream);

/* ot_log_probs restricted to rows [row_begin, row_end) of the same arrays
 * (any row boundary; utterances need not be complete). */
int ot_log_probs_range(const float *logits, const int32_t *targets,
                       const int32_t *target_lengths, const int32_t *row_splits,
                       int32_t N, int32_t targets_cols, int64_t rows, int32_t V,
                       int32_t blank, int32_t from_log_softmax, int64_t row_begin,
                       int64_t row_end, float *den, float *lp, void *stream);

/* Forward and backward lattice variables, both directions in one launch.
 * Replaces ComputeAlpha / ComputeBeta and their one-symbol-per-frame twins
 * (cuda.cu:162-306, kernels.cu:200-313, kernels.cu:415-519).
 * alpha, beta: (rows,) float.  scores_alpha[b] = alpha(T-1,U)+lp(T-1,U).blank,
 * scores_beta[b] = beta(0,0); both are log-likelihoods.  Cells outside the
 * band of the one-symbol-per-frame lattice (uninitialised in the reference)
 * are -inf.  max_u1 = max_b(U_b)+1 sizes the workgroup; must be <= OT_MAX_U1,
 * and every utterance must satisfy (T_b + 1300) * (U_b + 1) < 2^28. */
int ot_alpha_beta(const float *lp, const int32_t *logit_lengths,
                  const int32_t *target_lengths, const int32_t *row_splits,
                  int32_t N, int32_t max_u1, int32_t one_sym_per_frame,
                  float *alpha, float *beta, float *scores_alpha,
                  float *scores_beta, void *stream);

/* ot_alpha_beta for a caller that has not validated the batch yet (the host
 * is still waiting for ot_row_splits' status): every workgroup first checks on
 * the device that row_splits[N] == rows, T_b >= 1, U_b >= 0 and that the
 * utterance's cells fit 32-bit offsets, and writes nothing otherwise, so the
 * launch is memory-safe for any lengths; max_u1 may be an upper bound
 * (targets_cols + 1).  Results are meaningful only if the caller's own checks
 * pass afterwards. */
int ot_alpha_beta_guarded(const float *lp, const int32_t *logit_lengths,
                          const int32_t *target_lengths,
                          const int32_t *row_splits, int32_t N, int32_t max_u1,
                          int32_t one_sym_per_frame, int64_t rows, float *alpha,
                          float *beta, float *scores_alpha, float *scores_beta,
                          void *stream);

/* ot_alpha_beta restricted to utterances [utt_begin, utt_end); all arrays keep
 * their full-batch indexing. */
int ot_alpha_beta_range(const float *lp, const int32_t *logit_lengths,
                        const int32_t *target_lengths, const int32_t *row_splits,
                        int32_t N, int32_t max_u1, int32_t one_sym_per_frame,
                        int32_t utt_begin, int32_t utt_end, float *alpha,
                        float *beta, float *scores_alpha, float *scores_beta,
                        void *stream);

/* Gradient of the negative log-likelihood w.r.t. the rows of `logits`, times
 * grad_scale.
 * from_log_softmax == 0: ComputeGradient / ComputeGradientOneSymPerFrame
 *   (cuda.cu:308-346, kernels.cu:522-651); `grad` may be the same pointer as
 *   `logits` (the reference's in-place mode, cuda.cu:449) - every element is
 *   read before it is written, by the same thread.  lp is not used (may be NULL).
 * from_log_softmax != 0: ComputeGradientForLogSoftmax(+OneSymPerFrame)
 *   (cuda.cu:364-400, kernels.cu:653-779); `grad` must not alias `logits`;
 *   only lp is read, logits and den may be NULL.
 * An utterance whose beta(0,0) is not finite gets an all-zero gradient
 * (kernels.cu:558-563).  grad_scale = 1 reproduces the reference; 1/N folds
 * the `grad /= N` of reduction="mean" (transducer_loss.py:150).
 * Two launches: a per-row pass that turns (alpha, beta, den, targets) into six
 * coefficients per row in `row_scratch`, then one flat pass over (rows, V). */
int ot_gradient(const float *logits, const float *lp, const float *den,
                const float *alpha, const float *beta, const int32_t *targets,
                const int32_t *logit_lengths, const int32_t *target_lengths,
                const int32_t *row_splits, int32_t N, int32_t targets_cols,
                int64_t rows, int32_t V, int32_t blank,
                int32_t from_log_softmax, int32_t one_sym_per_frame,
                float grad_scale, void *row_scratch, float *grad, void *stream);

/* The two launches of ot_gradient on their own, for callers that want to time
 * or schedule them separately: per-row coefficients into `row_scratch`
 * (same arguments and meaning as in ot_gradient), then the flat pass that
 * reads `logits` and writes `grad`. */
int ot_row_coefficients(const float *lp, const float *den, const float *alpha,
                        const float *beta, const int32_t *targets,
                        const int32_t *logit_lengths,
                        const int32_t *target_lengths, const int32_t *row_splits,
                        int32_t N, int32_t targets_cols, int64_t rows,
                        int32_t blank, int32_t from_log_softmax,
                        int32_t one_sym_per_frame, float grad_scale,
                        void *row_scratch, void *stream);
int ot_gradient_apply(const float *logits, const void *row_scratch, int64_t rows,
                      int32_t V, int32_t from_log_softmax, float grad_scale,
                      float *grad, void *stream);

/* The same two launches restricted to rows [row_begin, row_end) (whole
 * utterances); `rows` stays the extent of the arrays.  Together with
 * ot_log_probs_range and ot_alpha_beta_range this lets a caller run the
 * latency-bound lattice kernel of one part of the batch on a second stream
 * while the streaming kernels of another part use the memory system. */
int ot_row_coefficients_range(const float *lp, const float *den,
                              const float *alpha, const float *beta,
                              const int32_t *targets,
                              const int32_t *logit_lengths,
                              const int32_t *target_lengths,
                              const int32_t *row_splits, int32_t N,
                              int32_t targets_cols, int64_t rows, int32_t blank,
                              int32_t from_log_softmax,
                              int32_t one_sym_per_frame, float grad_scale,
                              int64_t row_begin, int64_t row_end,
                              void *row_scratch, void *stream);
int ot_gradient_apply_range(const float *logits, const void *row_scratch,
                            int64_t rows, int32_t V, int32_t from_log_softmax,
                            float grad_scale, int64_t row_begin, int64_t row_end,
                            float *grad, void *stream);

/* ot_gradient_apply with one more factor, read from DEVICE memory when the
 * kernel runs: grad = d(-log-likelihood)/d(logits) * grad_scale * *device_factor.
 * For a caller that postpones the (rows, V) pass until the upstream gradient
 * of the loss is known (it keeps `row_scratch` and, for logits input, the
 * logits themselves alive until then): this folds ctx.grad.mul_(loss_grad)
 * (transducer_loss.py:162) into the one pass that writes the gradient, without
 * the host ever reading loss_grad. */
int ot_gradient_apply_device_factor(const float *logits, const void *row_scratch,
                                    int64_t rows, int32_t V,
                                    int32_t from_log_softmax, float grad_scale,
                                    const float *device_factor, float *grad,
                                    void *stream);

/* Bytes of 16-byte aligned device scratch ot_gradient needs in `row_scratch`
 * (per-row coefficients, 24 bytes per packed row). */
size_t ot_gradient_scratch_bytes(int64_t rows);

/* In-place x *= *factor for n floats, skipped entirely on the device when
 * *factor == 1.  Replaces ctx.grad.mul_(loss_grad) in backward
 * (transducer_loss.py:162) without a host read of loss_grad. */
int ot_scale_by_device_scalar(float *x, int64_t n, const float *factor,
                              void *stream);

/* *loss = -scale * sum_b scores[b]: the reduction of the per-utterance
 * log-likelihoods to the loss (transducer_loss.py:145-147: loss = -1 * scores,
 * then .sum() or .mean(); pass scale = 1 or 1/N).  One launch, fixed summation
 * order. */
int ot_negative_sum(const float *scores, int32_t N, float scale, float *loss,
                    void *stream);

/* ot_row_coefficients and ot_negative_sum in one launch: the per-row
 * coefficients of the whole batch into `row_scratch`, and
 * *loss = -loss_scale * sum_b scores[b] (transducer_loss.py:145-147) with the
 * summation order, hence the bits, of ot_negative_sum.  `scores` are the
 * per-utterance log-likelihoods ot_alpha_beta wrote on the same stream. */
int ot_row_coefficients_loss(const float *lp, const float *den, const float *alpha,
                             const float *beta, const int32_t *targets,
                             const int32_t *logit_lengths,
                             const int32_t *target_lengths,
                             const int32_t *row_splits, int32_t N,
                             int32_t targets_cols, int64_t rows, int32_t blank,
                             int32_t from_log_softmax, int32_t one_sym_per_frame,
                             float grad_scale, void *row_scratch,
                             const float *scores, float loss_scale, float *loss,
                             void *stream);

/* Bytes of device scratch ot_transducer_loss needs for N utterances and
 * `rows` packed rows. */
size_t ot_workspace_bytes(int32_t N, int64_t rows);

/* The whole path on one stream, no host synchronisation:
 * row_splits -> log_probs -> alpha_beta -> gradient (ComputeTransducerLossCuda,
 * cuda.cu:402-457).  scores: (N,) log-likelihoods from alpha.  grad may be
 * NULL (forward only), equal to logits (in place, logits input only) or a
 * separate (rows, V) buffer.  `status` receives the batch facts; the caller
 * is responsible for checking them (sum_tu == rows, targets_max < V, ...)
 * BEFORE calling when the inputs are untrusted, e.g. with ot_row_splits.
 * max_u1 must equal max_b(U_b)+1. */
int ot_transducer_loss(const float *logits, const int32_t *targets,
                       const int32_t *logit_lengths,
                       const int32_t *target_lengths, int32_t N,
                       int32_t targets_cols, int64_t rows, int32_t V,
                       int32_t blank, int32_t from_log_softmax,
                       int32_t one_sym_per_frame, int32_t max_u1,
                       float grad_scale, void *workspace,
                       size_t workspace_bytes, float *scores, float *grad,
                       ot_batch_status *status, void *stream);

/* ot_transducer_loss for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It
 * has no counterpart in the reference, whose launchers allocate every temporary
 * with torch::empty (cuda.cu:416-446).  Same arguments, kernels and results as
 * ot_transducer_loss without `workspace`: the temporaries live in an array of
 * OT_STATIC_WORKSPACE_BYTES that is part of the library's device image (every GPU
 * the library runs on holds its own copy until the process ends).  The call
 * itself calls no hipMalloc / hipFree.  A batch with
 * ot_workspace_bytes(N, rows) > OT_STATIC_WORKSPACE_BYTES (about 44 bytes per
 * packed row: 1.1 million rows) returns OT_E_TOO_LARGE and launches nothing.
 * All calls on one GPU share the array: calls that overlap in time on one GPU
 * (two streams, two threads) race; calls on one stream are ordered and need no
 * clearing in between.  The first call on a device looks the array's address up
 * (hipGetSymbolAddress); make it outside any graph capture. */
#define OT_STATIC_WORKSPACE_BYTES (48u << 20)
int ot_transducer_loss_static(const float *logits, const int32_t *targets,
                              const int32_t *logit_lengths,
                              const int32_t *target_lengths, int32_t N,
                              int32_t targets_cols, int64_t rows, int32_t V,
                              int32_t blank, int32_t from_log_softmax,
                              int32_t one_sym_per_frame, int32_t max_u1,
                              float grad_scale, float *scores, float *grad,
                              ot_batch_status *status, void *stream);

/* ---- packed joiner input: the data format on the input side of the loss ----
 *
 * The loss consumes the joiner output for the valid (t, u) cells only, in the
 * packed row order above.  The reference leaves producing the joiner INPUT in
 * that order to its caller and shows it with Python lists and torch.cat
 * (README.md:166-177):
 *   x = cat_b (enc[b, :T_b, None, :] + dec[b, None, :U_b+1, :]).reshape(-1, D)
 *   activation = tanh(x)
 * The functions below do that, and its gradient, from the padded tensors
 *   enc (N, t_stride, D), t_stride >= max_b T_b        (encoder output)
 *   dec (N, u_stride, D), u_stride >= max_b U_b + 1    (prediction network output)
 * all float32 and contiguous. */
#define OT_ACT_NONE 0 /* out = enc + dec                                      */
#define OT_ACT_TANH 1 /* out = tanh(enc + dec)                                */
#define OT_ACT_RELU 2 /* out = max(enc + dec, 0)                              */
#define OT_JOINER_TILE_FRAMES 16 /* frames per partial decoder sum            */

/* out (rows, D), rows = row_splits[N]: for utterance b and cell (t, u),
 *   out[row_splits[b] + t*(U_b+1) + u] = act(enc[b,t] + dec[b,u]);
 * one streaming pass, 4*D bytes written per row.  Lengths beyond the strides
 * are clamped (nothing is read outside enc and dec); it is the caller's
 * business that `out` holds row_splits[N] rows. */
int ot_joiner_pack(const float *enc, const float *dec,
                   const int32_t *logit_lengths, const int32_t *target_lengths,
                   const int32_t *row_splits, int32_t N, int32_t t_stride,
                   int32_t u_stride, int32_t D, int32_t activation, float *out,
                   void *stream);

/* Gradient of ot_joiner_pack: given grad_out (rows, D) = d loss / d out,
 *   grad_enc[b,t,:] = sum_u grad_out[row(b,t,u)] * act'(enc[b,t] + dec[b,u])
 *   grad_dec[b,u,:] = sum_t (the same terms)
 * and zeros in the padding (t >= T_b, u > U_b); both outputs are written in
 * full.  One pass over grad_out; the decoder sums go through per-16-frame
 * partial sums in `workspace` (16-byte aligned, ot_joiner_unpack_workspace_bytes)
 * and are added in a fixed order, so results do not vary from run to run.
 * enc and dec are read only for OT_ACT_TANH and OT_ACT_RELU (may be NULL otherwise). */
size_t ot_joiner_unpack_workspace_bytes(int32_t N, int32_t t_stride,
                                        int32_t u_stride, int32_t D);
int ot_joiner_unpack_grad(const float *grad_out, const float *enc,
                          const float *dec, const int32_t *logit_lengths,
                          const int32_t *target_lengths,
                          const int32_t *row_splits, int32_t N, int32_t t_stride,
                          int32_t u_stride, int32_t D, int32_t activation,
                          void *workspace, size_t workspace_bytes,
                          float *grad_enc, float *grad_dec, void *stream);

/* ---- half-precision logits (not in the reference, which takes float32 only,
 * transducer-loss.cc:33) ----
 *
 * For a joiner that runs under mixed precision: the two passes over the
 * (rows, V) array read (and, for the gradient, write) 2-byte elements, all
 * arithmetic and every per-row array stay float32.  Use these two in place of
 * ot_log_probs and ot_gradient_apply; row offsets, lattice and coefficients
 * (ot_row_splits, ot_alpha_beta, ot_row_coefficients) are the float32 ones. */
#define OT_DTYPE_F32 0
#define OT_DTYPE_F16 1  /* IEEE binary16 */
#define OT_DTYPE_BF16 2 /* bfloat16      */

/* ot_log_probs for logits of `dtype` (OT_DTYPE_F16 or OT_DTYPE_BF16). */
int ot_log_probs_half(const void *logits, int32_t dtype, const int32_t *targets,
                      const int32_t *target_lengths, const int32_t *row_splits,
                      int32_t N, int32_t targets_cols, int64_t rows, int32_t V,
                      int32_t blank, int32_t from_log_softmax, float *den,
                      float *lp, void *stream);

/* ot_gradient_apply for logits and gradient of `dtype`; the gradient is
 * rounded to nearest even.  device_factor may be NULL (see
 * ot_gradient_apply_device_factor). */
int ot_gradient_apply_half(const void *logits, int32_t dtype,
                           const void *row_scratch, int64_t rows, int32_t V,
                           int32_t from_log_softmax, float grad_scale,
                           const float *device_factor, void *grad, void *stream);

/* ot_scale_by_device_scalar for n elements of `dtype` (product rounded to
 * nearest even). */
int ot_scale_by_device_scalar_half(void *x, int32_t dtype, int64_t n,
                                   const float *factor, void *stream);

/* ot_joiner_pack with the output rounded (to nearest even) to out_dtype =
 * OT_DTYPE_F16 or OT_DTYPE_BF16: the activations of a joiner whose projection
 * runs in 16 bits (ot_joiner_project), without a float32 array and a cast pass
 * in between.  enc and dec stay float32; D a multiple of 8, enc / dec / out
 * 16-byte aligned. */
int ot_joiner_pack_half(const float *enc, const float *dec,
                        const int32_t *logit_lengths,
                        const int32_t *target_lengths,
                        const int32_t *row_splits, int32_t N, int32_t t_stride,
                        int32_t u_stride, int32_t D, int32_t activation,
                        int32_t out_dtype, void *out, void *stream);

/* ot_joiner_unpack_grad for an incoming gradient of grad_dtype (any of the
 * three OT_DTYPE_*): a 16-bit gradient, as the backward of a 16-bit projection
 * produces it, is widened on the fly; sums and outputs stay float32. */
int ot_joiner_unpack_grad_from(const void *grad_out, int32_t grad_dtype,
                               const float *enc, const float *dec,
                               const int32_t *logit_lengths,
                               const int32_t *target_lengths,
                               const int32_t *row_splits, int32_t N,
                               int32_t t_stride, int32_t u_stride, int32_t D,
                               int32_t activation, void *workspace,
                               size_t workspace_bytes, float *grad_enc,
                               float *grad_dec, void *stream);

/* ---- output projection of the joiner fused with the denominators (no
 * counterpart in the reference: its caller computes
 * logits = Linear(tanh(enc + dec)) with torch, README.md:166-177, and the loss
 * re-reads all of them for logits.logsumexp(1), cuda.cu:427) ----
 *
 * logits[r, v] = sum_k x[r, k] * weight[v, k] + bias[v] on the matrix cores,
 * float32 accumulation, rounded once to `logits_dtype`, and
 * den[r] = log sum_v exp(logits[r, v]) of exactly the stored values, taken from
 * the accumulators: the loss then needs no pass of its own over the logits for
 * the denominators (ot_log_probs_given_den instead of ot_log_probs).
 *
 * x (rows, D) and weight (V, D) row-major of `dtype` (OT_DTYPE_F16 or
 * OT_DTYPE_BF16), 16-byte aligned, D a multiple of 64; bias (V) float32 or
 * NULL; logits (rows, V) of logits_dtype = OT_DTYPE_F32 or `dtype`;
 * den (rows) float32. */
int ot_joiner_project(const void *x, const void *weight, const float *bias,
                      int32_t dtype, int64_t rows, int32_t D, int32_t V,
                      void *logits, int32_t logits_dtype, float *den,
                      void *stream);

/* ot_joiner_project for a caller that lends a workspace of
 * ot_joiner_project_workspace_bytes(rows, V) bytes (4-byte aligned; contents
 * irrelevant before and after; 0 bytes for V <= 256).  With it, the 256-column
 * passes over the vocabulary of one block of rows run side by side on
 * workgroups of one XCD instead of one after the other on one workgroup, so
 * that x leaves HBM once whatever V is; every pass leaves a partial
 * log-sum-exp per row in the workspace and a second kernel merges them in pass
 * order.  Same logits, bit for bit; den from the same stored values with its
 * terms grouped by pass.  A NULL or short workspace falls back to
 * ot_joiner_project. */
size_t ot_joiner_project_workspace_bytes(int64_t rows, int32_t V);
int ot_joiner_project_ws(const void *x, const void *weight, const float *bias,
                         int32_t dtype, int64_t rows, int32_t D, int32_t V,
                         void *logits, int32_t logits_dtype, float *den,
                         void *workspace, size_t workspace_bytes, void *stream);

/* Backward of that projection with respect to its parameters (no counterpart
 * in the reference either: there autograd's Linear does it, README.md:176-177
 * with the loss's gradient of cuda.cu:471-489 as input):
 *     grad_weight[v, k] = sum_r grad_logits[r, v] * x[r, k]
 *     grad_bias[v]      = sum_r grad_logits[r, v]
 * on the matrix cores with float32 accumulation, the rows split into slices
 * whose partial sums are added in a fixed order (same bits on every run);
 * grad_weight is rounded once to `dtype`, grad_bias (may be NULL) is float32.
 *
 * grad_logits (rows, V) and x (rows, D) row-major of `dtype` (OT_DTYPE_F16 or
 * OT_DTYPE_BF16), 16-byte aligned, V and D multiples of 8; rows up to 2^31-1;
 * workspace: ot_joiner_weight_grad_workspace_bytes(rows, V, D) bytes, 16-byte
 * aligned, contents irrelevant before and after.  OT_E_TOO_LONG when a slice of
 * the rows is longer than 32-bit byte offsets address (rows * max(V, D) beyond
 * about 2^35). */
size_t ot_joiner_weight_grad_workspace_bytes(int64_t rows, int32_t V, int32_t D);
int ot_joiner_weight_grad(const void *grad_logits, const void *x, int32_t dtype,
                          int64_t rows, int32_t V, int32_t D, void *workspace,
                          size_t workspace_bytes, void *grad_weight,
                          float *grad_bias, void *stream);

/* The gather step of ot_log_probs for denominators that are already known
 * (ComputeLogProbs, cpu.cc:52-100, without the log-sum-exp in front of it):
 * lp[row] = (logits[row, blank], logits[row, target(row)]) - den[row];
 * logits of `dtype` (any of the three), rows >= row_splits[N] are left alone. */
int ot_log_probs_given_den(const void *logits, int32_t dtype, const float *den,
                           const int32_t *targets,
                           const int32_t *target_lengths,
                           const int32_t *row_splits, int32_t N,
                           int32_t targets_cols, int64_t rows, int32_t V,
                           int32_t blank, float *lp, void *stream);

/* Plain device-to-device copy kernel of n floats; used to calibrate profiler
 * byte counters against a transfer of known size. */
int ot_copy_floats(const float *src, float *dst, int64_t n, void *stream);

/* Text for a return value of the functions above. */
const char *ot_error_string(int code);

#ifdef __cplusplus
}
#endif
#endif /* OT_TRANSDUCER_H_ */
