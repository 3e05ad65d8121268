/* TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's transducer
 * loss path (optimized_transducer/csrc/cpu.cc and the integer row bookkeeping
 * of optimized_transducer/csrc/cuda.cu).  It is the parity checker for the HIP
 * kernels and the timed CPU baseline; the shipped package never links it.
 *
 * Every function exists twice: suffix _f32 follows the reference's float
 * arithmetic (expf / log1pf / logf, threshold logf(FLT_EPSILON)); suffix _f64
 * runs the same recursions in double and serves as an arbiter when two fp32
 * implementations disagree because of cancellation at large |alpha|, |beta|.
 *
 * How each function is pinned (tests/test_oracle_*.py):
 *   row_splits / row_ids : numpy cumsum / repeat; compiled reference n/a (CUDA only)
 *   logsumexp            : torch.logsumexp, numpy float64
 *   log_probs            : torch.log_softmax + indexing; compiled reference
 *   alpha / beta / scores: brute-force path enumeration, closed form for
 *                          constant logits, per-diagonal occupancy invariant,
 *                          compiled reference (oracle/_ref) end to end
 *   gradient (4 variants): float64 autograd through an independent torch DP,
 *                          row-sum invariants, compiled reference end to end
 */
#include <float.h>
#include <math.h>
#include <stdint.h>
#include <stddef.h>

/* Exclusive prefix sum of T_b * (U_b + 1) in int32, as the ATen sequence
 * cumsum(int32) + cat(zero) at cuda.cu:411-414 produces it (wraps on
 * overflow like int32 arithmetic does).  Returns the int64 total. */
int64_t ot_oracle_row_splits(const int32_t *logit_lengths,
                             const int32_t *target_lengths, int32_t N,
                             int32_t *row_splits) {
  uint32_t acc = 0;
  int64_t total = 0;
  row_splits[0] = 0;
  for (int32_t b = 0; b < N; ++b) {
    uint32_t sz = (uint32_t)logit_lengths[b] * (uint32_t)(target_lengths[b] + 1);
    acc += sz;
    total += (int64_t)logit_lengths[b] * (int64_t)(target_lengths[b] + 1);
    row_splits[b + 1] = (int32_t)acc;
  }
  return total;
}

/* row_ids[i] = b such that row_splits[b] <= i < row_splits[b+1]; what
 * mgpu::load_balance_search computes at cuda.cu:56-57 (RowSplitsToRowIds,
 * cuda.cu:40-59). */
void ot_oracle_row_ids(const int32_t *row_splits, int32_t N, int32_t *row_ids) {
  for (int32_t b = 0; b < N; ++b)
    for (int32_t i = row_splits[b]; i < row_splits[b + 1]; ++i) row_ids[i] = b;
}

/* Row -> (b, t, u, target) decode used by every per-row CUDA kernel of the
 * reference (kernels.cu:40-47, kernels.cu:538-540): u = idx1 % (U+1),
 * t = idx1 / (U+1), target = targets[b][u] for u < U and -1 otherwise. */
void ot_oracle_decode_rows(const int32_t *row_splits, const int32_t *row_ids,
                           const int32_t *targets, int32_t targets_cols,
                           const int32_t *target_lengths, int32_t rows,
                           int32_t *out_btu_target /* (rows, 4) */) {
  for (int32_t i = 0; i < rows; ++i) {
    int32_t b = row_ids[i];
    int32_t U1 = target_lengths[b] + 1;
    int32_t idx1 = i - row_splits[b];
    int32_t t = idx1 / U1, u = idx1 % U1;
    out_btu_target[4 * i + 0] = b;
    out_btu_target[4 * i + 1] = t;
    out_btu_target[4 * i + 2] = u;
    out_btu_target[4 * i + 3] =
        (u < U1 - 1) ? targets[(int64_t)b * targets_cols + u] : -1;
  }
}

#define REAL float
#define SUFFIX _f32
#define R_EXP expf
#define R_LOG logf
#define R_LOG1P log1pf
/* logf(FLT_EPSILON), cpu.cc:15-16 */
#define MIN_LOG_DIFF (-15.9423847198486328125f)
#include "transducer_oracle_impl.h"
#undef REAL
#undef SUFFIX
#undef R_EXP
#undef R_LOG
#undef R_LOG1P
#undef MIN_LOG_DIFF

#define REAL double
#define SUFFIX _f64
#define R_EXP exp
#define R_LOG log
#define R_LOG1P log1p
/* log(DBL_EPSILON) */
#define MIN_LOG_DIFF (-36.04365338911715)
#include "transducer_oracle_impl.h"
