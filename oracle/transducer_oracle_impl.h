/* TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's transducer
 * loss path, used as the parity checker.  Nothing in the shipped package may
 * include, link or call this file; only tests, the smoke check and the
 * benchmark's CPU-baseline leg do.
 *
 * This header is a body that is included twice by transducer_oracle.c, once
 * with REAL = float (the reference's arithmetic) and once with REAL = double
 * (an arbiter with the same recursions and no fp32 cancellation).
 *
 * Layout (reference README.md:133-136): utterance b owns packed rows
 * [row_splits[b], row_splits[b+1]); inside it cell (t, u), 0 <= t < T_b,
 * 0 <= u <= U_b, is row  row_splits[b] + t * (U_b + 1) + u.
 *
 * Cells the reference leaves uninitialised are written as NaN here so that a
 * comparison has to mask them explicitly:
 *   - lp[r][1] at u == U            (optimized_transducer/csrc/cpu.cc:92-94)
 *   - alpha / beta outside the band of the one-symbol-per-frame lattice
 *                                    (cpu.cc:295-296, cpu.cc:430-431)
 */

#ifndef REAL
#error "include from transducer_oracle.c"
#endif

#define OT_CAT_(a, b) a##b
#define OT_CAT(a, b) OT_CAT_(a, b)
#define FN(name) OT_CAT(name, SUFFIX)

/* Two-term log-add.  Follows LogSumExp, cpu.cc:18-35: the larger operand plus
 * log1p(exp(-|a-b|)), and just the larger operand once the difference drops
 * below log(epsilon).  A NaN difference (-inf minus -inf) fails the >= test
 * and also yields the larger operand. */
static REAL FN(log_add)(REAL a, REAL b) {
  REAL diff;
  if (a < b) {
    diff = a - b;
    a = b;
  } else {
    diff = b - a;
  }
  if (diff >= MIN_LOG_DIFF) return a + R_LOG1P(R_EXP(diff));
  return a;
}

/* Per-row log-sum-exp over the vocabulary.  Stands in for the ATen call
 * `logits.logsumexp(1)` at cpu.cc:770 (and cuda.cu:427).  ATen evaluates
 *   m = max(row);  m = 0 if |m| is inf;  log(sum(exp(row - m))) + m
 * in the tensor's dtype with a cascade sum; here each term exp(x - m) is
 * rounded to REAL and the sum is carried in double, which is what a cascade
 * sum approximates. */
void FN(ot_oracle_logsumexp)(const float *logits, int64_t rows, int32_t V,
                             REAL *den) {
  for (int64_t r = 0; r < rows; ++r) {
    const float *x = logits + r * (int64_t)V;
    REAL m = (REAL)x[0];
    for (int32_t v = 1; v < V; ++v) {
      if ((REAL)x[v] > m) m = (REAL)x[v];
    }
    if (isinf(m)) m = 0;
    double s = 0.0;
    for (int32_t v = 0; v < V; ++v) s += (double)R_EXP((REAL)x[v] - m);
    den[r] = R_LOG((REAL)s) + m;
  }
}

/* Blank / target log-probability gather.
 * den != NULL: ComputeLogProbs, cpu.cc:52-100 (value minus denominator).
 * den == NULL: ComputeLogProbsForLogSoftmax, cpu.cc:116-155 (value as is).
 * lp is (rows, 2): column 0 blank, column 1 symbol (cpu.cc:12-13). */
void FN(ot_oracle_log_probs)(const float *logits, const REAL *den,
                             const int32_t *targets, int32_t targets_cols,
                             const int32_t *logit_lengths,
                             const int32_t *target_lengths, int32_t N,
                             int32_t V, int32_t blank, REAL *lp) {
  int64_t r = 0;
  for (int32_t b = 0; b < N; ++b) {
    const int32_t T = logit_lengths[b], U = target_lengths[b];
    const int32_t *tg = targets + (int64_t)b * targets_cols;
    for (int32_t t = 0; t < T; ++t) {
      for (int32_t u = 0; u <= U; ++u, ++r) {
        const float *x = logits + r * (int64_t)V;
        const REAL d = den ? den[r] : (REAL)0;
        lp[2 * r] = den ? (REAL)x[blank] - d : (REAL)x[blank];
        if (u < U)
          lp[2 * r + 1] = den ? (REAL)x[tg[u]] - d : (REAL)x[tg[u]];
        else
          lp[2 * r + 1] = (REAL)NAN; /* uninitialised in the reference */
      }
    }
  }
}

#define LPB(t, u) lpb[2 * ((int64_t)(t)*U1 + (u))]
#define LPS(t, u) lpb[2 * ((int64_t)(t)*U1 + (u)) + 1]
#define AL(t, u) a[(int64_t)(t)*U1 + (u)]
#define BE(t, u) be[(int64_t)(t)*U1 + (u)]

/* Forward variables.
 * one_sym_per_frame == 0: ComputeAlpha, cpu.cc:162-244.
 * one_sym_per_frame != 0: ComputeAlphaOneSymPerFrame, cpu.cc:246-317.
 * scores[b] = alpha(T-1, U) + lp(T-1, U).blank  (cpu.cc:240, cpu.cc:314). */
void FN(ot_oracle_alpha)(const REAL *lp, const int32_t *logit_lengths,
                         const int32_t *target_lengths, int32_t N,
                         int32_t one_sym_per_frame, REAL *alpha, REAL *scores) {
  int64_t off = 0;
  for (int32_t b = 0; b < N; ++b) {
    const int32_t T = logit_lengths[b], U1 = target_lengths[b] + 1;
    const REAL *lpb = lp + 2 * off;
    REAL *a = alpha + off;
    for (int64_t i = 0; i < (int64_t)T * U1; ++i) a[i] = (REAL)NAN;
    AL(0, 0) = 0;
    if (!one_sym_per_frame) {
      for (int32_t t = 1; t < T; ++t) AL(t, 0) = AL(t - 1, 0) + LPB(t - 1, 0);
      for (int32_t u = 1; u < U1; ++u) AL(0, u) = AL(0, u - 1) + LPS(0, u - 1);
      for (int32_t t = 1; t < T; ++t)
        for (int32_t u = 1; u < U1; ++u)
          AL(t, u) = FN(log_add)(AL(t - 1, u) + LPB(t - 1, u),
                                 AL(t, u - 1) + LPS(t, u - 1));
    } else {
      const int32_t diff = T - 1 - (U1 - 1); /* cpu.cc:279 */
      for (int32_t t = 1; t <= diff; ++t)
        AL(t, 0) = AL(t - 1, 0) + LPB(t - 1, 0);
      for (int32_t t = 1; t < T; ++t) {
        for (int32_t u = 1; u < U1; ++u) {
          if (u > t || t - u > diff) continue;
          if (t == u)
            AL(t, u) = AL(t - 1, u - 1) + LPS(t - 1, u - 1);
          else
            AL(t, u) = FN(log_add)(AL(t - 1, u) + LPB(t - 1, u),
                                   AL(t - 1, u - 1) + LPS(t - 1, u - 1));
        }
      }
    }
    scores[b] = AL(T - 1, U1 - 1) + LPB(T - 1, U1 - 1);
    off += (int64_t)T * U1;
  }
}

/* Backward variables.
 * one_sym_per_frame == 0: ComputeBeta, cpu.cc:319-382.
 * one_sym_per_frame != 0: ComputeBetaOneSymPerFrame, cpu.cc:384-451.
 * scores[b] = beta(0, 0)  (cpu.cc:377, cpu.cc:446). */
void FN(ot_oracle_beta)(const REAL *lp, const int32_t *logit_lengths,
                        const int32_t *target_lengths, int32_t N,
                        int32_t one_sym_per_frame, REAL *beta, REAL *scores) {
  int64_t off = 0;
  for (int32_t b = 0; b < N; ++b) {
    const int32_t T = logit_lengths[b], U1 = target_lengths[b] + 1;
    const int32_t U = U1 - 1;
    const REAL *lpb = lp + 2 * off;
    REAL *be = beta + off;
    for (int64_t i = 0; i < (int64_t)T * U1; ++i) be[i] = (REAL)NAN;
    BE(T - 1, U) = LPB(T - 1, U);
    if (!one_sym_per_frame) {
      for (int32_t t = T - 2; t >= 0; --t) BE(t, U) = BE(t + 1, U) + LPB(t, U);
      for (int32_t u = U - 1; u >= 0; --u)
        BE(T - 1, u) = BE(T - 1, u + 1) + LPS(T - 1, u);
      for (int32_t t = T - 2; t >= 0; --t)
        for (int32_t u = U - 1; u >= 0; --u)
          BE(t, u) = FN(log_add)(BE(t + 1, u) + LPB(t, u),
                                 BE(t, u + 1) + LPS(t, u));
    } else {
      const int32_t diff = T - 1 - U; /* cpu.cc:412 */
      for (int32_t t = T - 2; t >= U; --t) BE(t, U) = BE(t + 1, U) + LPB(t, U);
      for (int32_t t = T - 2; t >= 0; --t) {
        for (int32_t u = U - 1; u >= 0; --u) {
          if (u > t || t - u > diff) continue;
          if (t - u == diff)
            BE(t, u) = BE(t + 1, u + 1) + LPS(t, u);
          else
            BE(t, u) = FN(log_add)(BE(t + 1, u) + LPB(t, u),
                                   BE(t + 1, u + 1) + LPS(t, u));
        }
      }
    }
    scores[b] = BE(0, 0);
    off += (int64_t)T * U1;
  }
}

/* Gradient of -log-likelihood with respect to the rows of `logits`.
 *   den != NULL, one_sym == 0: ComputeGradient, cpu.cc:467-528
 *   den != NULL, one_sym != 0: ComputeGradientOneSymPerFrame, cpu.cc:545-612
 *   den == NULL, one_sym == 0: ComputeGradientForLogSoftmax, cpu.cc:626-676
 *   den == NULL, one_sym != 0: ComputeGradientForLogSoftmaxOneSymPerFrame,
 *                              cpu.cc:691-751
 * Evaluation order kept as in the reference: c = (alpha + loss) - den,
 * g = logit + c, then g + beta.  When REAL is float, `grad` may alias
 * `logits` (each element is read before it is written, cpu.cc:512-522).
 * `mag` (may be NULL; same shape as grad, must not alias logits) receives for
 * every entry the sum of the absolute values of the exponentials it is made
 * of, exp(g + beta) + sub: the scale on which a rounding difference in alpha,
 * beta or a denominator moves the entry.  It is not part of the reference; the
 * tests derive their per-entry comparison bound from it. */
void FN(ot_oracle_gradient)(const float *logits, const int32_t *targets,
                            int32_t targets_cols, const int32_t *logit_lengths,
                            const int32_t *target_lengths, int32_t N, int32_t V,
                            int32_t blank, const REAL *den, const REAL *alpha,
                            const REAL *beta, int32_t one_sym_per_frame,
                            REAL *grad, REAL *mag) {
  int64_t off = 0;
  for (int32_t b = 0; b < N; ++b) {
    const int32_t T = logit_lengths[b], U1 = target_lengths[b] + 1;
    const int32_t U = U1 - 1;
    const int32_t diff = T - 1 - U;
    const int32_t *tg = targets + (int64_t)b * targets_cols;
    const REAL *a = alpha + off, *be = beta + off;
    const REAL loss = -be[0];
    for (int32_t t = 0; t < T; ++t) {
      for (int32_t u = 0; u < U1; ++u) {
        const int64_t r = off + (int64_t)t * U1 + u;
        const float *x = logits + r * (int64_t)V;
        REAL *gr = grad + r * (int64_t)V;
        REAL *mg = mag ? mag + r * (int64_t)V : NULL;
        if (one_sym_per_frame && (u > t || t - u > diff)) {
          for (int32_t v = 0; v < V; ++v) gr[v] = 0; /* cpu.cc:582-586 */
          if (mg)
            for (int32_t v = 0; v < V; ++v) mg[v] = 0;
          continue;
        }
        const int32_t target_u = (u < U) ? tg[u] : -1;
        const REAL c = den ? AL(t, u) + loss - den[r] : AL(t, u) + loss;
        /* where the blank arc and the symbol arc out of (t, u) lead */
        const int blank_open = one_sym_per_frame ? (t - u < diff) : (t < T - 1);
        const REAL beta_sym =
            (u < U) ? (one_sym_per_frame ? (t + 1 < T ? BE(t + 1, u + 1) : 0)
                                         : BE(t, u + 1))
                    : 0;
        for (int32_t v = 0; v < V; ++v) {
          const REAL g = (REAL)x[v] + c;
          REAL sub;
          int special = 1;
          if (v == blank && t == T - 1 && u == U)
            sub = R_EXP(g);
          else if (v == blank && blank_open)
            sub = R_EXP(g + BE(t + 1, u));
          else if (u < U && v == target_u)
            sub = R_EXP(g + beta_sym);
          else {
            sub = 0;
            special = 0;
          }
          if (den) {
            const REAL whole = R_EXP(g + BE(t, u));
            gr[v] = special ? whole - sub : whole;
            if (mg) mg[v] = whole + sub;
          } else {
            gr[v] = special ? -sub : 0;
            if (mg) mg[v] = sub;
          }
        }
      }
    }
    off += (int64_t)T * U1;
  }
}

#undef LPB
#undef LPS
#undef AL
#undef BE

/* Whole path: ComputeTransducerLossCpu, cpu.cc:754-827.
 * `work` must hold 5 * rows REALs (den, lp x2, alpha, beta).
 * scores = log-likelihoods from alpha (not negated, cpu.cc:826);
 * scores_beta = beta(0,0), which the reference only uses for its allclose
 * sanity check (cpu.cc:795-797).  grad may be NULL (no gradient wanted). */
void FN(ot_oracle_transducer_loss)(
    const float *logits, const int32_t *targets, int32_t targets_cols,
    const int32_t *logit_lengths, const int32_t *target_lengths, int32_t N,
    int64_t rows, int32_t V, int32_t blank, int32_t from_log_softmax,
    int32_t one_sym_per_frame, REAL *work, REAL *scores, REAL *scores_beta,
    REAL *grad, REAL *mag) {
  REAL *den = work, *lp = work + rows, *alpha = work + 3 * rows,
       *beta = work + 4 * rows;
  if (!from_log_softmax) FN(ot_oracle_logsumexp)(logits, rows, V, den);
  FN(ot_oracle_log_probs)(logits, from_log_softmax ? NULL : den, targets,
                          targets_cols, logit_lengths, target_lengths, N, V,
                          blank, lp);
  FN(ot_oracle_alpha)(lp, logit_lengths, target_lengths, N, one_sym_per_frame,
                      alpha, scores);
  FN(ot_oracle_beta)(lp, logit_lengths, target_lengths, N, one_sym_per_frame,
                     beta, scores_beta);
  if (grad)
    FN(ot_oracle_gradient)(logits, targets, targets_cols, logit_lengths,
                           target_lengths, N, V, blank,
                           from_log_softmax ? NULL : den, alpha, beta,
                           one_sym_per_frame, grad, mag);
}

#undef FN
#undef OT_CAT
#undef OT_CAT_
