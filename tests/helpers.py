"""Shared test helpers: oracle access, independent float64 models, tolerances."""
import glob
import itertools
import math
import os

import numpy as np

from oracle import oracle

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN_DIR = os.path.join(ROOT, "tests", "golden")
EPS32 = float(np.finfo(np.float32).eps)

# north-star tolerance for fp32 losses and gradients
RTOL = 1e-5
ATOL = 1e-5


def golden_files():
    return sorted(glob.glob(os.path.join(GOLDEN_DIR, "*.npz")))


def golden_modes(g):
    """[(from_log_softmax, one_sym_per_frame)] stored in a golden file."""
    return [(bool(f), bool(o)) for f in (0, 1) for o in (0, 1)
            if "scores_fls%d_osf%d" % (f, o) in g.files]


def log_softmax32(x):
    m = x.max(axis=1, keepdims=True)
    z = (x - m).astype(np.float64)
    return (z - np.log(np.exp(z).sum(axis=1, keepdims=True))).astype(np.float32)


# Roundings of size ulp(|log-likelihood|) that two float32 evaluations of one gradient
# entry may differ by (see lattice_noise_tolerance).
NOISE_K = 4.0


def lattice_noise_tolerance(ref_grad, loss_per_row, mag, k=NOISE_K, scale=1.0):
    """Elementwise bound for comparing two fp32 evaluations of the gradient.

    Every entry is a difference of exponentials exp(x + c + beta) whose
    argument is a sum of terms of magnitude |loss| (cpu.cc:509-522), so two
    correct fp32 evaluations that differ by one rounding anywhere in alpha,
    beta or the denominator differ by about ulp(|loss|) in that argument, i.e.
    by ulp(|loss|) times each exponential.  ``mag`` is the sum of an entry's
    exponentials (``return_magnitude=True`` of the oracle), so the bound scales
    with the entry: the north-star tolerance plus k such roundings.  A wrong
    small entry fails; an all-zero result fails wherever the entry exceeds
    about 1e-5.  ``ref_grad`` and ``mag`` belong to the unscaled gradient;
    ``scale`` is the factor (upstream gradient, 1/N) the compared one carries:
    it multiplies the relative parts, and the absolute part when below 1.
    """
    noise = k * EPS32 * np.abs(loss_per_row)[:, None] * mag
    return min(scale, 1.0) * ATOL + scale * (RTOL * np.abs(ref_grad) + noise)


def oracle_noise_unit(x, targets, T, U, blank, fls, osf):
    """(scores, fp32 gradient, per-entry noise unit) from one run of the fp32 oracle: the
    unit is one float32 rounding of an entry's exponent, eps * |log-likelihood of the
    utterance| * (sum of the entry's exponentials); lattice_noise_tolerance allows
    NOISE_K of them on top of the north-star tolerance."""
    s, g, mag = oracle.compute_transducer_loss(np.ascontiguousarray(x).copy(), targets, T, U, blank,
                                               fls, osf, return_magnitude=True)
    return s, g, EPS32 * np.abs(per_row(s, T, U))[:, None] * mag


def oracle_tolerance(x, targets, T, U, blank, fls, osf, scale=1.0, k=NOISE_K):
    """(scores, unscaled fp32 gradient, elementwise bound for `scale` x that gradient)
    from one run of the fp32 oracle."""
    s, g, mag = oracle.compute_transducer_loss(np.ascontiguousarray(x).copy(), targets, T, U, blank,
                                               fls, osf, return_magnitude=True)
    return s, g, lattice_noise_tolerance(g, per_row(s, T, U), mag, k=k, scale=scale)


def per_row(values_per_utt, T, U):
    """Broadcast one value per utterance to its packed rows."""
    sizes = np.asarray(T, np.int64) * (np.asarray(U, np.int64) + 1)
    return np.repeat(np.asarray(values_per_utt), sizes)


# --------------------------------------------------------------------------
# independent float64 models (written from the recursions, not from the oracle)
# --------------------------------------------------------------------------
def brute_force_loglik(lp_blank, lp_sym, one_sym_per_frame):
    """log sum over all alignments, by explicit enumeration.

    lp_blank, lp_sym: (T, U+1) float64 arrays of log-probabilities.
    standard: a path is an interleaving of U symbol arcs and T-1 blank arcs
      from (0,0) to (T-1,U), followed by the final blank out of (T-1,U).
    modified: every arc advances t; a path picks at which U of the first T-1
      frames a symbol is emitted; the final blank leaves (T-1,U).
    """
    T, U1 = lp_blank.shape
    U = U1 - 1
    total = []
    if not one_sym_per_frame:
        for sym_pos in itertools.combinations(range(T - 1 + U), U):
            t = u = 0
            s = 0.0
            sym_pos = set(sym_pos)
            for i in range(T - 1 + U):
                if i in sym_pos:
                    s += lp_sym[t, u]
                    u += 1
                else:
                    s += lp_blank[t, u]
                    t += 1
            total.append(s + lp_blank[T - 1, U])
    else:
        if U > T - 1:
            return -math.inf
        for sym_frames in itertools.combinations(range(T - 1), U):
            sym_frames = set(sym_frames)
            u = 0
            s = 0.0
            for t in range(T - 1):
                if t in sym_frames:
                    s += lp_sym[t, u]
                    u += 1
                else:
                    s += lp_blank[t, u]
            total.append(s + lp_blank[T - 1, U])
    total = np.array(total)
    m = total.max()
    return float(m + np.log(np.exp(total - m).sum()))


def torch_loss_f64(logits, targets, T, U, blank, from_log_softmax, one_sym_per_frame):
    """Differentiable float64 transducer loss in plain torch (forward recursion
    only, written from README.md:49-61 of the reference); returns per-utterance
    log-likelihoods as a torch tensor attached to `logits`."""
    import torch
    lsm = logits if from_log_softmax else torch.log_softmax(logits, dim=1)
    out = []
    off = 0
    for b in range(len(T)):
        Tb, Ub = int(T[b]), int(U[b])
        U1 = Ub + 1
        block = lsm[off:off + Tb * U1].reshape(Tb, U1, -1)
        lpb = block[:, :, blank]
        if Ub > 0:
            idx = torch.as_tensor(np.asarray(targets[b][:Ub], dtype=np.int64))
            lps = block[:, :Ub, :].gather(2, idx.view(1, Ub, 1).expand(Tb, Ub, 1)).squeeze(2)
        neg = torch.tensor(-math.inf, dtype=lsm.dtype)
        alpha = [[None] * U1 for _ in range(Tb)]
        for t in range(Tb):
            for u in range(U1):
                if t == 0 and u == 0:
                    alpha[t][u] = torch.zeros((), dtype=lsm.dtype)
                    continue
                terms = []
                if not one_sym_per_frame:
                    if t > 0:
                        terms.append(alpha[t - 1][u] + lpb[t - 1, u])
                    if u > 0:
                        terms.append(alpha[t][u - 1] + lps[t, u - 1])
                else:
                    if t > 0:
                        terms.append(alpha[t - 1][u] + lpb[t - 1, u])
                    if t > 0 and u > 0:
                        terms.append(alpha[t - 1][u - 1] + lps[t - 1, u - 1])
                terms = [x for x in terms if x is not None and torch.isfinite(x)]
                alpha[t][u] = torch.logsumexp(torch.stack(terms), 0) if terms else neg
        out.append(alpha[Tb - 1][Ub] + lpb[Tb - 1, Ub])
        off += Tb * U1
    return torch.stack(out)


def oracle_full(x, w_targets, T, U, blank, fls, osf, dtype=np.float32):
    """Oracle scores, gradient and intermediate arrays for a batch."""
    return oracle.compute_transducer_loss(np.ascontiguousarray(x).copy(), w_targets, T, U, blank,
                                          fls, osf, dtype=dtype, return_parts=True)


def random_batch(rng, N, tmax, umax, V, one_sym_per_frame=False, tmin=1, umin=0, target_low=1):
    """Random ragged batch; targets are drawn from [target_low, V) (1 keeps them off blank=0)."""
    T = rng.integers(tmin, tmax + 1, size=N)
    U = np.array([rng.integers(umin, min(umax, (t - 1) if one_sym_per_frame else umax) + 1)
                  if (not one_sym_per_frame or t - 1 >= umin) else 0 for t in T])
    if U.max() == 0:
        T[-1] = max(T[-1], 3)
        U[-1] = min(umax, 2)
    targets = rng.integers(target_low, V, size=(N, int(U.max())))
    rows = int((T * (U + 1)).sum())
    logits = rng.standard_normal((rows, V)).astype(np.float32)
    return (T.astype(np.int32), U.astype(np.int32), targets.astype(np.int32), logits)
