"""ctypes/numpy front end of ``liboracle.so`` (TEST INFRASTRUCTURE ONLY).

The C side restates optimized_transducer/csrc/cpu.cc function by function; this
module only marshals numpy arrays and mirrors the Python-level arithmetic of
optimized_transducer/python/optimized_transducer/transducer_loss.py:133-170
(sign flip, reduction, ``grad /= N``, ``grad *= loss_grad``).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None


def build(force=False):
    """Compile liboracle.so with the Makefile next to this file."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE, "liboracle.so"] + (["-B"] if force else []),
                       check=True, stdout=subprocess.DEVNULL)


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.ot_oracle_row_splits.restype = ctypes.c_int64
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _i32(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.int32))


def row_splits(logit_lengths, target_lengths):
    """int32 (N+1,) exclusive prefix of T*(U+1) and the int64 total."""
    T, U = _i32(logit_lengths), _i32(target_lengths)
    out = np.empty(T.size + 1, dtype=np.int32)
    total = lib().ot_oracle_row_splits(_p(T), _p(U), ctypes.c_int32(T.size), _p(out))
    return out, int(total)


def row_ids(splits):
    splits = _i32(splits)
    out = np.empty(int(splits[-1]), dtype=np.int32)
    lib().ot_oracle_row_ids(_p(splits), ctypes.c_int32(splits.size - 1), _p(out))
    return out


def decode_rows(splits, ids, targets, target_lengths):
    splits, ids, targets, U = _i32(splits), _i32(ids), _i32(targets), _i32(target_lengths)
    out = np.empty((ids.size, 4), dtype=np.int32)
    lib().ot_oracle_decode_rows(_p(splits), _p(ids), _p(targets),
                                ctypes.c_int32(targets.shape[1]), _p(U),
                                ctypes.c_int32(ids.size), _p(out))
    return out


def _real(dtype):
    dtype = np.dtype(dtype)
    assert dtype in (np.float32, np.float64)
    return dtype, ("_f32" if dtype == np.float32 else "_f64")


def logsumexp(logits, dtype=np.float32):
    dtype, sfx = _real(dtype)
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    den = np.empty(logits.shape[0], dtype=dtype)
    getattr(lib(), "ot_oracle_logsumexp" + sfx)(
        _p(logits), ctypes.c_int64(logits.shape[0]), ctypes.c_int32(logits.shape[1]), _p(den))
    return den


def log_probs(logits, den, targets, logit_lengths, target_lengths, blank, dtype=np.float32):
    dtype, sfx = _real(dtype)
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    targets, T, U = _i32(targets), _i32(logit_lengths), _i32(target_lengths)
    if den is not None:
        den = np.ascontiguousarray(den, dtype=dtype)
    lp = np.empty((logits.shape[0], 2), dtype=dtype)
    getattr(lib(), "ot_oracle_log_probs" + sfx)(
        _p(logits), _p(den), _p(targets), ctypes.c_int32(targets.shape[1]), _p(T), _p(U),
        ctypes.c_int32(T.size), ctypes.c_int32(logits.shape[1]), ctypes.c_int32(blank), _p(lp))
    return lp


def _dp(name, lp, logit_lengths, target_lengths, one_sym_per_frame):
    dtype, sfx = _real(lp.dtype)
    lp = np.ascontiguousarray(lp)
    T, U = _i32(logit_lengths), _i32(target_lengths)
    out = np.empty(lp.shape[0], dtype=dtype)
    scores = np.empty(T.size, dtype=dtype)
    getattr(lib(), name + sfx)(_p(lp), _p(T), _p(U), ctypes.c_int32(T.size),
                               ctypes.c_int32(int(one_sym_per_frame)), _p(out), _p(scores))
    return out, scores


def alpha(lp, logit_lengths, target_lengths, one_sym_per_frame=False):
    return _dp("ot_oracle_alpha", lp, logit_lengths, target_lengths, one_sym_per_frame)


def beta(lp, logit_lengths, target_lengths, one_sym_per_frame=False):
    return _dp("ot_oracle_beta", lp, logit_lengths, target_lengths, one_sym_per_frame)


def gradient(logits, targets, logit_lengths, target_lengths, blank, den, alpha_, beta_,
             one_sym_per_frame=False, out=None, mag=None):
    """``mag`` (optional array like the gradient) receives the per-entry sum of the
    absolute values of the exponentials an entry is made of (a tolerance scale)."""
    dtype, sfx = _real(alpha_.dtype)
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    targets, T, U = _i32(targets), _i32(logit_lengths), _i32(target_lengths)
    grad = np.empty(logits.shape, dtype=dtype) if out is None else out
    getattr(lib(), "ot_oracle_gradient" + sfx)(
        _p(logits), _p(targets), ctypes.c_int32(targets.shape[1]), _p(T), _p(U),
        ctypes.c_int32(T.size), ctypes.c_int32(logits.shape[1]), ctypes.c_int32(blank),
        _p(den), _p(alpha_), _p(beta_), ctypes.c_int32(int(one_sym_per_frame)), _p(grad),
        _p(mag))
    return grad


def compute_transducer_loss(logits, targets, logit_lengths, target_lengths, blank,
                            from_log_softmax, one_sym_per_frame, want_grad=True,
                            dtype=np.float32, in_place=False, return_parts=False,
                            return_magnitude=False):
    """Counterpart of ``_optimized_transducer.compute_transducer_loss``.

    Returns ``(scores, grad)``; scores are +log-likelihoods (cpu.cc:826).  With
    ``in_place=True`` (float32, logits input) the gradient overwrites ``logits``
    as the reference does (cpu.cc:814).  With ``return_magnitude=True`` a third
    value follows: per gradient entry, the sum of the absolute values of the
    exponentials it is the difference of (see ``ot_oracle_gradient``).
    """
    dtype, sfx = _real(dtype)
    assert logits.dtype == np.float32 and logits.flags.c_contiguous
    targets, T, U = _i32(targets), _i32(logit_lengths), _i32(target_lengths)
    rows, V = logits.shape
    work = np.empty(5 * rows, dtype=dtype)
    scores = np.empty(T.size, dtype=dtype)
    scores_beta = np.empty(T.size, dtype=dtype)
    grad = None
    if want_grad:
        if in_place and not from_log_softmax and dtype == np.float32:
            grad = logits
        else:
            grad = np.empty((rows, V), dtype=dtype)
    mag = np.empty((rows, V), dtype=dtype) if (want_grad and return_magnitude) else None
    getattr(lib(), "ot_oracle_transducer_loss" + sfx)(
        _p(logits), _p(targets), ctypes.c_int32(targets.shape[1]), _p(T), _p(U),
        ctypes.c_int32(T.size), ctypes.c_int64(rows), ctypes.c_int32(V),
        ctypes.c_int32(blank), ctypes.c_int32(int(from_log_softmax)),
        ctypes.c_int32(int(one_sym_per_frame)), _p(work), _p(scores), _p(scores_beta), _p(grad),
        _p(mag))
    if return_magnitude:
        assert not return_parts
        return scores, grad, mag
    if return_parts:
        parts = dict(den=work[:rows], lp=work[rows:3 * rows].reshape(rows, 2),
                     alpha=work[3 * rows:4 * rows], beta=work[4 * rows:5 * rows],
                     scores_beta=scores_beta)
        return scores, grad, parts
    return scores, grad


def transducer_loss(logits, targets, logit_lengths, target_lengths, blank, from_log_softmax,
                    one_sym_per_frame=False, reduction="mean", loss_grad=1.0,
                    dtype=np.float32):
    """Loss value and d(loss * loss_grad)/d(logits), as transducer_loss.py:133-170."""
    assert reduction in ("mean", "sum")
    scores, grad = compute_transducer_loss(logits, targets, logit_lengths, target_lengths,
                                           blank, from_log_softmax, one_sym_per_frame,
                                           dtype=dtype)
    real = np.dtype(dtype).type
    loss = -scores
    n = len(scores)
    if reduction == "mean":
        loss = loss.mean(dtype=dtype)
        grad /= real(n)
    else:
        loss = loss.sum(dtype=dtype)
    grad *= real(loss_grad)
    return loss, grad


# ---------------------------------------------------------------- packed joiner input
def pack_joiner(encoder_out, decoder_out, logit_lengths, target_lengths, activation=None,
                dtype=np.float32):
    """The reference's recipe for the joiner input (README.md:166-177), literally:
    per utterance e[:T, None, :] + d[None, :U+1, :], reshaped to (T*(U+1), D),
    concatenated; then tanh when activation == "tanh" (the README's choice), max(x, 0)
    when activation == "relu"."""
    enc = np.asarray(encoder_out, dtype=dtype)
    dec = np.asarray(decoder_out, dtype=dtype)
    D = enc.shape[2]
    parts = []
    for i in range(enc.shape[0]):
        e = enc[i, :int(logit_lengths[i]), :]
        d = dec[i, :int(target_lengths[i]) + 1, :]
        parts.append((e[:, None, :] + d[None, :, :]).reshape(-1, D))
    x = np.concatenate(parts)
    if activation == "relu":
        return np.maximum(x, 0)
    return np.tanh(x) if activation == "tanh" else x


def pack_joiner_backward(grad_out, encoder_out, decoder_out, logit_lengths, target_lengths,
                         activation=None, dtype=np.float64):
    """Gradient of pack_joiner by the chain rule: the incoming gradient of a row,
    times 1 - tanh^2 for "tanh" (times [s > 0] for "relu"), is added to its encoder frame and to its decoder
    position; padding receives zero.  Returns (grad_enc, grad_dec, abs_enc, abs_dec):
    the last two are the same sums over the absolute values of the incoming
    gradient, the scale of the rounding error of a float32 evaluation (of the
    summation in any order, and of 1 - tanh^2 where tanh is close to 1)."""
    enc = np.asarray(encoder_out, dtype=dtype)
    dec = np.asarray(decoder_out, dtype=dtype)
    g = np.asarray(grad_out, dtype=dtype)
    ge, gd = np.zeros_like(enc), np.zeros_like(dec)
    ae, ad = np.zeros_like(enc), np.zeros_like(dec)
    D = enc.shape[2]
    r = 0
    for i in range(enc.shape[0]):
        T, U1 = int(logit_lengths[i]), int(target_lengths[i]) + 1
        gi = g[r:r + T * U1].reshape(T, U1, D)
        ae[i, :T] = np.abs(gi).sum(1)
        ad[i, :U1] = np.abs(gi).sum(0)
        if activation == "tanh":
            a = np.tanh(enc[i, :T, None, :] + dec[i, None, :U1, :])
            gi = gi * (1.0 - a * a)
        elif activation == "relu":
            gi = gi * ((enc[i, :T, None, :] + dec[i, None, :U1, :]) > 0)
        ge[i, :T] = gi.sum(1)
        gd[i, :U1] = gi.sum(0)
        r += T * U1
    return ge, gd, ae, ad


# ---------------------------------------------------------------- joiner output projection
def project_joiner(x, weight, bias=None):
    """The caller-side projection in front of the loss (README.md:176-177,
    `logits = linear(activation(x))`): x @ weight.T + bias in float64, and the
    sum of the absolute values of the terms of every entry (the scale of the rounding
    error of a float32 accumulation in any order).  The per-row denominators of the
    result are log_sum_exp's, as for any logits (cpu.cc:770)."""
    x = np.asarray(x, dtype=np.float64)
    w = np.asarray(weight, dtype=np.float64)
    out = x @ w.T
    mag = np.abs(x) @ np.abs(w).T
    if bias is not None:
        b = np.asarray(bias, dtype=np.float64)
        out = out + b[None, :]
        mag = mag + np.abs(b)[None, :]
    return out, mag


def project_joiner_weight_grad(grad_logits, x):
    """Backward of that projection in its parameters, as autograd's Linear forms it
    behind README.md:176-177: grad_weight = grad_logits^T x (V, D) and grad_bias = the
    column sums of grad_logits (V), in float64, each with the sum of the absolute values
    of its terms (the scale of the rounding error of a float32 accumulation in any
    order)."""
    g = np.asarray(grad_logits, dtype=np.float64)
    x = np.asarray(x, dtype=np.float64)
    gw = g.T @ x
    gw_mag = np.abs(g).T @ np.abs(x)
    return gw, gw_mag, g.sum(0), np.abs(g).sum(0)
