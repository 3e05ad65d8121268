"""ctypes binding of libot_transducer.so for the tests (device pointers come
from torch tensors; torch is only used for memory and streams here)."""
import ctypes
import os

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_PATH = os.environ.get(
    "OT_TRANSDUCER_LIB", os.path.join(ROOT, "optimized_transducer_amd", "libot_transducer.so"))
HEADER = os.path.join(ROOT, "include", "ot_transducer.h")


class BatchStatus(ctypes.Structure):
    _fields_ = [("sum_tu", ctypes.c_int64), ("targets_max", ctypes.c_int32),
                ("targets_min", ctypes.c_int32), ("target_len_max", ctypes.c_int32),
                ("target_len_min", ctypes.c_int32), ("logit_len_max", ctypes.c_int32),
                ("logit_len_min", ctypes.c_int32)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = ctypes.CDLL(LIB_PATH)
        _lib.ot_workspace_bytes.restype = ctypes.c_size_t
        _lib.ot_gradient_scratch_bytes.restype = ctypes.c_size_t
        _lib.ot_error_string.restype = ctypes.c_char_p
    return _lib


def ptr(t):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def check(rc):
    if rc != 0:
        raise RuntimeError("ot error %d: %s" % (rc, lib().ot_error_string(rc).decode()))


def row_splits(T, U, targets):
    N = T.numel()
    splits = torch.empty(N + 1, dtype=torch.int32, device=T.device)
    status = torch.zeros(ctypes.sizeof(BatchStatus), dtype=torch.uint8, device=T.device)
    cols = targets.shape[1]
    check(lib().ot_row_splits(ptr(T), ptr(U), ptr(targets if cols else None), ctypes.c_int32(N),
                              ctypes.c_int32(cols), ptr(splits), ptr(None), ptr(status), stream()))
    st = BatchStatus.from_buffer_copy(status.cpu().numpy().tobytes())
    return splits, st


def row_ids(splits, rows):
    out = torch.empty(rows, dtype=torch.int32, device=splits.device)
    check(lib().ot_row_ids(ptr(splits), ctypes.c_int32(splits.numel() - 1), ctypes.c_int64(rows),
                           ptr(out), stream()))
    return out


def log_probs(logits, targets, U, splits, blank, from_log_softmax):
    rows, V = logits.shape
    den = None if from_log_softmax else torch.empty(rows, dtype=torch.float32, device=logits.device)
    lp = torch.full((rows, 2), float("nan"), dtype=torch.float32, device=logits.device)
    cols = targets.shape[1]
    check(lib().ot_log_probs(ptr(logits), ptr(targets if cols else None), ptr(U), ptr(splits),
                             ctypes.c_int32(U.numel()), ctypes.c_int32(cols),
                             ctypes.c_int64(rows), ctypes.c_int32(V), ctypes.c_int32(blank),
                             ctypes.c_int32(int(from_log_softmax)), ptr(den), ptr(lp), stream()))
    return den, lp


def alpha_beta(lp, T, U, splits, max_u1, one_sym_per_frame):
    rows, N = lp.shape[0], T.numel()
    dev = lp.device
    alpha = torch.full((rows,), float("nan"), dtype=torch.float32, device=dev)
    beta = torch.full((rows,), float("nan"), dtype=torch.float32, device=dev)
    sa = torch.full((N,), float("nan"), dtype=torch.float32, device=dev)
    sb = torch.full((N,), float("nan"), dtype=torch.float32, device=dev)
    check(lib().ot_alpha_beta(ptr(lp), ptr(T), ptr(U), ptr(splits), ctypes.c_int32(N),
                              ctypes.c_int32(max_u1), ctypes.c_int32(int(one_sym_per_frame)),
                              ptr(alpha), ptr(beta), ptr(sa), ptr(sb), stream()))
    return alpha, beta, sa, sb


def alpha_beta_guarded(lp, T, U, splits, max_u1, one_sym_per_frame, rows):
    """ot_alpha_beta_guarded: `rows` is what the caller believes the batch adds up to."""
    N = T.numel()
    dev = lp.device
    alpha = torch.full((lp.shape[0],), float("nan"), dtype=torch.float32, device=dev)
    beta = torch.full((lp.shape[0],), float("nan"), dtype=torch.float32, device=dev)
    sa = torch.full((N,), float("nan"), dtype=torch.float32, device=dev)
    sb = torch.full((N,), float("nan"), dtype=torch.float32, device=dev)
    check(lib().ot_alpha_beta_guarded(ptr(lp), ptr(T), ptr(U), ptr(splits), ctypes.c_int32(N),
                                      ctypes.c_int32(max_u1), ctypes.c_int32(int(one_sym_per_frame)),
                                      ctypes.c_int64(rows), ptr(alpha), ptr(beta), ptr(sa), ptr(sb),
                                      stream()))
    return alpha, beta, sa, sb


def gradient(logits, lp, den, alpha, beta, targets, T, U, splits, blank, from_log_softmax,
             one_sym_per_frame, grad_scale=1.0, grad=None, device_factor=None):
    """ot_gradient; with device_factor (a one-element device tensor) the two launches
    ot_row_coefficients + ot_gradient_apply_device_factor instead."""
    rows, V = logits.shape
    if grad is None:
        grad = torch.full((rows, V), float("nan"), dtype=torch.float32, device=logits.device)
    cols = targets.shape[1]
    scratch = torch.empty(lib().ot_gradient_scratch_bytes(ctypes.c_int64(rows)), dtype=torch.uint8,
                          device=logits.device)
    if device_factor is not None:
        check(lib().ot_row_coefficients(
            ptr(lp), ptr(den), ptr(alpha), ptr(beta), ptr(targets if cols else None), ptr(T), ptr(U),
            ptr(splits), ctypes.c_int32(T.numel()), ctypes.c_int32(cols), ctypes.c_int64(rows),
            ctypes.c_int32(blank), ctypes.c_int32(int(from_log_softmax)),
            ctypes.c_int32(int(one_sym_per_frame)), ctypes.c_float(grad_scale), ptr(scratch),
            stream()))
        check(lib().ot_gradient_apply_device_factor(
            ptr(logits), ptr(scratch), ctypes.c_int64(rows), ctypes.c_int32(V),
            ctypes.c_int32(int(from_log_softmax)), ctypes.c_float(grad_scale), ptr(device_factor),
            ptr(grad), stream()))
        return grad
    check(lib().ot_gradient(ptr(logits), ptr(lp), ptr(den), ptr(alpha), ptr(beta),
                            ptr(targets if cols else None), ptr(T), ptr(U), ptr(splits),
                            ctypes.c_int32(T.numel()), ctypes.c_int32(cols), ctypes.c_int64(rows),
                            ctypes.c_int32(V), ctypes.c_int32(blank),
                            ctypes.c_int32(int(from_log_softmax)),
                            ctypes.c_int32(int(one_sym_per_frame)), ctypes.c_float(grad_scale),
                            ptr(scratch), ptr(grad), stream()))
    return grad


def transducer_loss(logits, targets, T, U, blank, from_log_softmax, one_sym_per_frame, max_u1,
                    grad_scale=1.0, grad="new"):
    """Whole path through ot_transducer_loss.  grad: "new", "inplace" or None."""
    rows, V = logits.shape
    N = T.numel()
    dev = logits.device
    nbytes = lib().ot_workspace_bytes(ctypes.c_int32(N), ctypes.c_int64(rows))
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    scores = torch.full((N,), float("nan"), dtype=torch.float32, device=dev)
    status = torch.zeros(ctypes.sizeof(BatchStatus), dtype=torch.uint8, device=dev)
    if grad == "new":
        g = torch.full((rows, V), float("nan"), dtype=torch.float32, device=dev)
    elif grad == "inplace":
        g = logits
    else:
        g = None
    cols = targets.shape[1]
    check(lib().ot_transducer_loss(
        ptr(logits), ptr(targets if cols else None), ptr(T), ptr(U), ctypes.c_int32(N),
        ctypes.c_int32(cols), ctypes.c_int64(rows), ctypes.c_int32(V), ctypes.c_int32(blank),
        ctypes.c_int32(int(from_log_softmax)), ctypes.c_int32(int(one_sym_per_frame)),
        ctypes.c_int32(max_u1), ctypes.c_float(grad_scale), ptr(ws), ctypes.c_size_t(nbytes),
        ptr(scores), ptr(g), ptr(status), stream()))
    st = BatchStatus.from_buffer_copy(status.cpu().numpy().tobytes())
    return scores, g, st


def scale_by_device_scalar(x, factor):
    check(lib().ot_scale_by_device_scalar(ptr(x), ctypes.c_int64(x.numel()), ptr(factor), stream()))


def copy_floats(src, dst):
    check(lib().ot_copy_floats(ptr(src), ptr(dst), ctypes.c_int64(src.numel()), stream()))


def joiner_pack(enc, dec, T, U, splits, rows, activation):
    N, t_stride, D = enc.shape
    out = torch.full((rows, D), float("nan"), dtype=torch.float32, device=enc.device)
    check(lib().ot_joiner_pack(ptr(enc), ptr(dec), ptr(T), ptr(U), ptr(splits), ctypes.c_int32(N),
                               ctypes.c_int32(t_stride), ctypes.c_int32(dec.shape[1]),
                               ctypes.c_int32(D), ctypes.c_int32(activation), ptr(out), stream()))
    return out


def joiner_unpack_grad(grad_out, enc, dec, T, U, splits, activation):
    N, t_stride, D = enc.shape
    u_stride = dec.shape[1]
    L = lib()
    L.ot_joiner_unpack_workspace_bytes.restype = ctypes.c_size_t
    nbytes = L.ot_joiner_unpack_workspace_bytes(ctypes.c_int32(N), ctypes.c_int32(t_stride),
                                                ctypes.c_int32(u_stride), ctypes.c_int32(D))
    ws = torch.empty(nbytes, dtype=torch.uint8, device=enc.device)
    ge = torch.full_like(enc, float("nan"))
    gd = torch.full_like(dec, float("nan"))
    if grad_out.dtype == torch.float32:
        check(L.ot_joiner_unpack_grad(ptr(grad_out), ptr(enc), ptr(dec), ptr(T), ptr(U), ptr(splits),
                                      ctypes.c_int32(N), ctypes.c_int32(t_stride),
                                      ctypes.c_int32(u_stride), ctypes.c_int32(D),
                                      ctypes.c_int32(activation), ptr(ws), ctypes.c_size_t(nbytes),
                                      ptr(ge), ptr(gd), stream()))
    else:  # a 16-bit incoming gradient
        code = {torch.float16: 1, torch.bfloat16: 2}[grad_out.dtype]
        check(L.ot_joiner_unpack_grad_from(ptr(grad_out), ctypes.c_int32(code), ptr(enc), ptr(dec),
                                           ptr(T), ptr(U), ptr(splits), ctypes.c_int32(N),
                                           ctypes.c_int32(t_stride), ctypes.c_int32(u_stride),
                                           ctypes.c_int32(D), ctypes.c_int32(activation), ptr(ws),
                                           ctypes.c_size_t(nbytes), ptr(ge), ptr(gd), stream()))
    return ge, gd


def row_coefficients(lp, den, alpha, beta, targets, T, U, splits, blank, from_log_softmax,
                     one_sym_per_frame, grad_scale=1.0, scores=None, loss_scale=1.0):
    """ot_row_coefficients, or ot_row_coefficients_loss when `scores` is given.
    Returns (row scratch as bytes, loss or None)."""
    rows = alpha.numel()
    cols = targets.shape[1]
    scratch = torch.zeros(lib().ot_gradient_scratch_bytes(ctypes.c_int64(rows)), dtype=torch.uint8,
                          device=alpha.device)
    head = (ptr(lp), ptr(den), ptr(alpha), ptr(beta), ptr(targets if cols else None), ptr(T), ptr(U),
            ptr(splits), ctypes.c_int32(T.numel()), ctypes.c_int32(cols), ctypes.c_int64(rows),
            ctypes.c_int32(blank), ctypes.c_int32(int(from_log_softmax)),
            ctypes.c_int32(int(one_sym_per_frame)), ctypes.c_float(grad_scale), ptr(scratch))
    if scores is None:
        check(lib().ot_row_coefficients(*head, stream()))
        return scratch, None
    loss = torch.full((1,), float("nan"), dtype=torch.float32, device=alpha.device)
    check(lib().ot_row_coefficients_loss(*head, ptr(scores), ctypes.c_float(loss_scale), ptr(loss),
                                         stream()))
    return scratch, loss


def negative_sum(scores, scale):
    loss = torch.full((1,), float("nan"), dtype=torch.float32, device=scores.device)
    check(lib().ot_negative_sum(ptr(scores), ctypes.c_int32(scores.numel()), ctypes.c_float(scale),
                                ptr(loss), stream()))
    return loss


DTYPE = {torch.float16: 1, torch.bfloat16: 2}


def log_probs_half(logits, targets, U, splits, blank, from_log_softmax):
    rows, V = logits.shape
    den = torch.full((rows,), float("nan"), dtype=torch.float32, device=logits.device)
    lp = torch.full((rows, 2), float("nan"), dtype=torch.float32, device=logits.device)
    cols = targets.shape[1]
    check(lib().ot_log_probs_half(ptr(logits), ctypes.c_int32(DTYPE[logits.dtype]),
                                  ptr(targets if cols else None), ptr(U), ptr(splits),
                                  ctypes.c_int32(U.numel()), ctypes.c_int32(cols),
                                  ctypes.c_int64(rows), ctypes.c_int32(V), ctypes.c_int32(blank),
                                  ctypes.c_int32(int(from_log_softmax)), ptr(den), ptr(lp), stream()))
    return den, lp


def gradient_half(logits, lp, den, alpha, beta, targets, T, U, splits, blank, from_log_softmax,
                  one_sym_per_frame, grad_scale=1.0, grad=None, device_factor=None):
    """ot_row_coefficients (float32) + ot_gradient_apply_half."""
    rows, V = logits.shape
    if grad is None:
        grad = torch.full((rows, V), float("nan"), dtype=logits.dtype, device=logits.device)
    cols = targets.shape[1]
    scratch = torch.empty(lib().ot_gradient_scratch_bytes(ctypes.c_int64(rows)), dtype=torch.uint8,
                          device=logits.device)
    check(lib().ot_row_coefficients(
        ptr(lp), ptr(den), ptr(alpha), ptr(beta), ptr(targets if cols else None), ptr(T), ptr(U),
        ptr(splits), ctypes.c_int32(T.numel()), ctypes.c_int32(cols), ctypes.c_int64(rows),
        ctypes.c_int32(blank), ctypes.c_int32(int(from_log_softmax)),
        ctypes.c_int32(int(one_sym_per_frame)), ctypes.c_float(grad_scale), ptr(scratch), stream()))
    check(lib().ot_gradient_apply_half(
        ptr(logits), ctypes.c_int32(DTYPE[logits.dtype]), ptr(scratch), ctypes.c_int64(rows),
        ctypes.c_int32(V), ctypes.c_int32(int(from_log_softmax)), ctypes.c_float(grad_scale),
        ptr(device_factor), ptr(grad), stream()))
    return grad


ANY_DTYPE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


def joiner_project(x, weight, bias, out_dtype, logits=None, workspace=False):
    """ot_joiner_project, or with workspace=True ot_joiner_project_ws on a workspace full of
    NaN patterns."""
    rows, D = x.shape
    V = weight.shape[0]
    if logits is None:
        logits = torch.full((rows, V), float("nan"), dtype=out_dtype, device=x.device)
    den = torch.full((rows,), float("nan"), dtype=torch.float32, device=x.device)
    if workspace:
        L = lib()
        L.ot_joiner_project_workspace_bytes.restype = ctypes.c_size_t
        nbytes = L.ot_joiner_project_workspace_bytes(ctypes.c_int64(rows), ctypes.c_int32(V))
        ws = torch.full((max(nbytes, 4),), 0xFF, dtype=torch.uint8, device=x.device)
        check(L.ot_joiner_project_ws(ptr(x), ptr(weight), ptr(bias), ctypes.c_int32(DTYPE[x.dtype]),
                                     ctypes.c_int64(rows), ctypes.c_int32(D), ctypes.c_int32(V),
                                     ptr(logits), ctypes.c_int32(ANY_DTYPE[out_dtype]), ptr(den),
                                     ptr(ws if nbytes else None), ctypes.c_size_t(nbytes), stream()))
        return logits, den
    check(lib().ot_joiner_project(ptr(x), ptr(weight), ptr(bias), ctypes.c_int32(DTYPE[x.dtype]),
                                  ctypes.c_int64(rows), ctypes.c_int32(D), ctypes.c_int32(V),
                                  ptr(logits), ctypes.c_int32(ANY_DTYPE[out_dtype]), ptr(den),
                                  stream()))
    return logits, den


def joiner_weight_grad(grad_logits, x, want_bias=True, workspace_fill=None):
    """(grad_weight (V, D) of x's dtype, grad_bias (V) float32 or None) through
    ot_joiner_weight_grad; workspace_fill: a byte value the workspace is filled with before
    the call (its contents must not matter)."""
    rows, V = grad_logits.shape
    D = x.shape[1]
    L = lib()
    L.ot_joiner_weight_grad_workspace_bytes.restype = ctypes.c_size_t
    nbytes = L.ot_joiner_weight_grad_workspace_bytes(ctypes.c_int64(rows), ctypes.c_int32(V), ctypes.c_int32(D))
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=x.device)
    if workspace_fill is not None:
        ws.fill_(workspace_fill)
    gw = torch.full((V, D), float("nan"), dtype=x.dtype, device=x.device)
    gb = torch.full((V,), float("nan"), dtype=torch.float32, device=x.device) if want_bias else None
    check(L.ot_joiner_weight_grad(ptr(grad_logits), ptr(x), ctypes.c_int32(DTYPE[x.dtype]),
                                  ctypes.c_int64(rows), ctypes.c_int32(V), ctypes.c_int32(D), ptr(ws),
                                  ctypes.c_size_t(nbytes), ptr(gw), ptr(gb), stream()))
    return gw, gb


def log_probs_given_den(logits, den, targets, U, splits, blank):
    rows, V = logits.shape
    lp = torch.full((rows, 2), float("nan"), dtype=torch.float32, device=logits.device)
    cols = targets.shape[1]
    check(lib().ot_log_probs_given_den(ptr(logits), ctypes.c_int32(ANY_DTYPE[logits.dtype]), ptr(den),
                                       ptr(targets if cols else None), ptr(U), ptr(splits),
                                       ctypes.c_int32(U.numel()), ctypes.c_int32(cols),
                                       ctypes.c_int64(rows), ctypes.c_int32(V), ctypes.c_int32(blank),
                                       ptr(lp), stream()))
    return lp


def joiner_pack_half(enc, dec, T, U, splits, rows, activation, out_dtype):
    N, Tm, D = enc.shape
    out = torch.full((rows, D), float("nan"), dtype=out_dtype, device=enc.device)
    check(lib().ot_joiner_pack_half(ptr(enc), ptr(dec), ptr(T), ptr(U), ptr(splits), ctypes.c_int32(N),
                                    ctypes.c_int32(Tm), ctypes.c_int32(dec.shape[1]), ctypes.c_int32(D),
                                    ctypes.c_int32(activation), ctypes.c_int32(DTYPE[out_dtype]), ptr(out),
                                    stream()))
    return out
