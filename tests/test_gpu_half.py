"""Half-precision logits (float16, bfloat16): an addition to the reference, which
takes float32 only (transducer-loss.cc:33).

The oracle is the CPU oracle on the logits converted to float32 (the conversion is
exact): the kernels do float32 arithmetic on exactly those values.  Denominators
and log-probabilities are float32 and meet the float32 tolerance; gradients are
rounded to the logits' dtype, so they are compared with the oracle's float32
gradient to within one unit in the last place of that dtype (2^-11 / 2^-8
relative) plus the float32 tolerance."""
import numpy as np
import pytest
import torch

import cabi
import helpers
from helpers import ATOL, RTOL
from oracle import oracle

pytestmark = pytest.mark.gpu

DTYPES = [torch.float16, torch.bfloat16]
ULP = {torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8}


def _dev(a, device):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def _half_batch(rng, N, tmax, umax, V, dtype, device, osf=False, scale=1.0):
    T, U, tg, x = helpers.random_batch(rng, N, tmax, umax, V, one_sym_per_frame=osf)
    tg = np.where(tg == 0, 1 % V, tg).astype(np.int32)
    xh = (torch.from_numpy(x) * scale).to(dtype)          # the logits the kernels see
    return T, U, tg, xh.to(device), xh.float().numpy()    # and their exact float32 values


# V: 500 -> 4 elements per access, 512 -> 8, 6 -> 2, 37 -> 1; 2048 / 5000 -> 4 chunks / any length;
# 8, 100, 1024: the other lane groupings of the flat denominator kernel
@pytest.mark.parametrize("dtype", DTYPES, ids=["f16", "bf16"])
@pytest.mark.parametrize("V", [500, 512, 6, 37, 2048, 5000, 1030, 8, 100, 1024])
def test_log_probs_and_gradient_kernels(V, dtype, device):
    rng = np.random.default_rng(V)
    T, U, tg, xh, x32 = _half_batch(rng, 5, 12, 6, V, dtype, device, scale=2.0)
    dT, dU, dtg = _dev(T, device), _dev(U, device), _dev(tg, device)
    splits, _ = cabi.row_splits(dT, dU, dtg)
    den, lp = cabi.log_probs_half(xh, dtg, dU, splits, 0, False)
    wden = oracle.logsumexp(x32)
    gden = den.cpu().numpy()
    ulp = np.spacing(np.maximum(np.abs(wden), np.abs(x32).max(1)).astype(np.float32))
    assert (np.abs(gden - wden) <= 4 * ulp).all(), (np.abs(gden - wden) / ulp).max()
    wlp = oracle.log_probs(x32, wden, tg, T, U, 0)
    m = ~np.isnan(wlp)
    got = lp.cpu().numpy()
    assert np.allclose(got[m], wlp[m], rtol=RTOL, atol=ATOL) and np.isneginf(got[~m]).all()
    # logits that start 2 bytes into an allocation take the narrow-access kernel
    flat = torch.zeros(xh.numel() + 1, dtype=dtype, device=device)
    view = flat[1:].view(xh.shape)
    view.copy_(xh)
    den_v, lp_v = cabi.log_probs_half(view, dtg, dU, splits, 0, False)
    assert (np.abs(den_v.cpu().numpy() - wden) <= 4 * ulp).all()
    assert np.allclose(lp_v.cpu().numpy()[m], wlp[m], rtol=RTOL, atol=ATOL)
    # log-softmax input: pure gather, bit exact
    xl = torch.log_softmax(xh.float(), 1).to(dtype)
    _, lp2 = cabi.log_probs_half(xl, dtg, dU, splits, 0, True)
    want = oracle.log_probs(xl.float().cpu().numpy(), None, tg, T, U, 0)
    got = lp2.cpu().numpy()
    assert (got[m] == want[m]).all() and np.isneginf(got[~m]).all()

    # gradient given the oracle's lattice
    for fls, xin in ((False, xh), (True, xl)):
        xin32 = xin.float().cpu().numpy()
        s, g, parts = helpers.oracle_full(xin32, tg, T, U, 0, fls, False)
        ninf = lambda v: np.where(np.isnan(v), -np.inf, v).astype(np.float32)  # noqa: E731
        args = (xin, _dev(ninf(parts["lp"]), device), None if fls else _dev(parts["den"], device),
                _dev(ninf(parts["alpha"]), device), _dev(ninf(parts["beta"]), device), dtg, dT, dU,
                splits, 0, fls, False)
        got = cabi.gradient_half(*args).float().cpu().numpy()
        assert got.shape == g.shape and not np.isnan(got).any()
        assert (np.abs(got - g) <= ULP[dtype] * np.abs(g) + 1e-6).all(), np.abs(got - g).max()
        four = torch.full((1,), 4.0, device=device)
        got8 = cabi.gradient_half(*args, grad_scale=2.0, device_factor=four).float().cpu().numpy()
        assert (np.abs(got8 - 8 * g) <= 8 * (ULP[dtype] * np.abs(g) + 1e-6)).all()
        if not fls:  # in place
            buf = xin.clone()
            out = cabi.gradient_half(buf, *args[1:], grad=buf)
            assert out.data_ptr() == buf.data_ptr() and torch.equal(buf.float().cpu(), torch.from_numpy(got))
            # a buffer that starts 2 bytes into an allocation: narrow accesses, same bits
            flat = torch.zeros(xin.numel() + 1, dtype=dtype, device=device)
            view = flat[1:].view(xin.shape)
            view.copy_(xin)
            cabi.gradient_half(view, *args[1:], grad=view)
            assert torch.equal(view.float().cpu(), torch.from_numpy(got)) and flat[0].item() == 0


@pytest.mark.parametrize("dtype", DTYPES, ids=["f16", "bf16"])
@pytest.mark.parametrize("V,rows_odd", [(20, True), (20, False), (6, True), (500, True), (9, True)])
def test_gradient_kernel_tail_of_the_array(V, rows_odd, dtype, device):
    # 16-byte accesses cover the array up to a multiple of 8 elements; the rest is done apart
    T = np.array([3, 2 if rows_odd else 3], np.int32)
    U = np.array([2, 1], np.int32)          # 9 + 4 = 13 rows, or 9 + 6 = 15 rows
    if not rows_odd:
        T[1], U[1] = 2, 2                   # 9 + 6 = 15 rows is odd too: make it 3*3 + 1*... even
        T[0] = 2                            # 6 + 6 = 12 rows
    rng = np.random.default_rng(V)
    rows = int((T * (U + 1)).sum())
    tg = rng.integers(1, V, size=(2, int(U.max()))).astype(np.int32)
    xh = torch.from_numpy(rng.standard_normal((rows, V)).astype(np.float32)).to(dtype)
    x32 = xh.float().numpy()
    s, g, parts = helpers.oracle_full(x32, tg, T, U, 0, False, False)
    ninf = lambda v: np.where(np.isnan(v), -np.inf, v).astype(np.float32)  # noqa: E731
    dT, dU, dtg = _dev(T, device), _dev(U, device), _dev(tg, device)
    splits, _ = cabi.row_splits(dT, dU, dtg)
    buf = xh.to(device)
    guard = torch.full((64,), 7.0, dtype=dtype, device=device)  # allocated right after, must survive
    cabi.gradient_half(buf, _dev(ninf(parts["lp"]), device), _dev(parts["den"], device),
                       _dev(ninf(parts["alpha"]), device), _dev(ninf(parts["beta"]), device), dtg, dT,
                       dU, splits, 0, False, False, grad=buf)
    got = buf.float().cpu().numpy()
    assert (np.abs(got - g) <= ULP[dtype] * np.abs(g) + 1e-6).all(), np.abs(got - g).max()
    assert (guard == 7.0).all()


@pytest.mark.parametrize("dtype", DTYPES, ids=["f16", "bf16"])
@pytest.mark.parametrize("fls,osf", [(False, False), (False, True), (True, False), (True, True)])
def test_python_entry_point_with_half_logits(fls, osf, dtype, device):
    import optimized_transducer_amd as ot
    rng = np.random.default_rng(17)
    T, U, tg, xh, x32 = _half_batch(rng, 6, 25, 70, 40, dtype, device, osf=osf)
    if fls:
        xh = torch.log_softmax(xh.float(), 1).to(dtype)
        x32 = xh.float().cpu().numpy()
    dT, dU, dtg = _dev(T, device), _dev(U, device), _dev(tg, device)
    want_loss, want = oracle.transducer_loss(x32.copy(), tg, T, U, 0, fls, osf, "mean", loss_grad=2.0)
    _, _, noise = helpers.oracle_tolerance(x32, tg, T, U, 0, fls, osf, scale=2.0 / len(T))
    for defer in (False, True):
        logits = xh.clone().requires_grad_(True)
        loss = ot.transducer_loss(logits, dtg, dT, dU, 0, fls, one_sym_per_frame=osf,
                                  reduction="mean", defer_gradient=defer)
        assert loss.dtype == torch.float32 and loss.dim() == 0
        (loss * 2.0).backward()
        assert np.allclose(loss.item(), want_loss, rtol=RTOL, atol=ATOL)
        assert logits.grad.dtype == dtype and logits.grad.shape == logits.shape
        got = logits.grad.float().cpu().numpy()
        assert (np.abs(got - want) <= 2 * ULP[dtype] * np.abs(want) + noise).all(), \
            np.abs(got - want).max()
        if not fls:
            assert logits.grad.data_ptr() == logits.data_ptr()  # in place, as for float32
    # the same call on the float32 values agrees in the loss to float32 rounding
    l32 = ot.transducer_loss(_dev(x32, device), dtg, dT, dU, 0, fls, one_sym_per_frame=osf)
    assert abs(l32.item() - loss.item()) <= 1e-5 * abs(loss.item()) + 1e-5


def test_other_dtypes_are_still_refused(device):
    import optimized_transducer_amd as ot
    rng = np.random.default_rng(3)
    T, U, tg, x = helpers.random_batch(rng, 2, 5, 3, 8)
    with pytest.raises(RuntimeError, match="Float"):
        ot.transducer_loss(_dev(x, device).double(), _dev(tg, device), _dev(T, device), _dev(U, device),
                           0, False)
