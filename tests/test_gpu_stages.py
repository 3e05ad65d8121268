"""GPU parity, stage by stage, through the C ABI (ctypes on libot_transducer.so).

Each kernel gets the oracle's output of the previous stage as its input, so
that the north-star tolerance (rel 1e-5 / abs 1e-5, bit-exact integers) can be
asserted per stage without the fp32 cancellation noise that an end-to-end
comparison of two fp32 implementations carries (that comparison lives in
test_gpu_end_to_end.py).
"""
import ctypes

import numpy as np
import pytest
import torch

import cabi
import helpers
import workloads
from helpers import ATOL, RTOL
from oracle import oracle

pytestmark = pytest.mark.gpu


def _dev(a, device):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def _cases():
    rng = np.random.default_rng(1234)
    out = []
    for w in (workloads.tiny(), workloads.tiny(one_sym_per_frame=True)):
        out.append((w.name + ("_mod" if w.one_sym_per_frame else ""), w.logit_lengths,
                    w.target_lengths, w.targets, w.logits_numpy(), 0, w.one_sym_per_frame))
    # ragged, U = 0 and T = 1 utterances, blank != 0, V odd (scalar loads), V = 3
    for name, N, tmax, umax, V, blank, osf in [
            ("ragged_V37", 9, 40, 20, 37, 5, False), ("ragged_V37_mod", 9, 40, 20, 37, 5, True),
            ("V3", 6, 9, 5, 3, 0, False), ("V3_mod", 6, 9, 5, 3, 0, True),
            ("two_waves_V64", 3, 90, 100, 64, 1, False), ("two_waves_V64_mod", 3, 120, 100, 64, 1, True),
            ("five_waves_V8", 2, 40, 300, 8, 0, False), ("five_waves_V8_mod", 2, 330, 300, 8, 0, True),
            ("many_utts_V16", 300, 6, 4, 16, 0, False),
            # beyond the 1024 utterances up to which a workgroup finds its utterances by a
            # wave-parallel count
            ("thousands_of_utts_V16", 3000, 5, 3, 16, 2, False),
            ("thousands_of_utts_V12_mod", 2500, 6, 3, 12, 0, True),
            ("V1000", 4, 12, 6, 1000, 999, False), ("V5000", 2, 7, 4, 5000, 0, False),
            ("V5004_mod", 2, 7, 4, 5004, 17, True), ("V2049", 2, 5, 3, 2049, 0, False)]:
        T, U, tg, x = helpers.random_batch(rng, N, tmax, umax, V, one_sym_per_frame=osf)
        if not osf:
            T[0], U[0] = 1, 0          # single-cell lattice
            if N > 1:
                T[1], U[1] = 1, min(int(U.max()), 3)  # one frame, several symbols
            rows = int((T.astype(np.int64) * (U + 1)).sum())
            x = rng.standard_normal((rows, V)).astype(np.float32)
            tg = np.ascontiguousarray(tg[:, :int(U.max())])
        tg = np.where(tg == blank, (blank + 1) % V, tg).astype(np.int32)
        out.append((name, T, U, tg, x, blank, osf))
    return out


CASES = _cases()


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_row_offsets_and_batch_facts_are_bit_exact(case, device):
    _, T, U, tg, x, blank, osf = case
    splits, st = cabi.row_splits(_dev(T, device), _dev(U, device), _dev(tg, device))
    want, total = oracle.row_splits(T, U)
    got = splits.cpu().numpy()
    assert got.dtype == np.int32 and (got == want).all()
    assert st.sum_tu == total == x.shape[0]
    assert st.targets_max == tg.max() and st.targets_min == tg.min()
    assert st.target_len_max == U.max() and st.target_len_min == U.min()
    assert st.logit_len_max == T.max() and st.logit_len_min == T.min()
    ids = cabi.row_ids(splits, x.shape[0]).cpu().numpy()
    assert (ids == oracle.row_ids(want)).all()


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_log_probs_kernel(case, device):
    _, T, U, tg, x, blank, osf = case
    dT, dU, dtg, dx = _dev(T, device), _dev(U, device), _dev(tg, device), _dev(x, device)
    splits, _ = cabi.row_splits(dT, dU, dtg)
    # log-softmax input: pure gather, so target indexing is checked bit for bit
    xl = helpers.log_softmax32(x)
    _, lp = cabi.log_probs(_dev(xl, device), dtg, dU, splits, blank, True)
    want = oracle.log_probs(xl, None, tg, T, U, blank)
    got = lp.cpu().numpy()
    m = ~np.isnan(want)
    assert (got[m] == want[m]).all()
    assert np.isneginf(got[~m]).all()  # undefined in the reference, -inf here
    # logits input: fused log-sum-exp + gather
    den, lp = cabi.log_probs(dx, dtg, dU, splits, blank, False)
    wden = oracle.logsumexp(x)
    gden = den.cpu().numpy()
    # hardware 2^x (1 ulp) on a product rounded once: a few ulp for a row of a few
    # comparable terms, about one for a long row where the term errors average out
    ulp = np.spacing(np.maximum(np.abs(wden), np.abs(x).max(1)).astype(np.float32))
    d64 = oracle.logsumexp(x, dtype=np.float64)
    k = 2 if x.shape[1] >= 64 else 4
    assert (np.abs(gden - wden) <= k * ulp).all(), (np.abs(gden - wden) / ulp).max()
    assert (np.abs(gden - d64) <= k * ulp).all(), (np.abs(gden - d64) / ulp).max()
    wlp = oracle.log_probs(x, wden, tg, T, U, blank)
    got = lp.cpu().numpy()
    assert np.allclose(got[m], wlp[m], rtol=RTOL, atol=ATOL)
    assert np.isneginf(got[~m]).all()


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_lattice_kernel_given_oracle_log_probs(case, device):
    _, T, U, tg, x, blank, osf = case
    s, _, parts = helpers.oracle_full(x, tg, T, U, blank, False, osf)
    lp = np.where(np.isnan(parts["lp"]), -np.inf, parts["lp"]).astype(np.float32)
    dT, dU = _dev(T, device), _dev(U, device)
    splits, _ = cabi.row_splits(dT, dU, _dev(tg, device))
    a, b, sa, sb = cabi.alpha_beta(_dev(lp, device), dT, dU, splits, int(U.max()) + 1, osf)
    a, b, sa, sb = (t.cpu().numpy() for t in (a, b, sa, sb))
    for got, want in ((a, parts["alpha"]), (b, parts["beta"])):
        m = ~np.isnan(want)
        assert np.allclose(got[m], want[m], rtol=RTOL, atol=ATOL), np.abs(got[m] - want[m]).max()
        assert np.isneginf(got[~m]).all()  # outside the band
    assert np.allclose(sa, s, rtol=RTOL, atol=ATOL)
    assert np.allclose(sb, parts["scores_beta"], rtol=RTOL, atol=ATOL)
    # the sweep is deterministic: same bits on a second launch
    a2, b2, _, _ = cabi.alpha_beta(_dev(lp, device), dT, dU, splits, int(U.max()) + 1, osf)
    assert (a2.cpu().numpy() == a).all() and (b2.cpu().numpy() == b).all()


WIDE = [  # (T, U) per utterance: 2..16 waves' worth of columns, mixed with short targets
    ("two_waves", [(50, 127), (9, 64), (20, 5), (1, 100), (70, 65), (33, 126)]),
    ("three_waves", [(50, 130), (9, 191), (20, 5)]),
    ("four_waves", [(300, 200), (7, 255), (64, 64), (1, 250)]),
    ("five_waves", [(40, 300), (3, 319), (100, 0)]),
    ("nine_waves", [(33, 575), (100, 577), (5, 70)]),
    ("ten_waves", [(25, 600), (1, 639), (80, 129)]),
    ("sixteen_waves", [(40, 1023), (3, 700), (17, 1000), (30, 63)]),
    # more columns than a workgroup has threads: tiles of 1024 columns, one after the other
    # (U + 1 = 1500 and 3000; 1024 and 1025 columns sit on the tile boundary)
    ("tiles_1500", [(60, 1499), (40, 1023), (9, 1024), (30, 63), (1, 1200)]),
    ("tiles_3000", [(120, 2999), (35, 2047), (7, 2048), (50, 100)]),
]


@pytest.mark.parametrize("osf", [False, True])
@pytest.mark.parametrize("name,shapes", WIDE, ids=[w[0] for w in WIDE])
def test_lattice_kernel_with_many_waves(name, shapes, osf, device):
    rng = np.random.default_rng(len(name))
    T = np.array([s[0] for s in shapes], np.int32)
    U = np.array([s[1] for s in shapes], np.int32)
    if osf:
        T = np.maximum(T, U + 1 + rng.integers(0, 40, size=len(T))).astype(np.int32)
    rows = int((T.astype(np.int64) * (U + 1)).sum())
    # log-probabilities of a plausible size; lp[., 1] at u == U is never read
    lp = (-rng.random((rows, 2)) * 6 - 0.05).astype(np.float32)
    fn_a = oracle.alpha if not osf else (lambda *a: oracle.alpha(*a, one_sym_per_frame=True))
    fn_b = oracle.beta if not osf else (lambda *a: oracle.beta(*a, one_sym_per_frame=True))
    wa, sa_w = fn_a(lp, T, U)
    wb, sb_w = fn_b(lp, T, U)
    dT, dU = _dev(T, device), _dev(U, device)
    splits, _ = cabi.row_splits(dT, dU, torch.zeros((len(T), 0), dtype=torch.int32, device=device))
    a, b, sa, sb = cabi.alpha_beta(_dev(lp, device), dT, dU, splits, int(U.max()) + 1, osf)
    a, b, sa, sb = (t.cpu().numpy() for t in (a, b, sa, sb))
    for got, want in ((a, wa), (b, wb)):
        m = ~np.isnan(want)
        assert np.allclose(got[m], want[m], rtol=RTOL, atol=ATOL), np.abs(got[m] - want[m]).max()
        assert np.isneginf(got[~m]).all()
    assert np.allclose(sa, sa_w, rtol=RTOL, atol=ATOL) and np.allclose(sb, sb_w, rtol=RTOL, atol=ATOL)
    a2, b2, _, _ = cabi.alpha_beta(_dev(lp, device), dT, dU, splits, int(U.max()) + 1, osf)
    assert (a2.cpu().numpy() == a).all() and (b2.cpu().numpy() == b).all()


@pytest.mark.parametrize("fls", [False, True])
@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_gradient_kernels_given_oracle_lattice(case, fls, device):
    _, T, U, tg, x, blank, osf = case
    xin = helpers.log_softmax32(x) if fls else x
    s, g, parts = helpers.oracle_full(xin, tg, T, U, blank, fls, osf)
    ninf = lambda v: np.where(np.isnan(v), -np.inf, v).astype(np.float32)  # noqa: E731
    dT, dU, dtg, dx = _dev(T, device), _dev(U, device), _dev(tg, device), _dev(xin, device)
    splits, _ = cabi.row_splits(dT, dU, dtg)
    den = None if fls else _dev(parts["den"], device)
    args = (dx, _dev(ninf(parts["lp"]), device), den, _dev(ninf(parts["alpha"]), device),
            _dev(ninf(parts["beta"]), device), dtg, dT, dU, splits, blank, fls, osf)
    got = cabi.gradient(*args).cpu().numpy()
    assert not np.isnan(got).any()
    assert np.allclose(got, g, rtol=RTOL, atol=ATOL), np.abs(got - g).max()
    assert np.abs(got - g).max() < 1e-6  # in fact the stage agrees to an ulp or two
    # folded scale (reduction="mean"): multiplication by 1/N, exact for a power of two
    got4 = cabi.gradient(*args, grad_scale=0.25).cpu().numpy()
    assert (got4 == got * np.float32(0.25)).all()
    # one more factor, read from device memory by the kernel (the upstream gradient of the
    # loss in the deferred mode); powers of two keep the comparison exact
    four = torch.full((1,), 4.0, device=device)
    got2 = cabi.gradient(*args, grad_scale=2.0, device_factor=four).cpu().numpy()
    assert (got2 == got * np.float32(8.0)).all()
    if not fls:
        # in place: the logits buffer itself receives the gradient (cuda.cu:449)
        buf = dx.clone()
        out = cabi.gradient(buf, *args[1:], grad=buf)
        assert out.data_ptr() == buf.data_ptr()
        assert (buf.cpu().numpy() == got).all()


def test_target_equal_to_blank_and_nonfinite_utterance(device):
    # reference branch order when a target equals blank (cpu.cc:514-523), and the
    # zero gradient for an utterance whose likelihood is not finite (kernels.cu:558-563)
    rng = np.random.default_rng(5)
    T = np.array([4, 3, 5], np.int32)
    U = np.array([2, 2, 1], np.int32)
    blank = 1
    tg = np.array([[1, 2], [3, 1], [1, 0]], np.int32)
    rows = int((T * (U + 1)).sum())
    x = rng.standard_normal((rows, 6)).astype(np.float32)
    s, g, parts = helpers.oracle_full(x, tg, T, U, blank, False, False)
    dT, dU, dtg, dx = _dev(T, device), _dev(U, device), _dev(tg, device), _dev(x, device)
    sc, gr, st = cabi.transducer_loss(dx, dtg, dT, dU, blank, False, False, 3, grad="new")
    assert np.allclose(sc.cpu().numpy(), s, rtol=RTOL, atol=ATOL)
    err = np.abs(gr.cpu().numpy() - g)
    assert np.allclose(gr.cpu().numpy(), g, rtol=1e-4, atol=2e-5), (err.max(), err.max(1), sc, s)
    # modified lattice with U > T-1 has no alignment: log-likelihood -inf, gradient 0
    T2 = np.array([2, 6], np.int32)
    U2 = np.array([3, 2], np.int32)
    tg2 = np.array([[2, 3, 4], [2, 3, 0]], np.int32)
    x2 = rng.standard_normal((int((T2 * (U2 + 1)).sum()), 6)).astype(np.float32)
    sc, gr, _ = cabi.transducer_loss(_dev(x2, device), _dev(tg2, device), _dev(T2, device),
                                     _dev(U2, device), blank, False, True, 4, grad="new")
    sc, gr = sc.cpu().numpy(), gr.cpu().numpy()
    assert np.isneginf(sc[0]) and np.isfinite(sc[1])
    assert (gr[:8] == 0).all() and np.abs(gr[8:]).max() > 0
    s2, g2 = oracle.compute_transducer_loss(x2[8:].copy(), tg2[1:, :2], T2[1:], U2[1:], blank,
                                            False, True)
    assert np.allclose(sc[1], s2[0], rtol=RTOL, atol=ATOL)
    assert np.allclose(gr[8:], g2, rtol=1e-4, atol=2e-5)


def test_scale_by_device_scalar(device):
    x = torch.randn(1000003, device=device)
    ref = x.clone()
    one = torch.ones((), device=device)
    cabi.scale_by_device_scalar(x, one)
    assert torch.equal(x, ref)
    three = torch.full((), 3.0, device=device)
    cabi.scale_by_device_scalar(x, three)
    assert torch.equal(x, ref * 3.0)
    y = x[1:]  # 4-byte aligned only
    cabi.scale_by_device_scalar(y, three)
    assert torch.equal(y, ref[1:] * 3.0 * 3.0)


def test_negative_sum(device):
    # loss = -scale * sum(scores) (transducer_loss.py:145-147), fixed order: same bits twice
    rng = np.random.default_rng(8)
    for n in (1, 3, 64, 257, 5000):
        x = (-rng.random(n) * 3000).astype(np.float32)
        d = _dev(x, device)
        for scale in (1.0, 1.0 / n):
            got = cabi.negative_sum(d, scale).item()
            want = -float(np.float32(scale)) * x.astype(np.float64).sum()
            assert abs(got - want) <= 1e-6 * abs(want), (n, scale, got, want)
            assert cabi.negative_sum(d, scale).item() == got
    inf = _dev(np.array([-1.0, -np.inf], np.float32), device)
    assert cabi.negative_sum(inf, 1.0).item() == np.inf


@pytest.mark.parametrize("fls", [False, True])
def test_row_coefficients_with_the_loss_in_the_same_launch(fls, device):
    # ot_row_coefficients_loss = ot_row_coefficients + ot_negative_sum: the same coefficient
    # bytes and the same bits of the loss (transducer_loss.py:145-147), twice in a row
    _, T, U, tg, x, blank, osf = CASES[0]
    xin = helpers.log_softmax32(x) if fls else x
    _, _, parts = helpers.oracle_full(xin, tg, T, U, blank, fls, osf)
    ninf = lambda v: np.where(np.isnan(v), -np.inf, v).astype(np.float32)  # noqa: E731
    dT, dU, dtg = _dev(T, device), _dev(U, device), _dev(tg, device)
    splits, _ = cabi.row_splits(dT, dU, dtg)
    den = None if fls else _dev(parts["den"], device)
    args = (_dev(ninf(parts["lp"]), device), den, _dev(ninf(parts["alpha"]), device),
            _dev(ninf(parts["beta"]), device), dtg, dT, dU, splits, blank, fls, osf)
    rng = np.random.default_rng(11)
    for n_scale in (1.0, 1.0 / len(T)):
        scores = _dev((-rng.random(len(T)) * 300).astype(np.float32), device)
        plain, none = cabi.row_coefficients(*args, grad_scale=n_scale)
        assert none is None
        want = cabi.negative_sum(scores, n_scale)
        for _ in range(2):
            fused, loss = cabi.row_coefficients(*args, grad_scale=n_scale, scores=scores,
                                                loss_scale=n_scale)
            assert torch.equal(fused, plain)
            assert torch.equal(loss, want), (loss.item(), want.item())
    # a missing scores or loss pointer is refused before anything is launched
    rows = int(parts["alpha"].size)
    scratch = torch.zeros(cabi.lib().ot_gradient_scratch_bytes(ctypes.c_int64(rows)),
                          dtype=torch.uint8, device=device)
    rc = cabi.lib().ot_row_coefficients_loss(
        cabi.ptr(args[0]), cabi.ptr(den), cabi.ptr(args[2]), cabi.ptr(args[3]), cabi.ptr(dtg),
        cabi.ptr(dT), cabi.ptr(dU), cabi.ptr(splits), ctypes.c_int32(len(T)),
        ctypes.c_int32(tg.shape[1]), ctypes.c_int64(rows), ctypes.c_int32(blank),
        ctypes.c_int32(int(fls)), ctypes.c_int32(int(osf)), ctypes.c_float(1.0), cabi.ptr(scratch),
        None, ctypes.c_float(1.0), None, cabi.stream())
    assert rc != 0


def test_copy_floats(device):
    a = torch.randn(1 << 20, device=device)
    b = torch.zeros_like(a)
    cabi.copy_floats(a, b)
    assert torch.equal(a, b)


@pytest.mark.parametrize("osf", [False, True])
def test_guarded_lattice_launch(osf, device):
    """ot_alpha_beta_guarded: the same results when the batch is what the caller believes, an
    upper bound on the columns is fine, and nothing is written when the rows do not add up or a
    length is out of range (the launch must be safe before the host has validated anything)."""
    rng = np.random.default_rng(41)
    T = np.array([9, 4, 17, 30], np.int32)
    U = np.array([3, 0, 70, 12], np.int32)
    if osf:
        T = np.maximum(T, U + 2).astype(np.int32)
    rows = int((T.astype(np.int64) * (U + 1)).sum())
    lp = (-rng.random((rows, 2)) * 5 - 0.05).astype(np.float32)
    dT, dU, dlp = _dev(T, device), _dev(U, device), _dev(lp, device)
    splits, _ = cabi.row_splits(dT, dU, torch.zeros((4, 0), dtype=torch.int32, device=device))
    want = cabi.alpha_beta(dlp, dT, dU, splits, int(U.max()) + 1, osf)
    for max_u1 in (int(U.max()) + 1, 100):   # exact, and an upper bound in the same launch shape
        got = cabi.alpha_beta_guarded(dlp, dT, dU, splits, max_u1, osf, rows)
        for g, w in zip(got, want):
            assert torch.equal(torch.nan_to_num(g, nan=7.0), torch.nan_to_num(w, nan=7.0))
    # rows that do not add up: untouched outputs
    for bad_rows in (rows - 1, rows + 5):
        got = cabi.alpha_beta_guarded(dlp, dT, dU, splits, int(U.max()) + 1, osf, bad_rows)
        assert all(torch.isnan(g).all() for g in got)
    # a negative length that leaves the sum intact, and too few columns for one utterance: those
    # workgroups write nothing, the others are unaffected by construction of the guard
    T2, U2 = T.copy(), U.copy()
    T2[1] = -T2[1]
    dT2 = _dev(T2, device)
    got = cabi.alpha_beta_guarded(dlp, dT2, dU, splits, int(U.max()) + 1, osf, rows)
    a = got[0].cpu().numpy()
    s0, s1 = int(splits[1].item()), int(splits[2].item())
    assert np.isnan(a[s0:s1]).all()
    got = cabi.alpha_beta_guarded(dlp, dT, dU, splits, 64, osf, rows)   # U = 70 needs 71 columns
    a = got[0].cpu().numpy()
    s2, s3 = int(splits[2].item()), int(splits[3].item())
    assert np.isnan(a[s2:s3]).all() and not np.isnan(a[:s0]).any()
