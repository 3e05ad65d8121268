"""Pins the CPU oracle (oracle/transducer_oracle.c) without a GPU.

Each function of the oracle is checked against something that does not share
its code: closed forms, brute-force enumeration of alignments, numpy/torch
library routines, float64 autograd through an independently written
recursion, the golden vectors produced by the compiled reference, and - where
it has been built - the compiled reference itself (oracle/_ref).
"""
import math

import numpy as np
import pytest
import torch

import helpers
from helpers import ATOL, EPS32, RTOL
from oracle import oracle, ref_loader

MODES = [(False, False), (False, True), (True, False), (True, True)]  # (from_log_softmax, one_sym)


# ------------------------------------------------------------------ integers
def test_row_splits_row_ids_decode_are_closed_form():
    rng = np.random.default_rng(7)
    T = rng.integers(1, 40, size=23).astype(np.int32)
    U = rng.integers(0, 12, size=23).astype(np.int32)
    targets = rng.integers(0, 50, size=(23, int(U.max()))).astype(np.int32)
    splits, total = oracle.row_splits(T, U)
    want = np.concatenate([[0], np.cumsum(T.astype(np.int64) * (U + 1))])
    assert total == want[-1]
    assert splits.dtype == np.int32 and (splits == want).all()
    ids = oracle.row_ids(splits)
    assert (ids == np.repeat(np.arange(23), T * (U + 1))).all()
    dec = oracle.decode_rows(splits, ids, targets, U)
    for b in range(23):
        sl = slice(splits[b], splits[b + 1])
        t, u = np.divmod(np.arange(T[b] * (U[b] + 1)), U[b] + 1)
        assert (dec[sl, 0] == b).all() and (dec[sl, 1] == t).all() and (dec[sl, 2] == u).all()
        tg = np.where(u < U[b], targets[b][np.minimum(u, max(U[b] - 1, 0))] if U[b] else -1, -1)
        assert (dec[sl, 3] == tg).all()


def test_row_splits_wraps_like_int32_cumsum():
    # 3 utterances of 2^30 rows: int32 cumsum wraps, the int64 total does not
    T = np.array([1 << 15] * 3, np.int32)
    U = np.array([(1 << 15) - 1] * 3, np.int32)
    splits, total = oracle.row_splits(T, U)
    assert total == 3 * (1 << 30)
    want = np.cumsum(np.array([1 << 30] * 3, np.int64)).astype(np.int32)  # wraps
    assert (splits[1:] == want).all()


# ------------------------------------------------------------ denominators
def test_logsumexp_matches_torch_and_float64():
    rng = np.random.default_rng(11)
    for V in (3, 32, 500, 1001):
        x = (rng.standard_normal((257, V)) * 3).astype(np.float32)
        x[5] *= 20  # peaky row
        d32 = oracle.logsumexp(x)
        d64 = oracle.logsumexp(x, dtype=np.float64)
        want64 = torch.logsumexp(torch.from_numpy(x).double(), 1).numpy()
        want32 = torch.logsumexp(torch.from_numpy(x), 1).numpy()
        assert np.allclose(d64, want64, rtol=1e-13, atol=1e-13)
        # fp32: within 2 ulp of ATen's fp32 result and of the float64 value, an ulp
        # being that of the larger of the result and the row maximum it is added to
        ulp = np.spacing(np.maximum(np.abs(want32), np.abs(x).max(1)).astype(np.float32))
        assert (np.abs(d32 - want32) <= 2 * ulp).all()
        assert (np.abs(d32 - want64) <= 2 * ulp).all()


def test_logsumexp_infinite_rows_follow_aten():
    x = np.zeros((3, 4), np.float32)
    x[0] = -np.inf
    x[1, 2] = np.inf
    x[2] = [1, 2, 3, 4]
    got = oracle.logsumexp(x)
    want = torch.logsumexp(torch.from_numpy(x), 1).numpy()
    assert got[0] == want[0] == -np.inf and got[1] == want[1] == np.inf
    assert abs(got[2] - want[2]) < 1e-6


def test_log_probs_is_log_softmax_gather():
    rng = np.random.default_rng(12)
    T, U, targets, x = helpers.random_batch(rng, 5, 9, 6, 17)
    blank = 3
    den = oracle.logsumexp(x)
    lp = oracle.log_probs(x, den, targets, T, U, blank)
    lsm = torch.log_softmax(torch.from_numpy(x), 1).numpy()
    splits, _ = oracle.row_splits(T, U)
    for b in range(len(T)):
        for t in range(T[b]):
            for u in range(U[b] + 1):
                r = splits[b] + t * (U[b] + 1) + u
                assert abs(lp[r, 0] - lsm[r, blank]) < 2e-6
                if u < U[b]:
                    assert abs(lp[r, 1] - lsm[r, targets[b, u]]) < 2e-6
                else:
                    assert np.isnan(lp[r, 1])  # left uninitialised by the reference
    # log-softmax input: values are taken as they are
    lp2 = oracle.log_probs(lsm, None, targets, T, U, blank)
    m = ~np.isnan(lp2)
    r = np.arange(x.shape[0])
    assert (lp2[:, 0] == lsm[r, blank]).all() and m[:, 0].all()


# ------------------------------------------------------- likelihoods (alpha, beta)
def _lp_tables(rng, T, U):
    """Random normalised-looking blank/symbol log-probs for one utterance."""
    lpb = np.log(rng.uniform(0.05, 0.6, size=(T, U + 1)))
    lps = np.log(rng.uniform(0.05, 0.4, size=(T, U + 1)))
    return lpb, lps


@pytest.mark.parametrize("one_sym", [False, True])
def test_alpha_beta_scores_equal_brute_force_enumeration(one_sym):
    rng = np.random.default_rng(21)
    shapes = [(1, 0), (2, 0), (2, 1), (3, 2), (4, 3), (5, 2), (6, 3), (4, 1), (7, 2)]
    for T, U in shapes:
        if one_sym and U > T - 1:
            continue
        lpb, lps = _lp_tables(rng, T, U)
        want = helpers.brute_force_loglik(lpb, lps, one_sym)
        lp = np.stack([lpb.reshape(-1), lps.reshape(-1)], 1)
        for dt, tol in ((np.float64, 1e-12), (np.float32, 2e-5)):
            a, sa = oracle.alpha(lp.astype(dt), [T], [U], one_sym)
            b, sb = oracle.beta(lp.astype(dt), [T], [U], one_sym)
            assert abs(sa[0] - want) < tol * max(1, abs(want)), (T, U, sa, want)
            assert abs(sb[0] - want) < tol * max(1, abs(want)), (T, U, sb, want)


@pytest.mark.parametrize("one_sym", [False, True])
def test_constant_logits_closed_form(one_sym):
    # every arc has probability 1/V: ll = log(#paths) - (#arcs) log V
    V = 11
    for T, U in [(1, 0), (5, 0), (6, 3), (9, 8), (12, 4), (30, 7)]:
        if one_sym and U > T - 1:
            continue
        rows = T * (U + 1)
        x = np.full((rows, V), 0.25, np.float32)
        targets = np.full((1, max(U, 1)), 4, np.int32)[:, :U]
        if one_sym:
            want = math.log(math.comb(T - 1, U)) - T * math.log(V)
        else:
            want = math.log(math.comb(T - 1 + U, U)) - (T + U) * math.log(V)
        for fls in (False, True):
            xin = helpers.log_softmax32(x) if fls else x
            s64, _ = oracle.compute_transducer_loss(xin.copy(), targets, [T], [U], 0, fls, one_sym,
                                                    dtype=np.float64)
            s32, _ = oracle.compute_transducer_loss(xin.copy(), targets, [T], [U], 0, fls, one_sym)
            assert abs(s64[0] - want) < 1e-5 * abs(want)  # inputs are fp32-rounded
            assert abs(s32[0] - want) < 1e-5 * abs(want)


@pytest.mark.parametrize("one_sym", [False, True])
def test_occupancy_invariant_every_path_crosses_every_cut_once(one_sym):
    # standard: LSE over each anti-diagonal t+u=n of alpha+beta equals ll;
    # modified: LSE over u of alpha(t,u)+beta(t,u) equals ll for every frame t.
    rng = np.random.default_rng(22)
    T, U, targets, x = helpers.random_batch(rng, 4, 14, 6, 9, one_sym_per_frame=one_sym, tmin=2)
    s, _, parts = helpers.oracle_full(x, targets, T, U, 0, False, one_sym, dtype=np.float64)
    splits, _ = oracle.row_splits(T, U)
    for b in range(len(T)):
        U1 = U[b] + 1
        ab = (parts["alpha"] + parts["beta"])[splits[b]:splits[b + 1]].reshape(T[b], U1)
        ab = np.where(np.isnan(ab), -np.inf, ab)
        assert abs(parts["scores_beta"][b] - s[b]) < 1e-10
        if one_sym:
            cuts = [ab[t, :] for t in range(T[b])]
        else:
            cuts = [np.array([ab[n - u, u] for u in range(U1) if 0 <= n - u < T[b]])
                    for n in range(T[b] + U[b])]
        for c in cuts:
            m = c.max()
            assert abs(m + math.log(np.exp(c - m).sum()) - s[b]) < 1e-9


def test_modified_band_and_uninitialised_cells():
    T, U = [7], [3]
    lp = np.zeros((7 * 4, 2))
    a, _ = oracle.alpha(lp, T, U, True)
    b, _ = oracle.beta(lp, T, U, True)
    a, b = a.reshape(7, 4), b.reshape(7, 4)
    diff = 7 - 1 - 3
    for t in range(7):
        for u in range(4):
            inband = u <= t and t - u <= diff
            assert np.isnan(a[t, u]) == (not inband)
            assert np.isnan(b[t, u]) == (not inband)
    assert (~np.isnan(a)).sum() == (diff + 1) * 4


# ---------------------------------------------------------------- gradients
@pytest.mark.parametrize("fls,one_sym", MODES)
def test_gradient_equals_float64_autograd_of_independent_recursion(fls, one_sym):
    rng = np.random.default_rng(31)
    T, U, targets, x = helpers.random_batch(rng, 3, 7, 4, 6, one_sym_per_frame=one_sym)
    blank = 2
    # a target equal to blank makes the reference drop one of the two arc terms
    # (pinned separately below); true derivatives need targets != blank
    targets = np.where(targets == blank, 5, targets).astype(np.int32)
    xin = helpers.log_softmax32(x) if fls else x
    xt = torch.from_numpy(xin).double().requires_grad_(True)
    ll = helpers.torch_loss_f64(xt, targets, T, U, blank, fls, one_sym)
    (-ll.sum()).backward()
    want = xt.grad.numpy()
    s64, g64 = oracle.compute_transducer_loss(xin.copy(), targets, T, U, blank, fls, one_sym,
                                              dtype=np.float64)
    assert np.allclose(s64, ll.detach().numpy(), rtol=1e-12, atol=1e-12)
    assert np.allclose(g64, want, rtol=1e-9, atol=1e-12)
    s32, g32 = oracle.compute_transducer_loss(xin.copy(), targets, T, U, blank, fls, one_sym)
    assert np.allclose(s32, s64, rtol=RTOL, atol=ATOL)
    assert np.allclose(g32, g64, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("one_sym", [False, True])
def test_gradient_row_sum_invariants(one_sym):
    rng = np.random.default_rng(32)
    T, U, targets, x = helpers.random_batch(rng, 3, 10, 5, 8, one_sym_per_frame=one_sym, tmin=2)
    # logits input: each row of d(-ll)/d(logits) sums to zero (softmax Jacobian)
    _, g = oracle.compute_transducer_loss(x.copy(), targets, T, U, 0, False, one_sym,
                                          dtype=np.float64)
    assert np.abs(g.sum(1)).max() < 1e-12
    # log-softmax input: row sum is minus the node occupancy; occupancies of a
    # cut (anti-diagonal / frame) sum to one
    xl = helpers.log_softmax32(x)
    _, gl = oracle.compute_transducer_loss(xl.copy(), targets, T, U, 0, True, one_sym,
                                           dtype=np.float64)
    splits, _ = oracle.row_splits(T, U)
    for b in range(len(T)):
        occ = -gl[splits[b]:splits[b + 1]].sum(1).reshape(T[b], U[b] + 1)
        if one_sym:
            cuts = [occ[t, :].sum() for t in range(T[b])]
        else:
            cuts = [sum(occ[n - u, u] for u in range(U[b] + 1) if 0 <= n - u < T[b])
                    for n in range(T[b] + U[b])]
        assert np.allclose(cuts, 1.0, atol=1e-10)
        assert (occ >= -1e-15).all()


def test_single_cell_lattice_closed_form():
    # T=1, U=0: loss = -log softmax(x)[blank], gradient = softmax(x) - onehot(blank)
    x = np.array([[0.3, -1.2, 2.0, 0.1, -0.4]], np.float32)
    targets = np.zeros((1, 0), np.int32)
    for one_sym in (False, True):
        s, g = oracle.compute_transducer_loss(x.copy(), targets, [1], [0], 3, False, one_sym)
        p = np.exp(x[0].astype(np.float64))
        p /= p.sum()
        assert abs(s[0] - math.log(p[3])) < 1e-6
        want = p.copy()
        want[3] -= 1
        assert np.allclose(g[0], want, atol=1e-6)


@pytest.mark.parametrize("one_sym", [False, True])
def test_log_softmax_input_is_chain_rule_of_logits_input(one_sym):
    # what the reference's test_log_softmax.py:55-80 and test_max_symbol_per_frame.py:40-65 assert
    rng = np.random.default_rng(33)
    T, U, targets, x = helpers.random_batch(rng, 2, 9, 5, 7, one_sym_per_frame=one_sym, tmin=2)
    s_a, g_a = oracle.compute_transducer_loss(x.copy(), targets, T, U, 0, False, one_sym,
                                              dtype=np.float64)
    xl64 = torch.log_softmax(torch.from_numpy(x).double(), 1)
    xl = xl64.float().numpy()
    s_b, g_b = oracle.compute_transducer_loss(xl.copy(), targets, T, U, 0, True, one_sym,
                                              dtype=np.float64)
    p = np.exp(xl64.numpy())
    chain = g_b - p * g_b.sum(1, keepdims=True)
    assert np.allclose(s_a, s_b, rtol=1e-6, atol=1e-5)
    assert np.allclose(g_a, chain, atol=2e-6)


def test_target_equal_to_blank_follows_reference_branch_order():
    # cpu.cc:514-523: the blank tests come first, so at a node whose symbol is the
    # blank id the column carries the blank arc's term (plus nothing for the symbol arc).
    T, U, blank, V = [3], [2], 1, 4
    targets = np.array([[1, 2]], np.int32)  # first target equals blank
    rng = np.random.default_rng(34)
    x = rng.standard_normal((3 * 3, V)).astype(np.float32)
    _, g, parts = helpers.oracle_full(x, targets, T, U, blank, False, False, dtype=np.float64)
    a, b, d = parts["alpha"], parts["beta"], parts["den"]
    loss = -b[0]
    # node (t=0,u=0): v == blank and t < T-1 -> blank branch with beta(1,0)
    r = 0
    gexp = math.exp(x[r, blank] + a[r] + loss - d[r] + b[r]) - \
        math.exp(x[r, blank] + a[r] + loss - d[r] + b[r + 3])
    assert abs(g[r, blank] - gexp) < 1e-12
    # node (t=2,u=0): last frame, not the last node -> the symbol branch owns the column
    r = 2 * 3
    gexp = math.exp(x[r, blank] + a[r] + loss - d[r] + b[r]) - \
        math.exp(x[r, blank] + a[r] + loss - d[r] + b[r + 1])
    assert abs(g[r, blank] - gexp) < 1e-12


def test_python_level_reduction_and_backward_scaling():
    # transducer_loss.py:145-162: loss = -scores; mean => /N on loss and grad; grad *= loss_grad
    rng = np.random.default_rng(35)
    T, U, targets, x = helpers.random_batch(rng, 4, 8, 4, 6)
    s, g = oracle.compute_transducer_loss(x.copy(), targets, T, U, 0, False, False,
                                          dtype=np.float64)
    for red, k in (("sum", 1.0), ("mean", 1.0 / 4)):
        loss, grad = oracle.transducer_loss(x.copy(), targets, T, U, 0, False, False, red,
                                            loss_grad=3.0, dtype=np.float64)
        assert abs(loss - (-s.sum() * k)) < 1e-12
        assert np.allclose(grad, g * k * 3.0, rtol=1e-14)


# ------------------------------------------------------ golden vectors, reference
@pytest.mark.parametrize("path", helpers.golden_files(), ids=lambda p: p.split("/")[-1][:-4])
def test_oracle_reproduces_golden_vectors_of_compiled_reference(path):
    g = np.load(path)
    T, U, targets, blank = g["logit_lengths"], g["target_lengths"], g["targets"], int(g["blank"])
    for fls, osf in helpers.golden_modes(g):
        x = helpers.log_softmax32(g["logits"]) if fls else g["logits"]
        s, gr = oracle.compute_transducer_loss(x.copy(), targets, T, U, blank, fls, osf)
        ws, wg = g["scores_fls%d_osf%d" % (fls, osf)], g["grad_fls%d_osf%d" % (fls, osf)]
        if fls:
            # no ATen call on this path: same scalar libm arithmetic, same bits
            assert (s == ws).all() and (gr == wg).all(), (path, fls, osf)
        else:
            # the denominators come from ATen's vectorised logsumexp in the reference
            # and differ in the last bit; everything downstream inherits that
            assert np.allclose(s, ws, rtol=RTOL, atol=ATOL)
            _, _, tol = helpers.oracle_tolerance(x, targets, T, U, blank, fls, osf)
            assert (np.abs(gr - wg) <= tol).all(), np.abs(gr - wg).max()


@pytest.mark.skipif(not ref_loader.available(), reason="oracle/_ref not built")
@pytest.mark.parametrize("fls,one_sym", MODES)
def test_oracle_against_compiled_reference_live(fls, one_sym):
    ref = ref_loader.load()
    rng = np.random.default_rng(41 + 2 * fls + one_sym)
    for trial in range(3):
        T, U, targets, x = helpers.random_batch(rng, 5, 40, 12, 23, one_sym_per_frame=one_sym,
                                                target_low=0)
        blank = int(rng.integers(0, 23))  # targets may hit it: exercises cpu.cc:514-523
        xin = helpers.log_softmax32(x) if fls else x
        xt = torch.from_numpy(xin.copy()).requires_grad_(True)
        ws, wg = ref.compute_transducer_loss(
            logits=xt, targets=torch.from_numpy(targets), logit_lengths=torch.from_numpy(T),
            target_lengths=torch.from_numpy(U), blank=blank, from_log_softmax=fls,
            one_sym_per_frame=one_sym)
        ws, wg = ws.detach().numpy(), wg.detach().numpy()
        s, g, parts = helpers.oracle_full(xin, targets, T, U, blank, fls, one_sym)
        if fls:
            assert (s == ws).all() and (g == wg).all()
        else:
            assert np.allclose(s, ws, rtol=RTOL, atol=ATOL)
            _, _, tol = helpers.oracle_tolerance(xin, targets, T, U, blank, fls, one_sym)
            assert (np.abs(g - wg) <= tol).all()
        # in-place mode overwrites the logits buffer with the same numbers (cpu.cc:814)
        if not fls:
            buf = xin.copy()
            _, g2 = oracle.compute_transducer_loss(buf, targets, T, U, blank, fls, one_sym,
                                                   in_place=True)
            assert g2 is buf and (buf == g).all()
            assert wg.ctypes.data == xt.detach().numpy().ctypes.data  # the reference aliases too


# ------------------------------------------------------------ packed joiner input
def _readme_joiner(encoder_out, decoder_out, logit_lengths, target_lengths, activation):
    # the reference's usage recipe, README.md:166-177, in torch (float64, autograd)
    N, D = encoder_out.shape[0], encoder_out.shape[2]
    encoder_out_list = [encoder_out[i, :logit_lengths[i], :] for i in range(N)]
    decoder_out_list = [decoder_out[i, :target_lengths[i] + 1, :] for i in range(N)]
    x = [e.unsqueeze(1) + d.unsqueeze(0) for e, d in zip(encoder_out_list, decoder_out_list)]
    x = [p.reshape(-1, D) for p in x]
    x = torch.cat(x)
    if activation == "relu":  # not in the README: another activation a joiner may use
        return torch.relu(x)
    return torch.tanh(x) if activation == "tanh" else x


@pytest.mark.parametrize("activation", [None, "tanh", "relu"])
def test_pack_joiner_oracle_matches_the_readme_recipe_and_its_autograd(activation):
    rng = np.random.default_rng(11)
    N, Tm, Um, D = 5, 9, 6, 7
    T = rng.integers(1, Tm + 1, size=N).astype(np.int32)
    U = rng.integers(0, Um, size=N).astype(np.int32)
    T[0], U[0] = 1, 0
    T[1], U[1] = Tm, Um - 1
    enc = rng.standard_normal((N, Tm, D))
    dec = rng.standard_normal((N, Um, D))
    te = torch.tensor(enc, requires_grad=True)
    td = torch.tensor(dec, requires_grad=True)
    want = _readme_joiner(te, td, T.tolist(), U.tolist(), activation)
    got = oracle.pack_joiner(enc, dec, T, U, activation, dtype=np.float64)
    assert got.shape == tuple(want.shape) == (int((T * (U + 1)).sum()), D)
    assert np.allclose(got, want.detach().numpy(), rtol=1e-14, atol=1e-14)
    # row order is the packed order of the loss: row_splits[b] + t*(U_b+1) + u
    splits, _ = oracle.row_splits(T, U)
    b, t, u = 1, 3, 2
    row = splits[b] + t * (U[b] + 1) + u
    s = enc[b, t] + dec[b, u]
    assert np.allclose(got[row], {None: s, "tanh": np.tanh(s), "relu": np.maximum(s, 0)}[activation])
    g = rng.standard_normal(got.shape)
    want.backward(torch.tensor(g))
    ge, gd, ae, ad = oracle.pack_joiner_backward(g, enc, dec, T, U, activation)
    assert np.allclose(ge, te.grad.numpy(), rtol=1e-12, atol=1e-12)
    assert np.allclose(gd, td.grad.numpy(), rtol=1e-12, atol=1e-12)
    assert (ge[0, 1:] == 0).all() and (gd[0, 1:] == 0).all()  # padding
    assert (ae >= np.abs(ge) - 1e-12).all() and (ad >= np.abs(gd) - 1e-12).all()
    assert np.isclose(ae.sum(), np.abs(g).sum()) and np.isclose(ad.sum(), np.abs(g).sum())
    # float32 evaluation of the forward agrees with float64 to rounding
    got32 = oracle.pack_joiner(enc.astype(np.float32), dec.astype(np.float32), T, U, activation)
    assert got32.dtype == np.float32 and np.allclose(got32, got, rtol=1e-6, atol=1e-6)


def test_project_joiner_oracle_is_the_linear_layer_of_the_readme():
    """README.md:176-177 projects the packed activations with nn.Linear: pinned against
    torch's float64 linear, against explicit sums on a tiny case, and by two properties a
    transposed weight or a dropped bias would break (identity weight, zero input)."""
    rng = np.random.default_rng(23)
    x = rng.standard_normal((9, 6))
    w = rng.standard_normal((4, 6))
    b = rng.standard_normal(4)
    got, mag = oracle.project_joiner(x, w, b)
    want = torch.nn.functional.linear(torch.tensor(x), torch.tensor(w), torch.tensor(b)).numpy()
    assert got.shape == (9, 4) and np.allclose(got, want, rtol=1e-14, atol=1e-14)
    for r, v in ((0, 0), (5, 3), (8, 1)):
        terms = [x[r, k] * w[v, k] for k in range(6)]
        assert abs(got[r, v] - (sum(terms) + b[v])) < 1e-13
        assert abs(mag[r, v] - (sum(abs(t) for t in terms) + abs(b[v]))) < 1e-13
    eye, _ = oracle.project_joiner(x, np.eye(6))
    assert np.array_equal(eye, x)
    zero, zmag = oracle.project_joiner(np.zeros((3, 6)), w, b)
    assert np.array_equal(zero, np.tile(b, (3, 1))) and np.array_equal(zmag, np.tile(np.abs(b), (3, 1)))


def test_project_joiner_weight_grad_oracle_is_autograds_linear_backward():
    """Pinned against torch's float64 autograd through nn.functional.linear, against
    explicit sums on single entries, and by cases that a transposed operand or a sum over
    the wrong axis would break (one-hot gradient: grad_weight picks a row of x; x of ones:
    every column of grad_weight is grad_bias)."""
    rng = np.random.default_rng(29)
    x = rng.standard_normal((9, 6))
    w = rng.standard_normal((4, 6))
    b = rng.standard_normal(4)
    g = rng.standard_normal((9, 4))
    gw, gw_mag, gb, gb_mag = oracle.project_joiner_weight_grad(g, x)
    tw = torch.tensor(w, requires_grad=True)
    tb = torch.tensor(b, requires_grad=True)
    torch.nn.functional.linear(torch.tensor(x), tw, tb).backward(torch.tensor(g))
    assert gw.shape == (4, 6) and np.allclose(gw, tw.grad.numpy(), rtol=1e-14, atol=1e-14)
    assert gb.shape == (4,) and np.allclose(gb, tb.grad.numpy(), rtol=1e-14, atol=1e-14)
    for v, k in ((0, 0), (3, 5), (2, 1)):
        terms = [g[r, v] * x[r, k] for r in range(9)]
        assert abs(gw[v, k] - sum(terms)) < 1e-13
        assert abs(gw_mag[v, k] - sum(abs(t) for t in terms)) < 1e-13
    assert np.allclose(gb_mag, np.abs(g).sum(0))
    onehot = np.zeros((9, 4))
    onehot[5, 2] = 1.0
    ow, _, ob, _ = oracle.project_joiner_weight_grad(onehot, x)
    assert np.array_equal(ow[2], x[5]) and not ow[[0, 1, 3]].any() and np.array_equal(ob, [0, 0, 1, 0])
    cw, _, cb, _ = oracle.project_joiner_weight_grad(g, np.ones((9, 6)))
    assert np.allclose(cw, np.tile(cb[:, None], (1, 6)), rtol=1e-14, atol=1e-14)
