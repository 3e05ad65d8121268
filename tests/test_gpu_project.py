"""Output projection of the joiner fused with the denominators (an addition to the
reference, whose caller runs torch's Linear and whose loss then re-reads the logits
for logsumexp, README.md:176-177, cuda.cu:427).

The oracle forms x @ W.T + bias in float64 from the 2-byte inputs (exact in float64)
and gives the scale of a float32 accumulation's rounding error; logits stored in a
2-byte type may in addition be off by one rounding of that type.  The denominators
are checked against the log-sum-exp of the values the kernel itself stored, which is
what the loss's own denominator pass would compute from them."""
import ctypes

import numpy as np
import pytest
import torch

import cabi
import helpers
from oracle import oracle

pytestmark = pytest.mark.gpu

HALF = {"f16": torch.float16, "bf16": torch.bfloat16}
ULP = {torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8, torch.float32: 0.0}


def _inputs(rng, rows, D, V, dtype, device, bias=True, scale=1.0):
    x = torch.from_numpy(np.tanh(rng.standard_normal((rows, D))).astype(np.float32)).to(dtype)
    w = torch.from_numpy((rng.standard_normal((V, D)) * scale / np.sqrt(D)).astype(np.float32)).to(dtype)
    b = torch.from_numpy(rng.standard_normal(V).astype(np.float32)) if bias else None
    return x.to(device), w.to(device), None if b is None else b.to(device)


def _check(x, w, b, out_dtype):
    logits, den = cabi.joiner_project(x, w, b, out_dtype)
    want, mag = oracle.project_joiner(x.float().cpu().numpy(), w.float().cpu().numpy(),
                                      None if b is None else b.cpu().numpy())
    got = logits.float().cpu().numpy().astype(np.float64)
    assert not np.isnan(got).any()
    tol = 2e-6 * mag + ULP[out_dtype] * np.abs(want) * 1.001 + 1e-30
    assert (np.abs(got - want) <= tol).all(), (np.abs(got - want) / tol).max()
    # denominators of the stored values
    m = got.max(1)
    ref = m + np.log(np.exp(got - m[:, None]).sum(1))
    d = den.cpu().numpy().astype(np.float64)
    assert (np.abs(d - ref) <= 4e-7 * np.maximum(np.abs(ref), np.abs(m)) + 1e-6).all(), np.abs(d - ref).max()
    # with a workspace (passes side by side, partial log-sum-exps merged): the same logits bit
    # for bit, denominators of the same stored values
    logits_ws, den_ws = cabi.joiner_project(x, w, b, out_dtype, workspace=True)
    assert torch.equal(logits_ws.view(torch.uint8), logits.view(torch.uint8))
    d = den_ws.cpu().numpy().astype(np.float64)
    assert (np.abs(d - ref) <= 4e-7 * np.maximum(np.abs(ref), np.abs(m)) + 1e-6).all(), np.abs(d - ref).max()
    return logits, den


@pytest.mark.parametrize("out", ["f32", "same"])
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("rows,D,V", [(700, 64, 500), (256, 64, 128), (1, 512, 37), (513, 192, 1030),
                                      (300, 128, 6), (64, 256, 130),
                                      # more 128-row tiles than resident workgroups: some take two
                                      # (and, with a workspace, the passes run side by side)
                                      (70001, 64, 40), (66000, 64, 300), (40000, 64, 1030), (33000, 128, 520),
                                      # four and eight passes side by side
                                      (40000, 64, 1000), (50000, 64, 2048),
                                      # many passes over the vocabulary, long rows of x
                                      (300, 128, 5000), (200, 1024, 777)])
def test_projection_and_denominators(rows, D, V, dtype, out, device):
    rng = np.random.default_rng(rows * 7 + V)
    dt = HALF[dtype]
    x, w, b = _inputs(rng, rows, D, V, dt, device)
    _check(x, w, b, torch.float32 if out == "f32" else dt)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_no_bias_and_large_values(dtype, device):
    rng = np.random.default_rng(5)
    dt = HALF[dtype]
    x, w, _ = _inputs(rng, 200, 64, 300, dt, device, bias=False, scale=40.0)
    _check(x, w, None, torch.float32)
    _check(x, w, None, dt)


def test_masked_logits_through_the_bias(device):
    # a -inf bias masks vocabulary entries: they must drop out of the denominator
    rng = np.random.default_rng(9)
    x, w, b = _inputs(rng, 100, 64, 200, torch.bfloat16, device)
    b[50:120] = -float("inf")
    logits, den = cabi.joiner_project(x, w, b, torch.float32)
    got = logits.cpu().numpy().astype(np.float64)
    assert np.isneginf(got[:, 50:120]).all() and np.isfinite(got[:, :50]).all()
    ref = torch.logsumexp(logits.double(), 1).cpu().numpy()
    assert np.allclose(den.cpu().numpy(), ref, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_log_probs_given_denominators(dtype, device):
    rng = np.random.default_rng(3)
    T, U, tg, x = helpers.random_batch(rng, 5, 9, 6, 41)
    xd = torch.from_numpy(x).to(dtype).to(device)
    x32 = xd.float().cpu().numpy()
    dT, dU, dtg = (torch.from_numpy(a).to(device) for a in (T, U, tg))
    splits, _ = cabi.row_splits(dT, dU, dtg)
    den = oracle.logsumexp(x32)
    want = oracle.log_probs(x32, den, tg, T, U, 0)
    got = cabi.log_probs_given_den(xd, torch.from_numpy(den).to(device), dtg, dU, splits, 0).cpu().numpy()
    m = np.isfinite(want)
    assert (got[m] == want[m]).all() and np.isneginf(got[~m]).all()


@pytest.mark.parametrize("V", [90, 96])   # 96: this package's weight-gradient kernel; 90: torch's products
@pytest.mark.parametrize("f32_logits", [True, False])
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_python_pipeline_matches_the_unfused_one(dtype, f32_logits, V, device):
    """project_joiner + transducer_loss(denominators=...) against torch's linear followed
    by transducer_loss on the same (rounded) logits: same loss, same gradients."""
    import optimized_transducer_amd as ot
    dt = HALF[dtype]
    rng = np.random.default_rng(17)
    T, U, tg, _ = helpers.random_batch(rng, 6, 12, 7, 8)
    rows, D = int((T * (U + 1)).sum()), 64
    tg = (tg % (V - 1) + 1).astype(np.int32)
    x0, w0, b0 = _inputs(rng, rows, D, V, dt, device)
    dT, dU, dtg = (torch.from_numpy(a).to(device) for a in (T, U, tg))

    def run(fused):
        x, w, b = (t.clone().requires_grad_(True) for t in (x0, w0, b0))
        if fused:
            logits, den = ot.project_joiner(x, w, b, float32_logits=f32_logits)
            loss = ot.transducer_loss(logits, dtg, dT, dU, 0, False, reduction="sum", denominators=den)
        else:
            logits = torch.nn.functional.linear(x.float(), w.float(), b)
            if not f32_logits:
                logits = logits.to(dt)
            loss = ot.transducer_loss(logits, dtg, dT, dU, 0, False, reduction="sum")
        (3.0 * loss).backward()
        return loss.item(), x.grad.float().cpu().numpy(), w.grad.float().cpu().numpy(), b.grad.cpu().numpy()

    lf, gxf, gwf, gbf = run(True)
    lu, gxu, gwu, gbu = run(False)
    # logits differ by float32 summation order (and, in 16 bits, by rare one-unit flips)
    unit = ULP[dt] if not f32_logits else 1e-6
    assert abs(lf - lu) <= 4 * unit * rows + 1e-4 * abs(lu), (lf, lu)
    for a, b_ in ((gxf, gxu), (gwf, gwu), (gbf, gbu)):
        scale = np.abs(b_).max()
        assert np.abs(a - b_).max() <= (0.02 if dt == torch.bfloat16 else 0.004) * scale + 1e-6, \
            (np.abs(a - b_).max(), scale)


@pytest.mark.parametrize("f32_logits", [True, False])
@pytest.mark.parametrize("bias", [True, False])
def test_padded_vocabulary_changes_nothing_but_the_shape(bias, f32_logits, device):
    """vocab_multiple: masked entries up to the next multiple.  Same logits and denominators
    in the real columns, -inf in the others; same loss; the same gradient bits with respect
    to the logits' real columns, zeros in the others; gradients of x, W, bias as without."""
    import optimized_transducer_amd as ot
    dt = torch.bfloat16
    rng = np.random.default_rng(23)
    T, U, tg, _ = helpers.random_batch(rng, 5, 11, 6, 8)
    rows, D, V = int((T * (U + 1)).sum()), 128, 90
    tg = (tg % (V - 1) + 1).astype(np.int32)
    x0, w0, b0 = _inputs(rng, rows, D, V, dt, device)
    dT, dU, dtg = (torch.from_numpy(a).to(device) for a in (T, U, tg))

    def run(multiple):
        x, w = x0.clone().requires_grad_(True), w0.clone().requires_grad_(True)
        b = b0.clone().requires_grad_(True) if bias else None
        logits, den = ot.project_joiner(x, w, b, float32_logits=f32_logits, vocab_multiple=multiple)
        leaf = logits.detach().clone().requires_grad_(True)
        loss = ot.transducer_loss(leaf, dtg, dT, dU, 0, False, reduction="sum", denominators=den)
        loss.backward()
        logits.backward(leaf.grad)
        return (logits.detach().clone(), den.clone(), loss.detach(), leaf.grad, x.grad, w.grad,
                b.grad if bias else None)

    plain = run(None)
    padded = run(32)
    assert plain[0].shape == (rows, V) and padded[0].shape == (rows, 96)
    assert torch.equal(padded[0][:, :V], plain[0]) and torch.isneginf(padded[0][:, V:]).all()
    assert torch.equal(padded[1], plain[1]) and torch.equal(padded[2], plain[2])
    assert torch.equal(padded[3][:, :V], plain[3]) and (padded[3][:, V:] == 0).all()
    # the backward products see V_p instead of V columns: the library may sum in another order
    for a, b_ in zip(padded[4:], plain[4:]):
        if b_ is None:
            assert a is None
            continue
        assert a.shape == b_.shape
        scale = b_.float().abs().max().item()
        assert (a.float() - b_.float()).abs().max().item() <= 0.02 * scale + 1e-6
    # a multiple that V already is: nothing is padded
    assert ot.project_joiner(x0, w0[:64].contiguous(), None, vocab_multiple=32)[0].shape == (rows, 64)
    with pytest.raises(ValueError, match="vocab_multiple"):
        ot.project_joiner(x0, w0, b0, vocab_multiple=0)


@pytest.mark.parametrize("osf", [False, True])
def test_joiner_transducer_loss_is_the_two_calls_in_one(osf, device):
    import optimized_transducer_amd as ot
    dt = torch.bfloat16
    rng = np.random.default_rng(29)
    T, U, tg, _ = helpers.random_batch(rng, 4, 10, 5, 8, one_sym_per_frame=osf)
    rows, D, V = int((T * (U + 1)).sum()), 64, 45
    tg = (tg % (V - 1) + 1).astype(np.int32)
    x0, w0, b0 = _inputs(rng, rows, D, V, dt, device)
    dT, dU, dtg = (torch.from_numpy(a).to(device) for a in (T, U, tg))

    def run(one_call):
        x, w, b = (t.clone().requires_grad_(True) for t in (x0, w0, b0))
        if one_call:
            loss = ot.joiner_transducer_loss(x, w, b, dtg, dT, dU, 0, osf, "sum")
        else:
            logits, den = ot.project_joiner(x, w, b)
            loss = ot.transducer_loss(logits, dtg, dT, dU, 0, False, osf, "sum", denominators=den)
        loss.backward()
        return loss.detach(), x.grad, w.grad, b.grad

    a, b_ = run(True), run(False)
    assert torch.equal(a[0], b_[0])
    for p, q in zip(a[1:], b_[1:]):
        scale = q.float().abs().max().item()
        assert p.shape == q.shape and (p.float() - q.float()).abs().max().item() <= 0.02 * scale + 1e-6


def test_denominators_argument_is_checked(device):
    import optimized_transducer_amd as ot
    rng = np.random.default_rng(2)
    T, U, tg, x = helpers.random_batch(rng, 3, 5, 3, 11)
    dT, dU, dtg = (torch.from_numpy(a).to(device) for a in (T, U, tg))
    logits = torch.from_numpy(x).to(device)
    den = torch.logsumexp(logits, 1)
    want = ot.transducer_loss(logits.clone(), dtg, dT, dU, 0, False).item()
    got = ot.transducer_loss(logits.clone(), dtg, dT, dU, 0, False, denominators=den).item()
    assert abs(got - want) <= 1e-5 * abs(want) + 1e-5
    with pytest.raises(RuntimeError, match="denominators"):
        ot.transducer_loss(logits.clone(), dtg, dT, dU, 0, False, denominators=den[:-1].contiguous())
    with pytest.raises(RuntimeError, match="denominators"):
        ot.transducer_loss(torch.log_softmax(logits, 1), dtg, dT, dU, 0, True, denominators=den)
    with pytest.raises(RuntimeError, match="multiple of 64"):
        ot.project_joiner(torch.zeros(4, 32, dtype=torch.bfloat16, device=device),
                          torch.zeros(5, 32, dtype=torch.bfloat16, device=device))


def test_projection_workspace_is_optional(device):
    """ot_joiner_project_ws without a workspace, or with one that is too short, is
    ot_joiner_project; a vocabulary of one pass needs none."""
    L = cabi.lib()
    L.ot_joiner_project_workspace_bytes.restype = ctypes.c_size_t
    rng = np.random.default_rng(3)
    rows, D, V = 70000, 64, 600
    assert L.ot_joiner_project_workspace_bytes(ctypes.c_int64(rows), ctypes.c_int32(256)) == 0
    assert L.ot_joiner_project_workspace_bytes(ctypes.c_int64(rows), ctypes.c_int32(257)) == 2 * rows * 4
    n = L.ot_joiner_project_workspace_bytes(ctypes.c_int64(rows), ctypes.c_int32(V))
    assert n == 3 * rows * 4
    x, w, b = _inputs(rng, rows, D, V, torch.bfloat16, device)
    want, want_den = cabi.joiner_project(x, w, b, torch.bfloat16)
    ws = torch.zeros(n, dtype=torch.uint8, device=device)
    for ws_ptr, ws_bytes in ((None, 0), (ws, n - 4), (None, n)):
        logits = torch.full((rows, V), float("nan"), dtype=torch.bfloat16, device=device)
        den = torch.full((rows,), float("nan"), dtype=torch.float32, device=device)
        cabi.check(L.ot_joiner_project_ws(cabi.ptr(x), cabi.ptr(w), cabi.ptr(b), ctypes.c_int32(2),
                                          ctypes.c_int64(rows), ctypes.c_int32(D), ctypes.c_int32(V),
                                          cabi.ptr(logits), ctypes.c_int32(2), cabi.ptr(den), cabi.ptr(ws_ptr),
                                          ctypes.c_size_t(ws_bytes), cabi.stream()))
        assert torch.equal(logits.view(torch.int16), want.view(torch.int16)) and torch.equal(den, want_den)
    # same argument checks as ot_joiner_project
    rc = L.ot_joiner_project_ws(cabi.ptr(x), cabi.ptr(w), cabi.ptr(b), ctypes.c_int32(0), ctypes.c_int64(rows),
                                ctypes.c_int32(D), ctypes.c_int32(V), cabi.ptr(want), ctypes.c_int32(2),
                                cabi.ptr(want_den), cabi.ptr(ws), ctypes.c_size_t(n), cabi.stream())
    assert rc == -1


# ---- backward of the projection in its parameters (ot_joiner_weight_grad)
def _weight_grad_inputs(rng, rows, V, D, dt, device):
    # a gradient of logits looks like this: small, mostly one sign per column, a few large entries
    g = rng.standard_normal((rows, V)) * 0.05 + 0.01
    g[rng.integers(0, rows, max(rows // 7, 1)), rng.integers(0, V, max(rows // 7, 1))] -= 1.0
    x = np.tanh(rng.standard_normal((rows, D)))
    return (torch.from_numpy(g.astype(np.float32)).to(dt).to(device),
            torch.from_numpy(x.astype(np.float32)).to(dt).to(device))


def _check_weight_grad(g, x, gw, gb):
    want_w, mag_w, want_b, mag_b = oracle.project_joiner_weight_grad(g.float().cpu().numpy(),
                                                                    x.float().cpu().numpy())
    got_w = gw.float().cpu().numpy().astype(np.float64)
    # float32 accumulation in slices (error relative to the sum of the absolute terms) and one
    # rounding to the 2-byte type
    tol = 2e-6 * mag_w + ULP[gw.dtype] * np.abs(want_w) * 1.001 + 1e-30
    assert not np.isnan(got_w).any()
    assert (np.abs(got_w - want_w) <= tol).all(), (np.abs(got_w - want_w) / tol).max()
    if gb is not None:
        got_b = gb.cpu().numpy().astype(np.float64)
        assert (np.abs(got_b - want_b) <= 2e-6 * mag_b + 1e-30).all(), np.abs(got_b - want_b).max()


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("rows,V,D", [
    (1, 8, 8), (100, 8, 8), (1000, 24, 64), (31, 504, 512), (5000, 504, 512),
    # several tiles either way, the last ones partly outside the matrix
    (3333, 264, 520), (257, 1032, 72), (600, 520, 1032),
    # fewer rows than slices; one row more than a whole number of stages per slice
    (40, 128, 64), (64 * 32 + 1, 40, 64),
    # many rows, narrow matrices
    (300001, 16, 24)])
def test_weight_and_bias_gradient_of_the_projection(rows, V, D, dtype, device):
    rng = np.random.default_rng(rows + 3 * V + D)
    dt = HALF[dtype]
    g, x = _weight_grad_inputs(rng, rows, V, D, dt, device)
    gw, gb = cabi.joiner_weight_grad(g, x, workspace_fill=0xFF)   # workspace full of NaN patterns
    _check_weight_grad(g, x, gw, gb)
    # same bits again, whatever the workspace holds; the bias gradient is optional
    gw2, none = cabi.joiner_weight_grad(g, x, want_bias=False, workspace_fill=0x7F)
    assert none is None and torch.equal(gw.view(torch.int16), gw2.view(torch.int16))
    gw3, gb3 = cabi.joiner_weight_grad(g, x)
    assert torch.equal(gw.view(torch.int16), gw3.view(torch.int16)) and torch.equal(gb, gb3)


def test_weight_gradient_on_random_shapes(device):
    """Shapes nobody picked: rows around the slice and stage boundaries, V and D any multiples of 8."""
    rng = np.random.default_rng(2024)
    for trial in range(24):
        V = 8 * int(rng.integers(1, 140))
        D = 8 * int(rng.integers(1, 140))
        rows = int(rng.choice([rng.integers(1, 70), rng.integers(70, 3000), 64 * 32 * int(rng.integers(1, 4)) + int(rng.integers(-2, 3))]))
        dt = (torch.float16, torch.bfloat16)[trial % 2]
        g, x = _weight_grad_inputs(rng, rows, V, D, dt, device)
        gw, gb = cabi.joiner_weight_grad(g, x, workspace_fill=0xFF)
        try:
            _check_weight_grad(g, x, gw, gb)
        except AssertionError as e:
            raise AssertionError("rows = %d, V = %d, D = %d, %s: %s" % (rows, V, D, dt, e))


def test_weight_gradient_is_linear_and_sees_every_row(device):
    """Properties no tolerance hides: a single nonzero row of g anywhere in the batch gives
    exactly g[r]^T x[r] rounded once (products of two 2-byte numbers are exact in float32);
    g of zeros gives zeros; swapping two rows of both operands changes nothing but the
    order of a float32 sum."""
    rng = np.random.default_rng(5)
    rows, V, D = 70000, 72, 136
    dt = torch.bfloat16
    g, x = _weight_grad_inputs(rng, rows, V, D, dt, device)
    zero = torch.zeros_like(g)
    gw, gb = cabi.joiner_weight_grad(zero, x)
    assert not gw.float().any() and not gb.any()
    for r in (0, 31, 32, 1093, 34999, 69999):
        one = torch.zeros_like(g)
        one[r] = g[r]
        gw, gb = cabi.joiner_weight_grad(one, x)
        want = (g[r].float()[:, None] * x[r].float()[None, :]).to(dt)
        assert torch.equal(gw.view(torch.int16), want.view(torch.int16)), r
        assert torch.equal(gb, g[r].float()), r


def test_weight_gradient_refuses_what_it_cannot_run(device):
    L = cabi.lib()
    L.ot_joiner_weight_grad_workspace_bytes.restype = ctypes.c_size_t
    g = torch.zeros((64, 16), dtype=torch.bfloat16, device=device)
    x = torch.zeros((64, 8), dtype=torch.bfloat16, device=device)
    out = torch.zeros((16, 8), dtype=torch.bfloat16, device=device)
    n = L.ot_joiner_weight_grad_workspace_bytes(ctypes.c_int64(64), ctypes.c_int32(16), ctypes.c_int32(8))
    ws = torch.zeros(n, dtype=torch.uint8, device=device)

    def call(g_=g, x_=x, dtype=2, rows=64, V=16, D=8, ws_=ws, n_=n, out_=out):
        return L.ot_joiner_weight_grad(cabi.ptr(g_), cabi.ptr(x_), ctypes.c_int32(dtype), ctypes.c_int64(rows),
                                       ctypes.c_int32(V), ctypes.c_int32(D), cabi.ptr(ws_), ctypes.c_size_t(n_),
                                       cabi.ptr(out_), cabi.ptr(None), cabi.stream())
    assert call() == 0
    assert call(dtype=0) == -1 and call(V=12) == -1 and call(D=4) == -1 and call(rows=0) == -1
    assert call(n_=n - 4) == -1 and call(g_=None) == -1 and call(ws_=None) == -1
    assert call(g_=g.view(-1)[1:]) == -3 and call(ws_=ws[4:], n_=n) == -3
    assert L.ot_joiner_weight_grad_workspace_bytes(ctypes.c_int64(0), ctypes.c_int32(16), ctypes.c_int32(8)) == 0


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_backward_of_project_joiner_uses_the_weight_gradient_kernel(dtype, device):
    """project_joiner's gradients of weight and bias against torch's own backward of the
    same linear layer on the same incoming gradient, padded vocabulary included."""
    import optimized_transducer_amd as ot
    rng = np.random.default_rng(41)
    dt = HALF[dtype]
    rows, D, V = 900, 128, 500
    x0, w0, b0 = _inputs(rng, rows, D, V, dt, device)
    for vocab_multiple, Vout in ((None, V), (32, 512), (8, 504)):
        gl = torch.from_numpy((rng.standard_normal((rows, Vout)) * 0.05).astype(np.float32)).to(dt).to(device)
        gl[:, V:] = 0.0    # what the loss hands back in masked columns
        x, w, b = (t.clone().requires_grad_(True) for t in (x0, w0, b0))
        ext = ot._optimized_transducer
        ext.set_profiling(True)
        ext.take_profile()
        logits, _ = ot.project_joiner(x, w, b, float32_logits=False, vocab_multiple=vocab_multiple)
        logits.backward(gl)
        names = [n for n, _ in ext.take_profile()]
        ext.set_profiling(False)
        # V = 500 itself is not a multiple of 8: torch's products; 504 and 512 are
        assert ("joiner_weight_grad" in names) == (Vout % 8 == 0 and vocab_multiple is not None), names
        want_w, mag_w, want_b, mag_b = oracle.project_joiner_weight_grad(
            gl[:, :V].float().cpu().numpy(), x0.float().cpu().numpy())
        got_w = w.grad.float().cpu().numpy().astype(np.float64)
        assert w.grad.shape == (V, D) and b.grad.shape == (V,) and b.grad.dtype == b0.dtype
        assert (np.abs(got_w - want_w) <= 2e-6 * mag_w + ULP[dt] * np.abs(want_w) * 1.001 + 1e-30).all()
        assert (np.abs(b.grad.cpu().numpy() - want_b) <= 2e-6 * mag_b + 1e-30).all()
        assert x.grad.shape == (rows, D)
