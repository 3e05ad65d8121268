"""GPU parity of the whole path: the Python entry points of the package and
ot_transducer_loss of the C ABI, against the golden vectors of the compiled
reference, the CPU oracle and - at the benchmark's full sizes - properties that
do not depend on size plus the oracle run on a slice of the batch."""
import numpy as np
import pytest
import torch

import cabi
import helpers
import workloads
from helpers import ATOL, RTOL
from oracle import oracle

pytestmark = pytest.mark.gpu

MODES = [(False, False), (False, True), (True, False), (True, True)]  # (from_log_softmax, one_sym)


def _dev(a, device):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def _run_api(x, tg, T, U, blank, fls, osf, reduction, device, upstream=1.0, module=False):
    import optimized_transducer_amd as ot
    logits = _dev(x, device).requires_grad_(True)
    args = (logits, _dev(tg, device), _dev(T, device), _dev(U, device))
    if module:
        loss = ot.TransducerLoss(blank=blank, reduction=reduction)(*args, fls, osf)
    else:
        loss = ot.transducer_loss(*args, blank, fls, one_sym_per_frame=osf, reduction=reduction)
    (loss * upstream if upstream != 1.0 else loss).backward()
    return loss, logits


# ------------------------------------------------------------------ golden vectors
@pytest.mark.parametrize("path", helpers.golden_files(), ids=lambda p: p.split("/")[-1][:-4])
def test_golden_vectors_of_the_compiled_reference(path, device):
    g = np.load(path)
    T, U, tg, blank = g["logit_lengths"], g["target_lengths"], g["targets"], int(g["blank"])
    for fls, osf in helpers.golden_modes(g):
        x = helpers.log_softmax32(g["logits"]) if fls else g["logits"]
        ws, wg = g["scores_fls%d_osf%d" % (fls, osf)], g["grad_fls%d_osf%d" % (fls, osf)]
        loss, logits = _run_api(x, tg, T, U, blank, fls, osf, "sum", device)
        assert np.allclose(loss.item(), -ws.sum(dtype=np.float64), rtol=RTOL, atol=ATOL)
        got = logits.grad.cpu().numpy()
        _, _, tol = helpers.oracle_tolerance(x, tg, T, U, blank, fls, osf)
        assert (np.abs(got - wg) <= tol).all(), (fls, osf, np.abs(got - wg).max())
        if np.abs(ws).max() < 50:  # short lattices: the plain north-star tolerance holds
            assert np.allclose(got, wg, rtol=RTOL, atol=ATOL)


# ------------------------------------------------------------------ Python API
@pytest.mark.parametrize("reduction", ["mean", "sum"])
@pytest.mark.parametrize("fls,osf", MODES)
def test_python_api_matches_oracle(fls, osf, reduction, device):
    w = workloads.tiny(from_log_softmax=fls, one_sym_per_frame=osf)
    x = w.logits_numpy()
    want_loss, want_grad = oracle.transducer_loss(x.copy(), w.targets, w.logit_lengths,
                                                  w.target_lengths, w.blank, fls, osf, reduction,
                                                  loss_grad=3.0)
    loss, logits = _run_api(x, w.targets, w.logit_lengths, w.target_lengths, w.blank, fls, osf,
                            reduction, device, upstream=3.0)  # as test_compute_transducer_loss.py:92
    assert loss.dim() == 0 and loss.dtype == torch.float32
    assert np.allclose(loss.item(), want_loss, rtol=RTOL, atol=ATOL)
    _, _, tol = helpers.oracle_tolerance(x, w.targets, w.logit_lengths, w.target_lengths, w.blank,
                                         fls, osf, scale=3.0 / (w.N if reduction == "mean" else 1))
    got = logits.grad.cpu().numpy()
    assert (np.abs(got - want_grad) <= tol).all(), np.abs(got - want_grad).max()
    # arbiter: the GPU is as close to the float64 evaluation as the fp32 reference arithmetic is
    _, g64 = oracle.transducer_loss(x.copy(), w.targets, w.logit_lengths, w.target_lengths,
                                    w.blank, fls, osf, reduction, loss_grad=3.0, dtype=np.float64)
    assert np.abs(got - g64).max() <= 2 * np.abs(want_grad - g64).max() + 1e-6


@pytest.mark.parametrize("reduction", ["mean", "sum"])
@pytest.mark.parametrize("defer", [False, True])
def test_loss_has_the_same_bits_with_and_without_a_gradient(defer, reduction, device):
    # with a gradient the loss is reduced inside the row-coefficient launch, without one by
    # a launch of its own (transducer_loss.py:145-147 either way): same summation, same bits,
    # and equal to the reduction of the binding's per-utterance scores
    import optimized_transducer_amd as ot
    from optimized_transducer_amd import _optimized_transducer as ext
    w = workloads.asr_batch(N=7, V=33, scale=0.1)
    x = torch.from_numpy(w.logits_numpy()).to(device)
    tg, T, U = (torch.from_numpy(a).to(device) for a in (w.targets, w.logit_lengths, w.target_lengths))
    plain = ot.transducer_loss(x.clone(), tg, T, U, w.blank, False, False, reduction)
    with_grad = ot.transducer_loss(x.clone().requires_grad_(True), tg, T, U, w.blank, False, False,
                                   reduction, defer_gradient=defer)
    scores, _ = ext.compute_transducer_loss(logits=x.clone(), targets=tg, logit_lengths=T,
                                            target_lengths=U, blank=w.blank, from_log_softmax=False,
                                            one_sym_per_frame=False)
    want = ext.negative_sum(scores, 1.0 / w.N if reduction == "mean" else 1.0)
    assert torch.equal(plain, want) and torch.equal(with_grad.detach(), want)


@pytest.mark.parametrize("big", [False, True], ids=["small", "large"])
def test_random_batches_against_the_oracle(big, device):
    # every option drawn at random per batch: recursion, input kind, reduction, blank anywhere in
    # [0, V), V with and without a factor of 4, an upstream gradient, the deferred mode
    import optimized_transducer_amd as ot
    rng = np.random.default_rng(20261125 + big)
    for case in range(12 if big else 60):
        osf, fls, defer = (bool(rng.integers(0, 2)) for _ in range(3))
        N = int(rng.integers(1, 5 if big else 7))
        V = int(rng.integers(2, 700 if big else 70))
        tmax = int(rng.integers(1, 300 if big else 60))
        umax = int(rng.integers(0, 160 if big else 20))
        T, U, tg, x = helpers.random_batch(rng, N, tmax, umax, V, one_sym_per_frame=osf)
        blank = int(rng.integers(0, V))
        reduction = ("mean", "sum")[int(rng.integers(0, 2))]
        up = float(rng.choice([1.0, 3.0, 0.5]))
        xin = helpers.log_softmax32(x) if fls else x
        want_loss, want_grad = oracle.transducer_loss(xin.copy(), tg, T, U, blank, fls, osf,
                                                      reduction, loss_grad=up)
        logits = _dev(xin.copy(), device).requires_grad_(True)
        loss = ot.transducer_loss(logits, _dev(tg, device), _dev(T, device), _dev(U, device), blank,
                                  fls, one_sym_per_frame=osf, reduction=reduction,
                                  defer_gradient=defer)
        (loss * up if up != 1.0 else loss).backward()
        what = dict(case=case, osf=osf, fls=fls, defer=defer, T=T.tolist(), U=U.tolist(), V=V,
                    blank=blank, reduction=reduction, up=up)
        assert np.allclose(loss.item(), want_loss, rtol=RTOL, atol=ATOL), what
        _, _, tol = helpers.oracle_tolerance(xin, tg, T, U, blank, fls, osf,
                                             scale=up / (N if reduction == "mean" else 1))
        err = np.abs(logits.grad.cpu().numpy() - want_grad)
        assert (err <= tol).all(), (what, err.max())


def test_in_place_and_aliasing_semantics(device):
    import optimized_transducer_amd as ot
    w = workloads.tiny()
    x = w.logits_numpy()
    tg, T, U = _dev(w.targets, device), _dev(w.logit_lengths, device), _dev(w.target_lengths, device)
    # logits input + requires_grad: the buffer is overwritten and IS the gradient (cpu.cc:814)
    logits = _dev(x, device).requires_grad_(True)
    ptr = logits.data_ptr()
    loss = ot.transducer_loss(logits, tg, T, U, 0, False, reduction="sum")
    assert not np.array_equal(logits.detach().cpu().numpy(), x)
    loss.backward()
    assert logits.grad.data_ptr() == ptr  # adopted, not cloned
    assert torch.equal(logits.grad, logits.detach())
    # no grad wanted: nothing is written
    logits2 = _dev(x, device)
    loss2 = ot.transducer_loss(logits2, tg, T, U, 0, False, reduction="sum")
    assert np.array_equal(logits2.cpu().numpy(), x) and not loss2.requires_grad
    assert np.allclose(loss2.item(), loss.item(), rtol=1e-6)
    # log-softmax input: the input survives, the gradient is a new tensor (cpu.cc:803)
    xl = helpers.log_softmax32(x)
    logits3 = _dev(xl, device).requires_grad_(True)
    ot.transducer_loss(logits3, tg, T, U, 0, True, reduction="sum").backward()
    assert np.array_equal(logits3.detach().cpu().numpy(), xl)
    assert logits3.grad.data_ptr() != logits3.data_ptr()
    # the extension function itself: (scores, grad) with grad aliasing logits; None without grad
    ext = ot._optimized_transducer
    l4 = _dev(x, device).requires_grad_(True)
    scores, grad = ext.compute_transducer_loss(logits=l4, targets=tg, logit_lengths=T,
                                               target_lengths=U, blank=0, from_log_softmax=False,
                                               one_sym_per_frame=False)
    assert grad.data_ptr() == l4.data_ptr() and scores.shape == (w.N,)
    assert np.allclose(-scores.sum().item(), loss.item(), rtol=1e-6)  # scores are +log-likelihoods
    scores5, grad5 = ext.compute_transducer_loss(logits=_dev(x, device), targets=tg, logit_lengths=T,
                                                 target_lengths=U, blank=0, from_log_softmax=False,
                                                 one_sym_per_frame=False)
    assert grad5 is None and torch.equal(scores5, scores)


def test_gradient_flows_into_the_network_that_made_the_logits(device):
    # logits as a non-leaf (the normal case: output of the joiner's Linear)
    import optimized_transducer_amd as ot
    w = workloads.tiny()
    x = w.logits_numpy()
    tg, T, U = _dev(w.targets, device), _dev(w.logit_lengths, device), _dev(w.target_lengths, device)
    torch.manual_seed(0)
    h = torch.randn(x.shape[0], 16, device=device)
    lin = torch.nn.Linear(16, w.V).to(device)
    loss = ot.TransducerLoss(blank=0, reduction="mean")(lin(h), tg, T, U, False)
    loss.backward()
    logits = lin(h).detach().cpu().numpy()
    _, g = oracle.transducer_loss(logits.copy(), w.targets, w.logit_lengths, w.target_lengths, 0,
                                  False, False, "mean", dtype=np.float64)
    want_w = g.T @ h.double().cpu().numpy()
    assert np.allclose(lin.weight.grad.cpu().numpy(), want_w, rtol=1e-3, atol=1e-4)
    assert np.allclose(lin.bias.grad.cpu().numpy(), g.sum(0), rtol=1e-3, atol=1e-4)


def test_argument_checks_on_the_device(device):
    import optimized_transducer_amd as ot
    w = workloads.tiny()
    x = w.logits_numpy()
    tg, T, U = _dev(w.targets, device), _dev(w.logit_lengths, device), _dev(w.target_lengths, device)

    def call(**kw):
        args = dict(logits=_dev(x, device).requires_grad_(True), targets=tg, logit_lengths=T,
                    target_lengths=U, blank=0, from_log_softmax=False)
        args.update(kw)
        return args, ot.transducer_loss(**args)

    bad_rows = _dev(x[:-1], device).requires_grad_(True)
    with pytest.raises(RuntimeError, match="Expected tensor to have size %d at dimension 0" % x.shape[0]):
        call(logits=bad_rows)
    assert np.array_equal(bad_rows.detach().cpu().numpy(), x[:-1])  # refused before any write
    big = w.targets.copy()
    big[0, 0] = w.V
    with pytest.raises(RuntimeError, match="targets.max\\(\\) vs logits.size\\(1\\) is 32 vs 32"):
        call(targets=_dev(big, device))
    with pytest.raises(RuntimeError, match="Expect 0 <= blank < logits.size\\(1\\)"):
        call(blank=w.V)
    wide = np.concatenate([w.targets, w.targets[:, :1]], 1)
    with pytest.raises(RuntimeError, match="targets.size\\(1\\) should be equal to target_lengths.max"):
        call(targets=_dev(wide, device))
    with pytest.raises(RuntimeError):  # tensors on different devices
        call(target_lengths=torch.from_numpy(w.target_lengths))
    neg = w.targets.copy()
    neg[1, 1] = -3
    with pytest.raises(RuntimeError, match="targets.min"):
        call(targets=_dev(neg, device))
    with pytest.raises(AssertionError):
        call(reduction="none")
    call()  # and the good call still works afterwards


def test_reference_test_shapes_modified_logits_vs_logsoftmax(device):
    # test_max_symbol_per_frame.py:14-65: T=107/209, U+1=51/62, V=200, rand logits,
    # targets in [1, V-1); log-softmax path == logits path, loss atol 1e-6 (relative to a
    # mean loss of a few hundred: we use rel 1e-6), grads atol 1e-4
    import optimized_transducer_amd as ot
    rng = np.random.default_rng(20220117)
    T = np.array([107, 209], np.int32)
    U = np.array([50, 61], np.int32)
    V = 200
    tg = rng.integers(1, V - 1, size=(2, 61)).astype(np.int32)
    x = rng.random((int((T * (U + 1)).sum()), V), dtype=np.float32)
    a = _dev(x, device).requires_grad_(True)
    b = _dev(x, device).requires_grad_(True)
    dtg, dT, dU = _dev(tg, device), _dev(T, device), _dev(U, device)
    la = ot.transducer_loss(b.log_softmax(-1), dtg, dT, dU, 0, True, one_sym_per_frame=True)
    lb = ot.transducer_loss(a, dtg, dT, dU, 0, False, one_sym_per_frame=True)
    la.backward()
    lb.backward()
    assert abs(la.item() - lb.item()) <= 1e-6 * abs(lb.item()) + 1e-6
    assert torch.allclose(a.grad, b.grad, atol=1e-4)
    # and both equal the oracle
    want_loss, want = oracle.transducer_loss(x.copy(), tg, T, U, 0, False, True, "mean")
    assert np.allclose(lb.item(), want_loss, rtol=RTOL, atol=ATOL)
    assert np.allclose(a.grad.cpu().numpy(), want, atol=1e-4)


def _cat_of_leaves(x, T, U, device):
    # the reference tests build logits as cat([leaf0, leaf1]) and read the leaves' grads
    sizes = (T.astype(np.int64) * (U + 1)).tolist()
    leaves = [t.clone().requires_grad_(True) for t in torch.split(_dev(x, device), sizes)]
    return leaves, torch.cat(leaves)


@pytest.mark.parametrize("reduction", ["mean", "sum"])
def test_reference_test_shapes_small(reduction, device):
    # test_cuda.py:15-70 (T=3/4, U+1=3/3, V=3; device result == CPU result) and
    # test_log_softmax.py:25-86 (T=8/5, U+1=4/5, V=3; logits path == log-softmax path,
    # atol 1e-3), targets = randint(1, V-1) = all ones, rand logits
    import optimized_transducer_amd as ot
    rng = np.random.default_rng(20211227)
    for Ts, U1s in (((3, 4), (3, 3)), ((8, 5), (4, 5))):
        T = np.array(Ts, np.int32)
        U = np.array(U1s, np.int32) - 1
        V = 3
        tg = np.ones((2, int(U.max())), np.int32)
        x = rng.random((int((T * (U + 1)).sum()), V), dtype=np.float32)
        dtg, dT, dU = _dev(tg, device), _dev(T, device), _dev(U, device)
        leaves, logits = _cat_of_leaves(x, T, U, device)
        loss = ot.transducer_loss(logits=logits, targets=dtg, logit_lengths=dT, target_lengths=dU,
                                  blank=0, from_log_softmax=False, reduction=reduction)
        loss.backward()
        leaves2, _ = _cat_of_leaves(x, T, U, device)
        loss2 = ot.transducer_loss(logits=torch.cat([l.log_softmax(-1) for l in leaves2]),
                                   targets=dtg, logit_lengths=dT, target_lengths=dU, blank=0,
                                   from_log_softmax=True, reduction=reduction)
        loss2.backward()
        want_loss, want = oracle.transducer_loss(x.copy(), tg, T, U, 0, False, False, reduction)
        assert torch.allclose(loss, loss2, atol=1e-3) and np.allclose(loss.item(), want_loss, atol=1e-6,
                                                                       rtol=1e-6)
        got = torch.cat([l.grad for l in leaves]).cpu().numpy()
        got2 = torch.cat([l.grad for l in leaves2]).cpu().numpy()
        assert np.allclose(got, got2, atol=1e-3)
        assert np.allclose(got, want, rtol=RTOL, atol=ATOL) and np.allclose(got2, want, rtol=1e-4,
                                                                             atol=ATOL)


def test_reference_test_shapes_large(device):
    # test_compute_transducer_loss.py:28-105: T in [100,1000) / [500,2000), U+1 in [100,300) /
    # [20,500), V in [5,100), rand logits, loss * 3 before backward, compared there with
    # torchaudio at atol 1e-3 (loss, first utterance) and 1e-2 (second); here with the CPU oracle
    import optimized_transducer_amd as ot
    rng = np.random.default_rng(20211230)
    T = np.array([rng.integers(100, 1000), rng.integers(500, 2000)], np.int32)
    U = np.array([rng.integers(100, 300), rng.integers(20, 500)], np.int32) - 1
    V = int(rng.integers(5, 100))
    tg = rng.integers(1, V - 1, size=(2, int(U.max()))).astype(np.int32)
    x = rng.random((int((T.astype(np.int64) * (U + 1)).sum()), V), dtype=np.float32)
    leaves, logits = _cat_of_leaves(x, T, U, device)
    loss = ot.transducer_loss(logits=logits, targets=_dev(tg, device), logit_lengths=_dev(T, device),
                              target_lengths=_dev(U, device), blank=0, from_log_softmax=False,
                              reduction="mean")
    (loss * 3).backward()
    want_loss, want = oracle.transducer_loss(x.copy(), tg, T, U, 0, False, False, "mean",
                                             loss_grad=3.0)
    assert abs(loss.item() - want_loss) <= 1e-3
    got = torch.cat([l.grad for l in leaves]).cpu().numpy()
    assert np.abs(got - want).max() <= 1e-3
    _, _, tol = helpers.oracle_tolerance(x, tg, T, U, 0, False, False, scale=1.5)
    assert (np.abs(got - want) <= tol).all(), np.abs(got - want).max()


def test_two_stream_schedule_gives_the_same_bits(device):
    # opt-in schedule: lattice kernel of one half of the batch on a second stream
    import optimized_transducer_amd as ot
    ext = ot._optimized_transducer
    w = workloads.asr_batch(N=8, V=512, scale=0.8)  # above the size threshold of the schedule
    x = w.logits_torch(device)
    tg, T, U = _dev(w.targets, device), _dev(w.logit_lengths, device), _dev(w.target_lengths, device)
    out = []
    for on in (False, True, False):
        ext.set_overlap(on)
        try:
            logits = x.clone().requires_grad_(True)
            loss = ot.transducer_loss(logits, tg, T, U, 0, False, reduction="mean")
            loss.backward()
            torch.cuda.synchronize()
            out.append((loss.detach().clone(), logits.grad.clone()))
        finally:
            ext.set_overlap(False)
    for loss, grad in out[1:]:
        assert torch.equal(loss, out[0][0]) and torch.equal(grad, out[0][1])


@pytest.mark.parametrize("fls,osf", MODES)
def test_deferred_gradient_mode(fls, osf, device):
    # defer_gradient=True: forward leaves logits alone, backward makes the one (rows, V)
    # pass with loss_grad folded in; same numbers as the reference order of operations
    import optimized_transducer_amd as ot
    w = workloads.tiny(from_log_softmax=fls, one_sym_per_frame=osf)
    x = w.logits_numpy()
    tg, T, U = _dev(w.targets, device), _dev(w.logit_lengths, device), _dev(w.target_lengths, device)

    def run(defer, upstream, reduction="mean", module=False):
        logits = _dev(x, device).requires_grad_(True)
        if module:
            m = ot.TransducerLoss(blank=w.blank, reduction=reduction)
            m.defer_gradient = defer
            loss = m(logits, tg, T, U, fls, osf)
        else:
            loss = ot.transducer_loss(logits, tg, T, U, w.blank, fls, one_sym_per_frame=osf,
                                      reduction=reduction, defer_gradient=defer)
        untouched = np.array_equal(logits.detach().cpu().numpy(), x)
        (loss * upstream).backward()
        return loss.detach(), logits, untouched

    for upstream, reduction in ((1.0, "mean"), (0.5, "sum"), (3.0, "mean")):
        l0, a, _ = run(False, upstream, reduction)
        l1, b, untouched = run(True, upstream, reduction)
        assert untouched  # forward wrote nothing
        assert torch.equal(l0, l1)
        if upstream in (1.0, 0.5):  # power-of-two factors: the two orders round alike
            assert torch.equal(a.grad, b.grad)
        assert torch.allclose(a.grad, b.grad, rtol=1e-6, atol=1e-30)
        if fls:
            assert np.array_equal(b.detach().cpu().numpy(), x)  # log-softmax input survives
            assert b.grad.data_ptr() != b.data_ptr()
        else:
            assert b.grad.data_ptr() == b.data_ptr()  # written in place, adopted by autograd
    l2, c, _ = run(True, 3.0, module=True)
    assert torch.equal(l2, l1) and torch.equal(c.grad, b.grad)
    want_loss, want = oracle.transducer_loss(x.copy(), w.targets, w.logit_lengths, w.target_lengths,
                                             w.blank, fls, osf, "mean", loss_grad=3.0)
    assert np.allclose(l2.item(), want_loss, rtol=RTOL, atol=ATOL)
    _, _, tol = helpers.oracle_tolerance(x, w.targets, w.logit_lengths, w.target_lengths, w.blank,
                                         fls, osf, scale=3.0 / w.N)
    assert (np.abs(c.grad.cpu().numpy() - want) <= tol).all()

    # no gradient wanted: nothing kept, nothing written
    plain = _dev(x, device)
    l3 = ot.transducer_loss(plain, tg, T, U, w.blank, fls, one_sym_per_frame=osf,
                            defer_gradient=True)
    assert not l3.requires_grad and torch.equal(l3, l1)
    # logits changed between forward and backward: autograd reports it
    logits = _dev(x, device).requires_grad_(True)
    h = logits * 1.0
    loss = ot.transducer_loss(h, tg, T, U, w.blank, fls, one_sym_per_frame=osf, defer_gradient=True)
    h.add_(1.0)
    with pytest.raises(RuntimeError, match="modified by an inplace operation"):
        loss.backward()


def test_side_stream_and_unaligned_views(device):
    # the launches follow torch's current stream (cuda.cu:92), and a contiguous view
    # that starts 4 bytes into an allocation (16-byte vector accesses impossible)
    # gives the same result as an aligned tensor
    import optimized_transducer_amd as ot
    rng = np.random.default_rng(77)
    T, U, tg, x = helpers.random_batch(rng, 5, 30, 12, 40)
    tg = np.where(tg == 0, 1, tg).astype(np.int32)
    dtg, dT, dU = _dev(tg, device), _dev(T, device), _dev(U, device)
    want_loss, want = oracle.transducer_loss(x.copy(), tg, T, U, 0, False, False, "sum")

    def check(loss, grad):
        assert np.allclose(loss.item(), want_loss, rtol=RTOL, atol=ATOL)
        _, _, tol = helpers.oracle_tolerance(x, tg, T, U, 0, False, False)
        assert (np.abs(grad.cpu().numpy() - want) <= tol).all()

    side = torch.cuda.Stream(device=device)
    logits = _dev(x, device).requires_grad_(True)
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        loss = ot.transducer_loss(logits, dtg, dT, dU, 0, False, reduction="sum")
        loss.backward()
    side.synchronize()
    check(loss, logits.grad)
    ref_grad = logits.grad.clone()

    flat = torch.zeros(x.size + 1, device=device)
    view = flat[1:].view(x.shape)
    view.copy_(_dev(x, device))
    assert view.data_ptr() % 16 == 4 and view.is_contiguous()
    view.requires_grad_(True)
    loss = ot.transducer_loss(view, dtg, dT, dU, 0, False, reduction="sum")
    loss.backward()
    check(loss, view.grad)
    assert torch.allclose(view.grad, ref_grad, rtol=1e-4, atol=1e-6)  # scalar vs vector code path
    assert flat[0].item() == 0  # nothing written in front of the view

    # log-softmax input on the view: gradient is a fresh (aligned) tensor
    xl = helpers.log_softmax32(x)
    view2 = torch.zeros(x.size + 1, device=device)[1:].view(x.shape)
    view2.copy_(_dev(xl, device))
    view2.requires_grad_(True)
    a = _dev(xl, device).requires_grad_(True)
    ot.transducer_loss(view2, dtg, dT, dU, 0, True, reduction="sum").backward()
    ot.transducer_loss(a, dtg, dT, dU, 0, True, reduction="sum").backward()
    assert torch.equal(view2.grad, a.grad)


def test_whole_path_replays_from_a_hip_graph(device):
    # ot_transducer_loss neither allocates nor synchronises nor clears memory with a memset,
    # so a caller can capture it once and replay it; every replay is checked against the
    # eager result for the data that is in the buffers at that moment
    import ctypes
    rng = np.random.default_rng(41)
    T, U, tg, x0 = helpers.random_batch(rng, 6, 40, 70, 48)   # two waves per lattice
    tg = np.where(tg == 0, 1, tg).astype(np.int32)
    N, rows, V = len(T), x0.shape[0], x0.shape[1]
    dT, dU, dtg = _dev(T, device), _dev(U, device), _dev(tg, device)
    L = cabi.lib()
    nbytes = L.ot_workspace_bytes(ctypes.c_int32(N), ctypes.c_int64(rows))
    ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
    logits = torch.empty((rows, V), device=device)
    scores = torch.empty(N, device=device)
    status = torch.zeros(64, dtype=torch.uint8, device=device)

    def launch():
        cabi.check(L.ot_transducer_loss(
            cabi.ptr(logits), cabi.ptr(dtg), cabi.ptr(dT), cabi.ptr(dU), ctypes.c_int32(N),
            ctypes.c_int32(tg.shape[1]), ctypes.c_int64(rows), ctypes.c_int32(V), ctypes.c_int32(0),
            ctypes.c_int32(0), ctypes.c_int32(0), ctypes.c_int32(int(U.max()) + 1),
            ctypes.c_float(0.5), cabi.ptr(ws), ctypes.c_size_t(nbytes), cabi.ptr(scores),
            cabi.ptr(logits), cabi.ptr(status), cabi.stream()))

    inputs = [x0] + [rng.standard_normal(x0.shape).astype(np.float32) for _ in range(3)]
    eager = []
    for xi in inputs:
        logits.copy_(_dev(xi, device))
        launch()
        torch.cuda.synchronize()
        eager.append((scores.clone(), logits.clone()))

    graph = torch.cuda.CUDAGraph()
    logits.copy_(_dev(inputs[0], device))
    torch.cuda.synchronize()
    with torch.cuda.graph(graph):
        launch()
    for k in (1, 2, 3, 0, 2):
        logits.copy_(_dev(inputs[k], device))   # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(scores, eager[k][0]) and torch.equal(logits, eager[k][1]), k


# ------------------------------------------------------------------ full sizes
FULL = [
    ("asr", lambda: workloads.asr_batch()),
    ("asr_logsoftmax_modified", lambda: workloads.asr_batch_logsoftmax_modified()),
    ("largevocab", lambda: workloads.large_vocab()),
    ("ragged", lambda: workloads.ragged()),
    ("ragged_modified", lambda: workloads.ragged(one_sym_per_frame=True)),
    # more than 2^31 logits: element offsets need 64 bits (the reference's CUDA kernels
    # index with int there, kernels.cu:49)
    ("beyond_int32", lambda: workloads.beyond_int32()),
]


# gradient against the fp32 oracle: every entry within rel 1e-5 / abs 1e-5 ...
PLAIN_TOLERANCE = ("asr_logsoftmax_modified", "ragged", "ragged_modified")
# ... or at least this share of the entries, none further than NOISE_UNITS_MAX roundings of
# its exponent
NOISE_LIMITED = {"asr": 0.9999, "largevocab": 0.999999}
NOISE_UNITS_MAX = helpers.NOISE_K  # measured: 1.0 to 2.4 over the six workloads


@pytest.mark.parametrize("api", ["cabi", "python"])
@pytest.mark.parametrize("name,make", FULL, ids=[f[0] for f in FULL])
def test_full_size_workloads(name, make, api, device):
    # api "cabi": ot_transducer_loss (plain lattice launch, exact max_u1);
    # api "python": the shipped entry point, whose extension launches the lattice kernel
    # before its host-side validation, guarded on the device, with targets.size(1) + 1 columns
    import optimized_transducer_amd as ot
    from optimized_transducer_amd import _optimized_transducer as ext
    w = make()
    fls, osf = w.from_log_softmax, w.one_sym_per_frame
    T, U, tg = w.logit_lengths, w.target_lengths, w.targets
    x = w.logits_torch(device)
    dT, dU, dtg = _dev(T, device), _dev(U, device), _dev(tg, device)
    max_u1 = int(U.max()) + 1
    splits, total = oracle.row_splits(T, U)
    assert total == x.shape[0]

    # oracle on a slice: utterances are independent, so the rows of any subset of
    # utterances must equal the oracle run on that subset alone.  Take the longest
    # lattice, the first and the last utterance, and every degenerate one.
    pick = sorted(set([int(np.argmax(T + U)), 0, len(T) - 1]
                      + [int(i) for i in np.where((T == 1) | (U == 0))[0][:4]]))
    huge = x.numel() > 2 ** 31
    if huge:  # the first and the last utterance only: the last one straddles element 2^31
        pick = [0, len(T) - 1]
        assert int(splits[-2]) * w.V < 2 ** 31 < int(splits[-1]) * w.V
    xs = torch.cat([x[splits[b]:splits[b + 1]] for b in pick]).cpu().numpy()
    tgs = np.ascontiguousarray(tg[pick][:, :max(int(U[pick].max()), 0)])
    # the workload's own reduction: "mean" multiplies the gradient by 1/N (transducer_loss.py:150)
    scale = 1.0 / len(T) if w.reduction == "mean" else 1.0
    s32, g32, unit = helpers.oracle_noise_unit(xs, tgs, T[pick], U[pick], w.blank, fls, osf)
    g32 *= np.float32(scale)
    unit *= np.float32(scale)
    plain = ATOL + RTOL * np.abs(g32)
    # the absolute part shrinks with the scale, so that the bound keeps its power for "mean"
    tol = min(scale, 1.0) * ATOL + RTOL * np.abs(g32) + helpers.NOISE_K * unit
    if huge:  # no float64 run at this size (memory, time)
        s64, g64 = s32, None
    else:
        s64, g64 = oracle.compute_transducer_loss(xs.copy(), tgs, T[pick], U[pick], w.blank, fls,
                                                  osf, dtype=np.float64)
        g64 *= scale

    work = x.clone()
    if api == "cabi":
        scores, grad, st = cabi.transducer_loss(work, dtg, dT, dU, w.blank, fls, osf, max_u1,
                                                grad_scale=scale, grad=("new" if fls else "inplace"))
        assert st.sum_tu == total and st.targets_max == tg.max() and st.target_len_max == U.max()
    else:
        scores, _ = ext.compute_transducer_loss(
            logits=x.clone(), targets=dtg, logit_lengths=dT, target_lengths=dU, blank=w.blank,
            from_log_softmax=fls, one_sym_per_frame=osf)
        work.requires_grad_(True)
        loss = ot.transducer_loss(work, dtg, dT, dU, w.blank, fls, osf, w.reduction)
        loss.backward()
        grad = work.grad
        work = work.detach()
        # loss = -sum or -mean of the per-utterance log-likelihoods (transducer_loss.py:145-147)
        want_loss = -scale * float(scores.double().sum())
        assert abs(loss.item() - want_loss) <= 1e-6 * abs(want_loss), (loss.item(), want_loss)
    scores_np = scores.cpu().numpy()
    assert np.isfinite(scores_np).all()

    got_s = scores_np[pick]
    got_g = torch.cat([grad[splits[b]:splits[b + 1]] for b in pick]).cpu().numpy()
    assert np.allclose(got_s, s32, rtol=RTOL, atol=ATOL), np.abs(got_s - s32).max()
    err = np.abs(got_g - g32)
    assert (err <= tol).all(), (err.max(), (err / tol).max())
    # The measured record per workload, pinned.  With the 1/N of their "mean" reduction the
    # log-softmax workload, the large vocabulary and the ragged batches meet the plain
    # rel 1e-5 / abs 1e-5 on every entry or all but a few in 10^7; on the long lattices of the
    # "sum" workload, with |log-likelihood| of 2-3 thousand and no 1/N, a few entries in 10^5
    # differ by some roundings of their exponent (eps * |log-likelihood| * the entry's
    # exponentials; entries with a unit below 1e-30 are denormal results, which the GPU
    # flushes to zero).
    within = err <= plain
    ok = unit > 1e-30
    units = (err[ok] / unit[ok]).max() if ok.any() else 0.0
    print("parity %s/%s (%s): max |err| = %.3g, share within rel/abs 1e-5 = %.8f, largest error = %.2f "
          "noise units" % (name, api, w.reduction, err.max(), within.mean(), units))
    if name in PLAIN_TOLERANCE:
        assert within.all(), (name, err.max(), 1.0 - within.mean())
    elif name in NOISE_LIMITED:
        assert within.mean() >= NOISE_LIMITED[name] and units <= NOISE_UNITS_MAX, (name, within.mean(), units)
    del within, ok
    # float64 arbiter: no further from the exact gradient than the fp32 reference arithmetic
    if g64 is not None:
        assert np.abs(got_g - g64).max() <= 2 * np.abs(g32 - g64).max() + 1e-6 * scale
    del xs, g32, g64, got_g

    # size-independent properties over the whole batch
    if fls:
        occ = -grad.sum(1) / scale  # node occupancies
        assert (occ >= -1e-6).all()
        assert (occ <= 1 + 64 * helpers.EPS32 * np.abs(scores_np).max()).all()
        # occupancies of one frame (modified) / all frames (standard) add up per utterance
        per_utt = np.add.reduceat(occ.double().cpu().numpy(), splits[:-1])
        want = T.astype(np.float64) if osf else (T + U).astype(np.float64)
        assert np.allclose(per_utt, want, rtol=5e-3)
        assert torch.equal(work, x)  # log-softmax input is never written
    else:
        rs = grad.sum(1).abs().max().item()
        # rows of d loss / d logits sum to zero, up to the fp32 noise of exponents of size |loss|
        assert rs < 1e-5 + 4 * helpers.EPS32 * np.abs(scores_np).max(), rs
        assert grad.data_ptr() == work.data_ptr()
    # entries are probabilities up to the fp32 noise of exp(arguments of size |loss|)
    assert grad.abs().max().item() <= 1 + 64 * helpers.EPS32 * np.abs(scores_np).max()

    # same bits on a second run (no atomics, no data races)
    work2 = x.clone()
    scores2, grad2, _ = cabi.transducer_loss(work2, dtg, dT, dU, w.blank, fls, osf, max_u1,
                                             grad_scale=scale, grad=("new" if fls else "inplace"))
    assert torch.equal(scores2, scores) and torch.equal(grad2, grad)
