"""The drop-in surface on a GPU box: code written against the reference package runs
with the import line unchanged.  The cases follow the reference's own test scripts
(optimized_transducer/python/tests/test_cuda.py:15-70, test_log_softmax.py:24-97,
test_max_symbol_per_frame.py): same shapes, same call sequence, CPU tensors first and
device tensors second, compared with each other and with the CPU oracle."""
import numpy as np
import pytest
import torch

import helpers
from helpers import ATOL, RTOL
from oracle import oracle

pytestmark = pytest.mark.gpu


def _two_utterances(seed, T1, T2, U1, U2, V, device):
    # test_cuda.py:15-36 / test_log_softmax.py:26-47: a padded (2, T, U, V) tensor cut
    # into two leaves; U1, U2 count the blank-prepended targets, i.e. they are U + 1
    g = torch.Generator().manual_seed(seed)
    logits = torch.rand(2, max(T1, T2), max(U1, U2), V, dtype=torch.float32, generator=g)
    targets = torch.randint(low=1, high=V - 1, size=(2, max(U1, U2) - 1), dtype=torch.int32,
                            generator=g)
    logit_lengths = torch.tensor([T1, T2], dtype=torch.int32)
    target_lengths = torch.tensor([U1, U2], dtype=torch.int32) - 1
    l0 = logits[0, :T1, :U1, :].reshape(-1, V).to(device).requires_grad_(True)
    l1 = logits[1, :T2, :U2, :].reshape(-1, V).to(device).requires_grad_(True)
    return l0, l1, targets.to(device), logit_lengths.to(device), target_lengths.to(device)


@pytest.mark.parametrize("osf", [False, True])
@pytest.mark.parametrize("reduction", ["mean", "sum"])
@pytest.mark.parametrize("fls", [False, True])
def test_cpu_tensors_and_device_tensors_give_the_same_numbers(fls, reduction, osf, device):
    import optimized_transducer  # the reference's import line

    results = []
    for dev in (torch.device("cpu"), device):
        # shapes of test_cuda.py (T 3/4, U+1 3/3, V 3) and of test_log_softmax.py (8/5, 4/5, 3)
        for shape in ((3, 4, 3, 3, 3), (8, 5, 4, 5, 3), (40, 31, 12, 7, 23)):
            l0, l1, tg, T, U = _two_utterances(20211227, *shape, dev)
            logits = torch.cat([l0, l1])
            if fls:
                logits = logits.log_softmax(dim=-1)
            before = logits.detach().clone()
            loss = optimized_transducer.transducer_loss(
                logits=logits, targets=tg, logit_lengths=T, target_lengths=U, blank=0,
                from_log_softmax=fls, one_sym_per_frame=osf, reduction=reduction)
            assert loss.device == logits.device and loss.dim() == 0
            # logits input: the gradient overwrites the caller's buffer, on either device
            # (cpu.cc:814, cuda.cu:449); log-softmax input stays as it was (cpu.cc:803)
            assert torch.equal(logits.detach(), before) == fls
            (loss * 3).backward()  # test_compute_transducer_loss.py:92
            results.append((dev.type, shape, loss.detach().cpu(), l0.grad.cpu(), l1.grad.cpu(),
                            before.cpu(), tg.cpu(), T.cpu(), U.cpu()))
    half = len(results) // 2
    for cpu, gpu in zip(results[:half], results[half:]):
        assert cpu[1] == gpu[1] and cpu[0] == "cpu" and gpu[0] == "cuda"
        if not fls:
            # both run the same kernels on the same values: the same bits
            assert torch.equal(cpu[2], gpu[2])
            assert torch.equal(cpu[3], gpu[3]) and torch.equal(cpu[4], gpu[4])
        else:
            # torch's own log_softmax (and its backward) in front differs between host and device
            # (inputs that differ in the last bit, amplified by the lattice like any other rounding)
            assert torch.allclose(cpu[2], gpu[2], rtol=1e-6)
            assert torch.allclose(cpu[3], gpu[3], rtol=1e-4, atol=1e-5)
            assert torch.allclose(cpu[4], gpu[4], rtol=1e-4, atol=1e-5)
        # ... and they are the reference's numbers
        _, _, loss, g0, g1, x, tg, T, U = cpu
        want_loss, want = oracle.transducer_loss(x.numpy().copy(), tg.numpy(), T.numpy(), U.numpy(),
                                                 0, fls, osf, reduction, loss_grad=3.0)
        assert np.allclose(loss.item(), want_loss, rtol=RTOL, atol=ATOL)
        if fls:  # the oracle's gradient is w.r.t. the log-softmax values x: chain rule to the leaves
            w = torch.from_numpy(want)
            want = (w - x.exp() * w.sum(1, keepdim=True)).numpy()
        got = torch.cat([g0, g1]).numpy()
        assert np.allclose(got, want, rtol=1e-4, atol=1e-5), np.abs(got - want).max()


def test_reference_module_paths_and_module_form(device):
    # test_compute_transducer_loss.py:55-70 builds the module form; the reference's class
    # cannot be called (it never initialises nn.Module), its functional form is what runs
    import optimized_transducer
    from optimized_transducer.transducer_loss import TransducerLoss, transducer_loss
    assert transducer_loss is optimized_transducer.transducer_loss
    l0, l1, tg, T, U = _two_utterances(7, 6, 9, 3, 5, 11, device)
    a = torch.cat([l0, l1])
    b = a.detach().clone().requires_grad_(True)
    la = transducer_loss(a, tg, T, U, 0, False)
    lb = TransducerLoss(blank=0)(b, tg, T, U, from_log_softmax=False)
    assert torch.equal(la, lb)


def test_padding_of_minus_one_is_accepted_and_negative_ids_that_are_read_are_not(device):
    # the reference reads targets[b][u] only for u < U_b (kernels.cu:49-50, cpu.cc:80-86) and
    # checks targets.max() alone (transducer-loss.cc:53), so -1 padding works there
    import optimized_transducer_amd as ot
    rng = np.random.default_rng(5)
    T, U, tg, x = helpers.random_batch(rng, 5, 20, 9, 17)
    padded = tg.copy()
    for b in range(len(U)):
        padded[b, U[b]:] = -1
    assert (padded == -1).any()
    dT, dU = torch.from_numpy(T).to(device), torch.from_numpy(U).to(device)

    def run(t):
        logits = torch.from_numpy(x).to(device).requires_grad_(True)
        loss = ot.transducer_loss(logits, torch.from_numpy(t).to(device), dT, dU, 0, False)
        loss.backward()
        return loss, logits.grad

    l1, g1 = run(tg)
    l2, g2 = run(padded)
    assert torch.equal(l1, l2) and torch.equal(g1, g2)
    bad = padded.copy()
    bad[int(np.argmax(U)), 0] = -1
    with pytest.raises(RuntimeError, match="Expect targets >= 0"):
        run(bad)
    # the same through CPU tensors
    with pytest.raises(RuntimeError, match="Expect targets >= 0"):
        ot.transducer_loss(torch.from_numpy(x), torch.from_numpy(bad), torch.from_numpy(T),
                           torch.from_numpy(U), 0, False)


@pytest.mark.parametrize("fls", [False, True])
def test_second_backward_through_the_same_graph(fls, device):
    # the reference's backward returns ctx.grad.mul_(loss_grad) every time it is called
    # (transducer_loss.py:158-170), so with retain_graph=True a leaf accumulates
    # g * w1 + g * w1 * w2.  Here the first backward hands the buffer itself to autograd
    # (no (rows, V) copy) and only a further backward copies.
    import optimized_transducer_amd as ot
    rng = np.random.default_rng(6)
    T, U, tg, x = helpers.random_batch(rng, 3, 10, 4, 9)
    if fls:
        x = helpers.log_softmax32(x)
    _, g = oracle.compute_transducer_loss(x.copy(), tg, T, U, 0, fls, False)
    g = g / len(T)
    logits = torch.from_numpy(x).to(device).requires_grad_(True)
    loss = ot.transducer_loss(logits, torch.from_numpy(tg).to(device), torch.from_numpy(T).to(device),
                              torch.from_numpy(U).to(device), 0, fls)
    (loss * 0.5).backward(retain_graph=True)
    first = logits.grad
    if not fls:
        assert first.data_ptr() == logits.data_ptr()   # adopted, not cloned
    assert np.allclose(first.cpu().numpy(), 0.5 * g, rtol=RTOL, atol=ATOL)
    (loss * 3.0).backward(retain_graph=True)
    assert logits.grad.data_ptr() == first.data_ptr()   # accumulated in place
    assert np.allclose(logits.grad.cpu().numpy(), (0.5 + 0.5 * 3.0) * g, rtol=RTOL, atol=2e-5)
    # a buffer that was changed in place since it was handed over cannot be returned again
    logits.grad = None
    loss.backward(retain_graph=True)
    logits.grad.zero_()
    with pytest.raises(RuntimeError, match="modified in place"):
        loss.backward()


@pytest.mark.parametrize("osf", [False, True])
@pytest.mark.parametrize("fls", [False, True])
def test_targets_longer_than_one_lattice_tile(fls, osf, device):
    # U + 1 = 1201 and 1101 columns: two tiles of the lattice kernel; the reference's CPU path,
    # the parity target, loops over any U (cpu.cc:162-244, 319-382)
    import optimized_transducer_amd as ot
    rng = np.random.default_rng(1200 + 2 * fls + osf)
    V = 8
    T = np.array([1300, 37, 1250], np.int32)
    U = np.array([1200, 5, 1100], np.int32)
    tg = rng.integers(1, V, size=(3, 1200)).astype(np.int32)
    rows = int((T.astype(np.int64) * (U + 1)).sum())
    x = rng.standard_normal((rows, V)).astype(np.float32)
    if fls:
        x = helpers.log_softmax32(x)
    s, g, tol = helpers.oracle_tolerance(x, tg, T, U, 0, fls, osf)
    logits = torch.from_numpy(x).to(device).requires_grad_(True)
    loss = ot.transducer_loss(logits, torch.from_numpy(tg).to(device), torch.from_numpy(T).to(device),
                              torch.from_numpy(U).to(device), 0, fls, osf, "sum")
    loss.backward()
    assert np.isfinite(s).all()
    assert np.allclose(loss.item(), -s.sum(dtype=np.float64), rtol=RTOL, atol=ATOL)
    err = np.abs(logits.grad.cpu().numpy() - g)
    assert (err <= tol).all(), (err.max(), (err / tol).max())
