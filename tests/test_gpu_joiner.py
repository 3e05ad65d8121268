"""GPU parity of the packed joiner input (the data format on the input side of
the loss): C ABI and Python entry point against the numpy restatement of the
reference's README.md:166-177 recipe and the closed-form gradient.

Tolerances.  Forward: one addition (and one tanh); |delta| <= 1e-6 + 1e-6 |ref|
for tanh, bit-exact without activation.  Gradient: each output is a sum of up to
max(T, U+1) float32 terms g * (1 - tanh^2); the bound is 1e-5 relative plus 1e-6
times the sum of |g| over the same cells (a float32 sum in any order errs by at
most eps times that sum times the number of terms, and 1 - tanh^2 carries an
absolute error of about eps where tanh is close to 1)."""
import zlib

import numpy as np
import pytest
import torch

import cabi
from oracle import oracle

pytestmark = pytest.mark.gpu

ACT = {None: 0, "tanh": 1, "relu": 2}


def _dev(a, device):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def _batch(rng, N, Tm, U1m, D, pad_t=0, pad_u=0):
    T = rng.integers(1, Tm + 1, size=N).astype(np.int32)
    U = rng.integers(0, U1m, size=N).astype(np.int32)
    T[0], U[0] = 1, 0
    if N > 1:
        T[1], U[1] = Tm, U1m - 1
    if N > 2:
        T[2], U[2] = 1, U1m - 1
    enc = rng.standard_normal((N, Tm + pad_t, D)).astype(np.float32)
    dec = rng.standard_normal((N, U1m + pad_u, D)).astype(np.float32)
    return T, U, enc, dec


CASES = [  # name, N, Tmax, U1max, D, pad_t, pad_u
    ("small_D8", 4, 9, 5, 8, 0, 0),
    ("D7_scalar_path", 5, 20, 6, 7, 2, 1),
    ("D64_one_slab", 6, 37, 19, 64, 0, 3),
    ("D100_partial_slab", 3, 50, 33, 100, 5, 0),
    ("D512_long_T", 3, 130, 40, 512, 0, 0),
    ("many_utts", 70, 6, 4, 16, 1, 1),
]


@pytest.mark.parametrize("activation", [None, "tanh", "relu"])
@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_pack_and_unpack_through_the_c_abi(case, activation, device):
    _, N, Tm, U1m, D, pad_t, pad_u = case
    rng = np.random.default_rng(zlib.crc32(case[0].encode()))
    T, U, enc, dec = _batch(rng, N, Tm, U1m, D, pad_t, pad_u)
    dT, dU, denc, ddec = _dev(T, device), _dev(U, device), _dev(enc, device), _dev(dec, device)
    splits, st = cabi.row_splits(dT, dU, torch.zeros((N, 0), dtype=torch.int32, device=device))
    rows = int(st.sum_tu)
    want = oracle.pack_joiner(enc, dec, T, U, activation)
    assert want.shape == (rows, D)

    out = cabi.joiner_pack(denc, ddec, dT, dU, splits, rows, ACT[activation]).cpu().numpy()
    # without activation every entry is one float32 addition: bit exact, which also pins the
    # row -> (utterance, frame, position) arithmetic
    if activation in (None, "relu"):  # (the larger of that sum and 0 is exact as well)
        assert (out == want).all()
    else:
        assert np.allclose(out, want, rtol=1e-6, atol=1e-6), np.abs(out - want).max()

    g = rng.standard_normal((rows, D)).astype(np.float32)
    ge, gd = cabi.joiner_unpack_grad(_dev(g, device), denc, ddec, dT, dU, splits, ACT[activation])
    ge, gd = ge.cpu().numpy(), gd.cpu().numpy()
    we, wd, ae, ad = oracle.pack_joiner_backward(g, enc, dec, T, U, activation)
    assert not np.isnan(ge).any() and not np.isnan(gd).any()  # written in full, padding included
    assert (np.abs(ge - we) <= 1e-5 * np.abs(we) + 1e-6 * ae + 1e-30).all(), np.abs(ge - we).max()
    assert (np.abs(gd - wd) <= 1e-5 * np.abs(wd) + 1e-6 * ad + 1e-30).all(), np.abs(gd - wd).max()
    for b in range(N):  # padding is exactly zero
        assert (ge[b, T[b]:] == 0).all() and (gd[b, U[b] + 1:] == 0).all()
    # fixed summation order: same bits on a second run
    ge2, gd2 = cabi.joiner_unpack_grad(_dev(g, device), denc, ddec, dT, dU, splits, ACT[activation])
    assert (ge2.cpu().numpy() == ge).all() and (gd2.cpu().numpy() == gd).all()


def test_tanh_accuracy_over_the_whole_range(device):
    # enc = x, dec = 0: out = tanh(x); relative error of a few ulp everywhere (8 allowed)
    x = np.concatenate([np.linspace(-12, 12, 4001), np.array([0.0, 1e-8, -1e-8, 1e-4, 0.2499, 0.25,
                       0.2501, 20.0, -20.0, 100.0, -100.0])]).astype(np.float32)
    n = x.size
    pad = (-n) % 4
    x = np.concatenate([x, np.zeros(pad, np.float32)])
    enc = x.reshape(1, 1, -1)
    dec = np.zeros_like(enc)
    T, U = np.array([1], np.int32), np.array([0], np.int32)
    dT, dU = _dev(T, device), _dev(U, device)
    splits, _ = cabi.row_splits(dT, dU, torch.zeros((1, 0), dtype=torch.int32, device=device))
    out = cabi.joiner_pack(_dev(enc, device), _dev(dec, device), dT, dU, splits, 1, 1).cpu().numpy()[0]
    want = np.tanh(x.astype(np.float64))
    assert (np.abs(out - want) <= 8 * np.spacing(np.abs(want).astype(np.float32)) + 1e-45).all()
    assert (np.sign(out) == np.sign(want)).all() and np.abs(out).max() <= 1.0


@pytest.mark.parametrize("activation", [None, "tanh", "relu"])
def test_python_entry_point_and_autograd(activation, device):
    import optimized_transducer_amd as ot
    rng = np.random.default_rng(3)
    T, U, enc, dec = _batch(rng, 6, 25, 9, 48, pad_t=3, pad_u=2)
    dT, dU = _dev(T, device), _dev(U, device)
    te = _dev(enc, device).requires_grad_(True)
    td = _dev(dec, device).requires_grad_(True)
    x = ot.pack_joiner(te, td, dT, dU, activation=activation)
    want = oracle.pack_joiner(enc, dec, T, U, activation)
    assert x.shape == want.shape and np.allclose(x.detach().cpu().numpy(), want, rtol=1e-6, atol=1e-6)
    # the README.md:166-177 recipe in torch on the device gives the same numbers and gradients
    re = _dev(enc, device).requires_grad_(True)
    rd = _dev(dec, device).requires_grad_(True)
    parts = [(re[i, :T[i]].unsqueeze(1) + rd[i, :U[i] + 1].unsqueeze(0)).reshape(-1, 48)
             for i in range(6)]
    y = torch.cat(parts)
    if activation == "tanh":
        y = torch.tanh(y)
    if activation == "relu":
        y = torch.relu(y)
    assert torch.allclose(x, y, rtol=1e-6, atol=1e-6)
    g = torch.randn_like(x)
    x.backward(g)
    y.backward(g)
    assert torch.allclose(te.grad, re.grad, rtol=1e-4, atol=1e-5)
    assert torch.allclose(td.grad, rd.grad, rtol=1e-4, atol=1e-5)

    # end to end: joiner -> Linear -> transducer loss, gradients reach encoder and decoder
    torch.manual_seed(0)
    lin = torch.nn.Linear(48, 20).to(device)
    tg = _dev(rng.integers(1, 20, size=(6, int(U.max()))).astype(np.int32), device)
    te.grad = td.grad = None
    loss = ot.transducer_loss(lin(ot.pack_joiner(te, td, dT, dU, activation="tanh")), tg, dT, dU, 0,
                              False, reduction="sum")
    loss.backward()
    assert torch.isfinite(loss) and te.grad.abs().sum() > 0 and td.grad.abs().sum() > 0
    assert (te.grad[0, T[0]:] == 0).all()


def test_argument_checks(device):
    import optimized_transducer_amd as ot
    rng = np.random.default_rng(4)
    T, U, enc, dec = _batch(rng, 3, 8, 4, 8)
    dT, dU, de, dd = _dev(T, device), _dev(U, device), _dev(enc, device), _dev(dec, device)
    with pytest.raises(RuntimeError, match="logit_lengths.max"):
        ot.pack_joiner(de[:, :5].contiguous(), dd, dT, dU)
    with pytest.raises(RuntimeError, match="target_lengths.max"):
        ot.pack_joiner(de, dd[:, :2].contiguous(), dT, dU)
    with pytest.raises(RuntimeError, match="last dimension"):
        ot.pack_joiner(de, dd[:, :, :4].contiguous(), dT, dU)
    with pytest.raises(RuntimeError, match="activation"):
        ot.pack_joiner(de, dd, dT, dU, activation="gelu")
    with pytest.raises(RuntimeError, match="no CPU"):
        ot.pack_joiner(torch.from_numpy(enc), torch.from_numpy(dec), torch.from_numpy(T),
                       torch.from_numpy(U))
    bad = T.copy()
    bad[1] = 0
    with pytest.raises(RuntimeError, match="logit_lengths >= 1"):
        ot.pack_joiner(de, dd, _dev(bad, device), dU)
    assert ot.pack_joiner(de, dd, dT, dU).shape == (int((T * (U + 1)).sum()), 8)


HALF_CASES = [c for c in CASES if c[4] % 8 == 0]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
@pytest.mark.parametrize("activation", [None, "tanh", "relu"])
@pytest.mark.parametrize("case", HALF_CASES, ids=[c[0] for c in HALF_CASES])
def test_pack_with_16_bit_output(case, activation, dtype, device):
    """float32 arithmetic, one rounding to nearest even: without activation the float32
    kernel's output rounded by torch gives the same bits; the tanh of this kernel is accurate
    to the 16-bit result, so it may differ from that by one unit in the last place."""
    _, N, Tm, U1m, D, pad_t, pad_u = case
    rng = np.random.default_rng(zlib.crc32(case[0].encode()) + 1)
    T, U, enc, dec = _batch(rng, N, Tm, U1m, D, pad_t, pad_u)
    dT, dU, denc, ddec = _dev(T, device), _dev(U, device), _dev(enc, device), _dev(dec, device)
    splits, st = cabi.row_splits(dT, dU, torch.zeros((N, 0), dtype=torch.int32, device=device))
    rows = int(st.sum_tu)
    got = cabi.joiner_pack_half(denc, ddec, dT, dU, splits, rows, ACT[activation], dtype)
    full = cabi.joiner_pack(denc, ddec, dT, dU, splits, rows, ACT[activation])
    assert got.dtype == dtype
    if activation in (None, "relu"):
        assert torch.equal(got, full.to(dtype))
    else:
        one = 2.0 ** -10 if dtype == torch.float16 else 2.0 ** -7   # one unit in the last place
        d = (got.float() - full.to(dtype).float()).abs()
        assert (d <= one * full.abs() + 1e-7).all()
        assert (d > 0).float().mean() < 0.02   # and rarely differs at all
    want = torch.from_numpy(oracle.pack_joiner(enc, dec, T, U, activation)).to(dtype)
    ulp = 2.0 ** -11 if dtype == torch.float16 else 2.0 ** -8
    diff = (got.float().cpu() - want.float()).abs()
    assert (diff <= 2 * ulp * want.float().abs() + 1e-6).all()


def test_pack_16_bit_output_in_the_python_pipeline(device):
    import optimized_transducer_amd as ot
    rng = np.random.default_rng(8)
    T, U, enc, dec = _batch(rng, 5, 14, 6, 64)
    dT, dU = _dev(T, device), _dev(U, device)
    te = _dev(enc, device).requires_grad_(True)
    td = _dev(dec, device).requires_grad_(True)
    x = ot.pack_joiner(te, td, dT, dU, activation="tanh", out_dtype=torch.bfloat16)
    ref = ot.pack_joiner(te.detach(), td.detach(), dT, dU, activation="tanh")
    assert x.dtype == torch.bfloat16
    assert ((x.float() - ref).abs() <= 2.0 ** -7 * ref.abs() + 1e-7).all()
    # joiner -> 16-bit projection with the denominators -> loss; gradients reach both inputs
    torch.manual_seed(1)
    w = (torch.randn(30, 64, device=device) / 8).to(torch.bfloat16).requires_grad_(True)
    b = torch.randn(30, device=device, requires_grad=True)
    tg = _dev(rng.integers(1, 30, size=(5, int(U.max()))).astype(np.int32), device)
    logits, den = ot.project_joiner(x, w, b)
    loss = ot.transducer_loss(logits, tg, dT, dU, 0, False, reduction="sum", denominators=den)
    loss.backward()
    # the same through float32 tensors and torch's own ops
    re = _dev(enc, device).requires_grad_(True)
    rd = _dev(dec, device).requires_grad_(True)
    y = ot.pack_joiner(re, rd, dT, dU, activation="tanh")
    l2 = ot.transducer_loss(torch.nn.functional.linear(y, w.detach().float(), b.detach()), tg, dT, dU, 0,
                            False, reduction="sum")
    l2.backward()
    assert abs(loss.item() - l2.item()) <= 0.02 * abs(l2.item())
    for a, r in ((te.grad, re.grad), (td.grad, rd.grad)):
        assert (a - r).abs().max() <= 0.05 * r.abs().max() + 1e-4
    with pytest.raises(RuntimeError, match="multiple of 8"):
        ot.pack_joiner(torch.zeros(1, 2, 12, device=device), torch.zeros(1, 2, 12, device=device),
                       torch.ones(1, dtype=torch.int32, device=device),
                       torch.ones(1, dtype=torch.int32, device=device), out_dtype=torch.float16)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
@pytest.mark.parametrize("activation", [None, "tanh", "relu"])
@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_unpack_of_a_16_bit_gradient(case, activation, dtype, device):
    """The incoming gradient is widened (exactly) inside the kernel, for 4 columns per thread and
    for the scalar path; the sums are taken in another order than in the float32 kernel (wider
    slabs), so the oracle's bound applies, not bit equality."""
    _, N, Tm, U1m, D, pad_t, pad_u = case
    rng = np.random.default_rng(zlib.crc32(case[0].encode()) + 2)
    T, U, enc, dec = _batch(rng, N, Tm, U1m, D, pad_t, pad_u)
    dT, dU, denc, ddec = _dev(T, device), _dev(U, device), _dev(enc, device), _dev(dec, device)
    splits, st = cabi.row_splits(dT, dU, torch.zeros((N, 0), dtype=torch.int32, device=device))
    g = torch.from_numpy(rng.standard_normal((int(st.sum_tu), D)).astype(np.float32)).to(dtype).to(device)
    ge, gd = cabi.joiner_unpack_grad(g, denc, ddec, dT, dU, splits, ACT[activation])
    ge, gd = ge.cpu().numpy(), gd.cpu().numpy()
    we, wd, ae, ad = oracle.pack_joiner_backward(g.float().cpu().numpy(), enc, dec, T, U, activation)
    assert not np.isnan(ge).any() and not np.isnan(gd).any()
    assert (np.abs(ge - we) <= 1e-5 * np.abs(we) + 1e-6 * ae + 1e-30).all(), np.abs(ge - we).max()
    assert (np.abs(gd - wd) <= 1e-5 * np.abs(wd) + 1e-6 * ad + 1e-30).all(), np.abs(gd - wd).max()
    for b in range(N):  # padding is exactly zero
        assert (ge[b, T[b]:] == 0).all() and (gd[b, U[b] + 1:] == 0).all()
    ge2, gd2 = cabi.joiner_unpack_grad(g, denc, ddec, dT, dU, splits, ACT[activation])
    assert (ge2.cpu().numpy() == ge).all() and (gd2.cpu().numpy() == gd).all()  # fixed order
