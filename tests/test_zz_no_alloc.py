"""ot_transducer_loss_static, the entry point that allocates nothing, against
ot_transducer_loss (same kernels, caller-provided workspace) through the C ABI.

Both run the same launches on the same inputs, so scores, gradient and batch
facts must agree bit for bit.  Two calls in a row share the library's static
device array; the second batch is smaller, so it runs on top of what the first
one left there.
"""
import ctypes

import numpy as np
import pytest
import torch

import cabi
import helpers

pytestmark = pytest.mark.gpu


def _device_memory(dev):
    """(free bytes as the driver reports them, bytes torch's allocator holds)"""
    torch.cuda.synchronize()
    return torch.cuda.mem_get_info(dev)[0], torch.cuda.memory_reserved(dev)


def _static_loss(logits, targets, T, U, blank, fls, osf, max_u1, grad_scale, grad, memory=None):
    """`memory`: a list that receives the device memory figures right before and right
    after the C call (the helper's own output tensors are allocated before the first)."""
    rows, V = logits.shape
    N = T.numel()
    dev = logits.device
    scores = torch.full((N,), float("nan"), dtype=torch.float32, device=dev)
    status = torch.zeros(ctypes.sizeof(cabi.BatchStatus), dtype=torch.uint8, device=dev)
    if grad == "new":
        g = torch.full((rows, V), float("nan"), dtype=torch.float32, device=dev)
    elif grad == "inplace":
        g = logits
    else:
        g = None
    cols = targets.shape[1]
    if memory is not None:
        memory.append(_device_memory(dev))
    cabi.check(cabi.lib().ot_transducer_loss_static(
        cabi.ptr(logits), cabi.ptr(targets if cols else None), cabi.ptr(T), cabi.ptr(U),
        ctypes.c_int32(N), ctypes.c_int32(cols), ctypes.c_int64(rows), ctypes.c_int32(V),
        ctypes.c_int32(blank), ctypes.c_int32(int(fls)), ctypes.c_int32(int(osf)),
        ctypes.c_int32(max_u1), ctypes.c_float(grad_scale), cabi.ptr(scores), cabi.ptr(g),
        cabi.ptr(status), cabi.stream()))
    if memory is not None:
        memory.append(_device_memory(dev))
    st = cabi.BatchStatus.from_buffer_copy(status.cpu().numpy().tobytes())
    return scores, g, st


def _same_bits(a, b):
    return torch.equal(a.view(torch.int32), b.view(torch.int32))


CASES = [
    # (from_log_softmax, one_sym_per_frame, V): V = 37 takes the 4-byte path, 64 the 16-byte one
    (False, False, 64),
    (False, True, 37),
    (True, False, 37),
    (True, True, 64),
]


@pytest.mark.parametrize("fls,osf,V", CASES)
def test_static_entry_point_matches_the_workspace_one_twice_in_a_row(fls, osf, V, device):
    rng = np.random.default_rng(100 + V + 2 * fls + osf)
    # first a batch with a two-wave lattice, then a smaller one on the same array
    for N, tmax, umax in ((9, 120, 90), (3, 40, 12)):
        T, U, tg, x = helpers.random_batch(rng, N, tmax, umax, V, one_sym_per_frame=osf)
        if fls:
            x = helpers.log_softmax32(x)
        dT, dU, dtg = (torch.from_numpy(a).to(device) for a in (T, U, tg))
        max_u1 = int(U.max()) + 1
        mode = "new" if fls else "inplace"
        x_ws = torch.from_numpy(x).to(device)
        x_st = x_ws.clone()
        s_ws, g_ws, st_ws = cabi.transducer_loss(x_ws, dtg, dT, dU, 0, fls, osf, max_u1,
                                                 grad_scale=0.25, grad=mode)
        # the static call takes no device memory: neither from the driver (free memory as
        # hipMemGetInfo reports it) nor from torch's allocator
        memory = []
        s_st, g_st, st_st = _static_loss(x_st, dtg, dT, dU, 0, fls, osf, max_u1, 0.25, mode, memory)
        torch.cuda.synchronize()
        (free_before, held_before), (free_after, held_after) = memory
        assert held_after == held_before and free_after >= free_before, memory
        assert torch.isfinite(s_ws).all()
        assert _same_bits(s_st, s_ws)
        assert _same_bits(g_st, g_ws)
        assert bytes(st_st) == bytes(st_ws)
        # forward only: nothing but the scores is written
        x_fw = torch.from_numpy(x).to(device)
        s_fw, _, _ = _static_loss(x_fw, dtg, dT, dU, 0, fls, osf, max_u1, 1.0, None)
        assert _same_bits(s_fw, s_ws)
        assert torch.equal(x_fw, torch.from_numpy(x).to(device))


def test_static_entry_point_refuses_a_batch_beyond_its_array(device):
    L = cabi.lib()
    one = torch.zeros(64, dtype=torch.float32, device=device)
    rows = 1200000  # 44 bytes per row: more than the 48 MiB array
    assert L.ot_workspace_bytes(ctypes.c_int32(2), ctypes.c_int64(rows)) > 48 << 20
    rc = L.ot_transducer_loss_static(
        cabi.ptr(one), cabi.ptr(one), cabi.ptr(one), cabi.ptr(one), ctypes.c_int32(2),
        ctypes.c_int32(1), ctypes.c_int64(rows), ctypes.c_int32(4), ctypes.c_int32(0),
        ctypes.c_int32(0), ctypes.c_int32(0), ctypes.c_int32(2), ctypes.c_float(1.0),
        cabi.ptr(one), cabi.ptr(None), cabi.ptr(one), cabi.stream())
    assert rc == -4
    assert b"OT_STATIC_WORKSPACE_BYTES" in L.ot_error_string(rc)


def test_static_entry_point_replays_from_a_hip_graph(device):
    # what the entry point is for: a caller under graph capture.  The first call on the
    # device (which looks the array's address up) stays outside the capture; every replay is
    # checked against the eager result for the data that is in the buffers at that moment,
    # with eager work and synchronisations between the replays.
    rng = np.random.default_rng(77)
    T, U, tg, x0 = helpers.random_batch(rng, 6, 40, 70, 48)   # two waves per lattice
    N, rows, V = len(T), x0.shape[0], x0.shape[1]
    dT, dU, dtg = (torch.from_numpy(a).to(device) for a in (T, U, tg))
    logits = torch.empty((rows, V), device=device)
    scores = torch.empty(N, device=device)
    status = torch.zeros(ctypes.sizeof(cabi.BatchStatus), dtype=torch.uint8, device=device)
    L = cabi.lib()

    def launch():
        cabi.check(L.ot_transducer_loss_static(
            cabi.ptr(logits), cabi.ptr(dtg), cabi.ptr(dT), cabi.ptr(dU), ctypes.c_int32(N),
            ctypes.c_int32(tg.shape[1]), ctypes.c_int64(rows), ctypes.c_int32(V), ctypes.c_int32(0),
            ctypes.c_int32(0), ctypes.c_int32(0), ctypes.c_int32(int(U.max()) + 1),
            ctypes.c_float(0.5), cabi.ptr(scores), cabi.ptr(logits), cabi.ptr(status),
            cabi.stream()))

    inputs = [x0] + [rng.standard_normal(x0.shape).astype(np.float32) for _ in range(3)]
    eager = []
    for xi in inputs:
        logits.copy_(torch.from_numpy(xi).to(device))
        launch()
        torch.cuda.synchronize()
        eager.append((scores.clone(), logits.clone()))

    graph = torch.cuda.CUDAGraph()
    logits.copy_(torch.from_numpy(inputs[0]).to(device))
    torch.cuda.synchronize()
    with torch.cuda.graph(graph):
        launch()
    for k in (1, 2, 3, 0, 2):
        logits.copy_(torch.from_numpy(inputs[k]).to(device))   # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert _same_bits(scores, eager[k][0]) and _same_bits(logits, eager[k][1]), k
