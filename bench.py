#!/usr/bin/env python3
"""Throughput of the transducer loss (forward + backward) on one MI355X.

A step is ``loss = transducer_loss(logits, ...); loss.backward()`` on one batch
of synthetic packed logits that are already resident in HBM.  The logits path
overwrites its input, so every step gets its own pristine copy, cloned before
the timed region (288 GB of HBM hold dozens of 1.4 GB batches).

Prints ONE JSON line: utterances/s for the whole job, the HBM roofline of the
dominant kernel (the in-place gradient kernel) measured with hipEvents on the
launch stream, and the reference's CPU path timed on this machine's host cores.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published peak



def measured_traffic(workload_name, kernel):
    """HBM bytes per launch of `kernel` on `workload_name` as a committed counter
    summary records them (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by the same
    counters on the library's 1 GiB copy kernel): the line
    `traffic_bytes_per_launch <workload> <kernel> <bytes> source_sha <sha>` of a
    profiles/hbm_traffic_*.md file.  Returns (bytes, source) or (None, None): nothing
    is echoed that is not on file, and the source names the commit it was measured at."""
    import glob
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", "hbm_traffic_*.md"))):
        with open(path) as f:
            for line in f:
                parts = line.replace("`", " ").split()
                if (len(parts) >= 6 and parts[0] == "traffic_bytes_per_launch"
                        and parts[1] == workload_name and parts[2] == kernel):
                    return float(parts[3]), "profiles/%s @ %s" % (os.path.basename(path), parts[5])
    return None, None


def make_workload(name):
    import workloads
    if name == "asr":  # N=32, T~U{200..500}, U~U{20..100}, V=500, logits, sum
        return workloads.asr_batch()
    if name == "asr_logsoftmax_modified":
        return workloads.asr_batch_logsoftmax_modified()
    if name == "largevocab":
        return workloads.large_vocab()
    if name == "ragged":
        return workloads.ragged()
    if name == "ragged_modified":
        return workloads.ragged(one_sym_per_frame=True)
    if name == "tiny":
        return workloads.tiny()
    raise SystemExit("unknown workload %r" % name)


def algorithmic_bytes(w, esize=4):
    """Bytes per launch each kernel has to move, per packed row of V elements of esize bytes."""
    R, V = w.rows, w.V
    if w.from_log_softmax:
        return {"gather": 16 * R, "alpha_beta": 24 * R, "grad_logsoftmax": (esize * V + 24) * R}
    return {"lse_gather": (esize * V + 4 + 8) * R, "alpha_beta": 24 * R,
            "grad_logits": (2 * esize * V + 20) * R}


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(w, logits_host, max_seconds=30.0):
    """The reference's CPU path (oracle/_ref) or, failing that, the C port, on
    the same batch; bounded to about max_seconds of CPU time.  Returns the record
    for the JSON line and the (scores, loss, gradient) of the last run, which the
    parity check compares the GPU's results with."""
    import numpy as np
    import torch
    from oracle import oracle, ref_loader

    ref = ref_loader.load()
    threads = torch.get_num_threads()
    tg = torch.from_numpy(w.targets)
    T = torch.from_numpy(w.logit_lengths)
    U = torch.from_numpy(w.target_lengths)

    result = {}

    def once():
        x = logits_host.clone()
        t0 = time.perf_counter()
        if ref is not None:
            x.requires_grad_(True)
            scores, grad = ref.compute_transducer_loss(
                logits=x, targets=tg, logit_lengths=T, target_lengths=U, blank=w.blank,
                from_log_softmax=w.from_log_softmax, one_sym_per_frame=w.one_sym_per_frame)
            with torch.no_grad():  # what the reference's autograd.Function does around the call
                loss = -scores
                loss = loss.mean() if w.reduction == "mean" else loss.sum()
                if w.reduction == "mean":
                    grad /= w.N
                grad.mul_(torch.ones(()))  # backward's mul_(loss_grad)
            dt = time.perf_counter() - t0
            result.update(scores=scores.detach(), loss=float(loss), grad=grad.detach())
        else:
            loss, grad = oracle.transducer_loss(x.numpy(), w.targets, w.logit_lengths,
                                                w.target_lengths, w.blank, w.from_log_softmax,
                                                w.one_sym_per_frame, w.reduction)
            dt = time.perf_counter() - t0
            scores, _ = oracle.compute_transducer_loss(
                logits_host.numpy().copy(), w.targets, w.logit_lengths, w.target_lengths, w.blank,
                w.from_log_softmax, w.one_sym_per_frame, want_grad=False)
            result.update(scores=torch.from_numpy(scores), loss=float(loss),
                          grad=torch.from_numpy(grad))
        return dt

    times = [once()]
    while len(times) < 3 and sum(times) + times[-1] < max_seconds:
        times.append(once())
    best = float(np.median(times))
    kind = "reference" if ref is not None else "port"
    return {
        "value": w.N / best, "unit": "utterances/s", "cores": threads if ref is not None else 1,
        "os_cpu_count": os.cpu_count(), "cpu_model": cpu_model(),
        "kind": kind,
        "sample": "%d full batch(es) of workload %s (N=%d, rows=%d, V=%d), median of %d; "
                  "%s" % (len(times), w.name, w.N, w.rows, w.V, len(times),
                          "ATen logsumexp on %d threads, lattice and gradient loops single-threaded "
                          "as the reference runs them" % threads if ref is not None
                          else "single-threaded C port of the reference's CPU path"),
        "seconds_per_batch": best,
    }, result


def grad_error_stats(got_grad, ref_grad, unit=None, output_rounding=0.0):
    """How far two gradients of one batch are apart: the north-star tolerance (rel 1e-5 /
    abs 1e-5) entry by entry and, with `unit` (one rounding of an entry's exponent:
    eps * |log-likelihood of the utterance| * sum of the entry's exponentials), the
    largest difference in those units and the per-entry bound 1e-5 + 1e-5 |ref| + 4 units
    that the end-to-end tests assert.  `output_rounding`: relative rounding of the stored
    gradient when it is not float32 (2^-8 for bfloat16, 2^-11 for float16), added to the
    bound only."""
    import torch
    diff = (got_grad - ref_grad).abs_()
    big = ref_grad.abs() > 1e-4
    within = diff <= 1e-5 + 1e-5 * ref_grad.abs()
    rec = {
        "grad_max_abs_err": float(diff.max()),
        "grad_max_rel_err_over_1e-4": float((diff[big] / ref_grad[big].abs()).max()) if bool(big.any()) else 0.0,
        "grad_entries_over_1e-4": int(big.sum()),
        "grad_frac_within_1e-5": float(within.double().mean()),
        "grad_allclose_rtol1e-5_atol1e-5": bool(within.all()),
    }
    del big, within
    if unit is not None:
        ok = unit > 1e-30  # smaller ones belong to denormal entries, which the GPU flushes to zero
        rec["grad_max_err_in_noise_units"] = float((diff[ok] / unit[ok]).max()) if bool(ok.any()) else 0.0
        rec["grad_within_noise_bound"] = bool(
            (diff <= 1e-5 + (1e-5 + output_rounding) * ref_grad.abs() + NOISE_K * unit).all())
        del ok
    return rec


NOISE_K = 4.0  # roundings of an entry's exponent that two float32 evaluations may differ by


def parity_record(w, args, pristine, targets, T, U, ref, with_f64):
    """The timed workload once more through the shipped Python entry point, outside
    the timed region, against what the CPU baseline computed for the same batch
    (the compiled reference, float32): the parity gate of this run.

    Three views of the gradient error: against the north-star tolerance as it stands;
    in units of one float32 rounding of an entry's exponent (the exponent is a sum of
    terms as large as the utterance's log-likelihood, cpu.cc:509-522, so two correct
    float32 evaluations differ by a few such units); and the same comparison with the
    reference's own denominators (ATen's logsumexp on the host, cpu.cc:770) handed to the
    GPU, which leaves only the lattice and gradient arithmetic to differ."""
    import numpy as np
    import torch
    import optimized_transducer_amd as ot
    from optimized_transducer_amd import _optimized_transducer as ext
    from oracle import oracle

    def gpu_gradient(**kwargs):
        buf = pristine.clone().requires_grad_(True)
        loss = ot.transducer_loss(buf, targets, T, U, w.blank, w.from_log_softmax,
                                  w.one_sym_per_frame, w.reduction,
                                  defer_gradient=args.defer_gradient, **kwargs)
        (loss * args.loss_weight if args.loss_weight != 1.0 else loss).backward()
        return float(loss), buf.grad.float().cpu()

    got_loss, got_grad = gpu_gradient()
    scores, _ = ext.compute_transducer_loss(
        logits=pristine.clone(), targets=targets, logit_lengths=T, target_lengths=U, blank=w.blank,
        from_log_softmax=w.from_log_softmax, one_sym_per_frame=w.one_sym_per_frame)
    got_scores = scores.cpu()
    del scores

    ref_grad = ref["grad"] if args.loss_weight == 1.0 else ref["grad"] * args.loss_weight
    host_logits = pristine.float().cpu()
    sizes = w.logit_lengths.astype(np.int64) * (w.target_lengths.astype(np.int64) + 1)
    scale = args.loss_weight / (w.N if w.reduction == "mean" else 1.0)
    # the unit of the noise figures, from the float32 CPU restatement on the same batch
    # (its gradient function also emits the sum of every entry's exponentials)
    s32, _, m32 = oracle.compute_transducer_loss(
        host_logits.numpy(), w.targets, w.logit_lengths, w.target_lengths, w.blank,
        w.from_log_softmax, w.one_sym_per_frame, return_magnitude=True)
    unit = torch.from_numpy(m32)
    unit *= torch.from_numpy(
        (np.finfo(np.float32).eps * abs(scale) * np.repeat(np.abs(s32), sizes)).astype(np.float32))[:, None]
    del m32

    rec = {
        "entry_point": "optimized_transducer_amd.transducer_loss(...).backward()",
        "against": "the CPU baseline's output for the same batch (float32)",
        "noise_unit": "eps(float32) * |log-likelihood of the utterance| * sum of the entry's "
                      "exponentials, from the float32 CPU restatement (oracle/) on this batch",
        "loss": got_loss, "loss_reference": ref["loss"],
        "loss_rel_err": abs(got_loss - ref["loss"]) / max(abs(ref["loss"]), 1e-30),
        "scores_max_rel_err": float(((got_scores - ref["scores"]).abs()
                                     / ref["scores"].abs().clamp_min(1e-30)).max()),
        "scores_allclose_rtol1e-5_atol1e-5": bool(torch.allclose(got_scores, ref["scores"], rtol=1e-5, atol=1e-5)),
    }
    rounding = {torch.float32: 0.0, torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}[pristine.dtype]
    rec.update(grad_error_stats(got_grad, ref_grad, unit, rounding))
    if not w.from_log_softmax and pristine.dtype == torch.float32:
        # ATen's logsumexp on the host is where the reference's denominators come from
        den = torch.logsumexp(host_logits, 1).to(pristine.device)
        loss_d, grad_d = gpu_gradient(denominators=den)
        rec["with_reference_denominators"] = dict(
            grad_error_stats(grad_d, ref_grad, unit),
            loss_rel_err=abs(loss_d - ref["loss"]) / max(abs(ref["loss"]), 1e-30),
            what="the same batch with the reference's own denominators handed to the GPU "
                 "(transducer_loss(..., denominators=torch.logsumexp(logits_cpu, 1))): only the "
                 "lattice and gradient arithmetic differ from the reference")
        del den, grad_d
    # the gate: integers bit for bit (below), loss and scores at rel/abs 1e-5, every gradient
    # entry within 1e-5 + 1e-5 |ref| + NOISE_K noise units
    rec["parity_ok"] = bool(rec["loss_rel_err"] <= 1e-5 and rec["scores_allclose_rtol1e-5_atol1e-5"]
                            and rec["grad_within_noise_bound"])
    # the integer part of the gate, through the C ABI: row offsets and the row -> utterance
    # map against numpy's cumsum / repeat, bit for bit
    import ctypes
    lib = ctypes.CDLL(os.path.join(ROOT, "optimized_transducer_amd", "libot_transducer.so"))
    N = int(T.numel())
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    splits = torch.empty(N + 1, dtype=torch.int32, device=T.device)
    status = torch.zeros(64, dtype=torch.uint8, device=T.device)
    ids = torch.empty(w.rows, dtype=torch.int32, device=T.device)
    ptr = lambda t: ctypes.c_void_p(t.data_ptr())  # noqa: E731
    rc = lib.ot_row_splits(ptr(T), ptr(U), ptr(targets), ctypes.c_int32(N),
                           ctypes.c_int32(int(targets.shape[1])), ptr(splits), ctypes.c_void_p(None),
                           ptr(status), stream)
    rc = rc or lib.ot_row_ids(ptr(splits), ctypes.c_int32(N), ctypes.c_int64(w.rows), ptr(ids), stream)
    want_splits = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
    rec["row_splits_bit_equal"] = bool(rc == 0 and np.array_equal(splits.cpu().numpy(), want_splits))
    rec["row_ids_bit_equal"] = bool(rc == 0 and np.array_equal(
        ids.cpu().numpy(), np.repeat(np.arange(N, dtype=np.int32), sizes)))
    rec["parity_ok"] = bool(rec["parity_ok"] and rec["row_splits_bit_equal"] and rec["row_ids_bit_equal"])
    del splits, status, ids, unit
    if with_f64:
        # the same recursions in float64 as the arbiter between two float32 evaluations
        s64, g64, m64 = oracle.compute_transducer_loss(
            host_logits.numpy(), w.targets, w.logit_lengths, w.target_lengths, w.blank,
            w.from_log_softmax, w.one_sym_per_frame, dtype=np.float64, return_magnitude=True)
        g64 *= scale
        m64 *= scale
        unit64 = np.finfo(np.float32).eps * np.repeat(np.abs(s64), sizes)[:, None] * m64
        ok = unit64 > 1e-30
        rec["float64"] = {}
        for name, g, sc in (("gpu", got_grad.numpy(), got_scores.numpy()),
                            ("reference", ref_grad.numpy(), ref["scores"].numpy())):
            d = np.abs(g - g64)
            rec["float64"][name] = {
                "grad_max_abs_err": float(d.max()),
                # in units of eps * |log-likelihood| * (sum of the entry's exponentials)
                "grad_max_err_in_noise_units": float((d[ok] / unit64[ok]).max()),
                "scores_max_rel_err": float((np.abs(sc - s64) / np.abs(s64)).max()),
            }
            del d
    return rec


def timed_steps(torch, step, K, W):
    """W untimed steps, then K timed ones between two synchronisations; also the spread
    of the K steps, each between two events on the launch stream.  Returns (seconds,
    {"median", "min", "max"} in milliseconds)."""
    for _ in range(W):
        step()
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(K + 1)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    marks[0].record()
    for i in range(K):
        step()
        marks[i + 1].record()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(K))
    median = ms[K // 2] if K % 2 else 0.5 * (ms[K // 2 - 1] + ms[K // 2])
    return elapsed, {"median": median, "min": ms[0], "max": ms[-1]}


def bench_joiner(args):
    """Secondary benchmark: the packed joiner input (pack_joiner, tanh) forward +
    backward for the lengths of the chosen workload; not the headline metric."""
    import numpy as np
    import torch
    import optimized_transducer_amd as ot
    from optimized_transducer_amd import _optimized_transducer as ext

    dev = torch.device("cuda", 0)
    w = make_workload(args.workload)
    K, W, D = args.steps, args.warmup, args.joiner_dim
    N, R = w.N, w.rows
    Tm, U1m = int(w.logit_lengths.max()), int(w.target_lengths.max()) + 1
    gen = torch.Generator(device="cpu").manual_seed(w.seed)
    enc_h = torch.randn((N, Tm, D), generator=gen)
    dec_h = torch.randn((N, U1m, D), generator=gen)
    enc = enc_h.to(dev).requires_grad_(True)
    dec = dec_h.to(dev).requires_grad_(True)
    T = torch.from_numpy(w.logit_lengths).to(dev)
    U = torch.from_numpy(w.target_lengths).to(dev)
    out_dtype = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[args.logits_dtype]
    esize = 4 if out_dtype == torch.float32 else 2
    g = torch.randn((R, D), device=dev).to(out_dtype)

    def step():
        enc.grad = dec.grad = None
        x = ot.pack_joiner(enc, dec, T, U, activation="tanh", out_dtype=out_dtype)
        x.backward(g)

    elapsed, spread = timed_steps(torch, step, K, W)
    out = {
        "metric": "utterances/sec packed joiner input (tanh) fwd+bwd; achieved HBM GB/s vs peak",
        "value": N * K / elapsed, "unit": "utterances/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": 1e3 * elapsed / K, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "step_ms": spread, "dtype": "f32" if esize == 4 else "f32->" + args.logits_dtype,
        "data": "synthetic",
        "config": {"workload": "joiner_input_of_" + w.name, "N": N, "D": D, "packed_rows": R,
                   "T_max": Tm, "U1_max": U1m, "activation": "tanh", "packed_bytes": esize * R * D},
    }
    ext.set_profiling(True)
    for _ in range(K):
        step()
    torch.cuda.synchronize()
    ext.set_profiling(False)
    per = {}
    for name, ms in ext.take_profile():
        per.setdefault(name, []).append(ms)
    # pack: writes (rows, D) once; unpack: reads (rows, D) once and
    # writes + re-reads one partial decoder sum per 16 frames
    alg = {"joiner_pack": esize * D * R, "joiner_unpack_grad": 4 * D * R + 2 * (4 * D * R // 16)}
    kernels = {}
    for name, ms in per.items():
        per_step = sum(ms) / K
        kernels[name] = {"ms_per_step": per_step, "launches_per_step": len(ms) / K}
        if name in alg:
            kernels[name]["algorithmic_bytes"] = alg[name]
            kernels[name]["achieved_GBps"] = alg[name] / (per_step * 1e-3) / 1e9
    dom = max(alg, key=lambda k: kernels[k]["ms_per_step"])
    out["roofline"] = {"bound": "hbm", "kernel": dom + "_kernel", "peak": HBM_PEAK_GBPS,
                       "achieved": kernels[dom]["achieved_GBps"], "unit": "GB/s",
                       "frac": kernels[dom]["achieved_GBps"] / HBM_PEAK_GBPS, "traffic": None,
                       "kernel_ms_per_step": kernels[dom]["ms_per_step"],
                       "algorithmic_bytes_per_step": alg[dom]}
    out["kernels"] = kernels
    if not args.no_cpu_baseline:
        # the reference's own recipe (README.md:166-177) in torch on the host cores
        e = enc_h.clone().requires_grad_(True)
        d = dec_h.clone().requires_grad_(True)
        gh = g.cpu()
        Tl, Ul = w.logit_lengths.tolist(), w.target_lengths.tolist()
        t0 = time.perf_counter()
        parts = [(e[i, :Tl[i]].unsqueeze(1) + d[i, :Ul[i] + 1].unsqueeze(0)).reshape(-1, D)
                 for i in range(N)]
        torch.tanh(torch.cat(parts)).backward(gh)
        sec = time.perf_counter() - t0
        out["cpu_baseline"] = {"value": N / sec, "unit": "utterances/s",
                               "cores": torch.get_num_threads(), "kind": "reference",
                               "sample": "one full batch: the README.md:166-177 recipe "
                                         "(list of slices, cat, tanh) and its autograd in torch",
                               "seconds_per_batch": sec}
    print(json.dumps(out), flush=True)


def bench_project(args):
    """Secondary benchmark: the joiner's output projection fused with the loss's
    denominators (project_joiner, 16-bit activations and weight, matrix cores),
    followed by the loss forward + backward on its logits; beside it the same step
    with torch's own projection and the loss's own denominator pass."""
    import torch
    import optimized_transducer_amd as ot
    from optimized_transducer_amd import _optimized_transducer as ext

    dev = torch.device("cuda", 0)
    w = make_workload(args.workload)
    K, W, D = args.steps, args.warmup, args.joiner_dim
    N, R, V = w.N, w.rows, w.V
    act = torch.bfloat16 if args.logits_dtype != "f16" else torch.float16
    f32_logits = args.logits_dtype == "f32"
    gen = torch.Generator(device="cpu").manual_seed(w.seed)
    x = torch.tanh(torch.randn((R, D), generator=gen)).to(act).to(dev)
    wt = (torch.randn((V, D), generator=gen) / D ** 0.5).to(act).to(dev)
    bias = torch.randn((V,), generator=gen).to(dev)
    targets = torch.from_numpy(w.targets).to(dev)
    T = torch.from_numpy(w.logit_lengths).to(dev)
    U = torch.from_numpy(w.target_lengths).to(dev)

    # --vocab-multiple m: the fused variant runs on a vocabulary padded with masked entries
    # to the next multiple of m (same loss, same gradient in the real columns), as
    # project_joiner(..., vocab_multiple=m) does; the weight is padded once, outside the step
    wt_f, bias_f = wt, bias
    if args.vocab_multiple and V % args.vocab_multiple:
        Vp = -(-V // args.vocab_multiple) * args.vocab_multiple
        wt_f = torch.zeros((Vp, D), dtype=act, device=dev)
        wt_f[:V] = wt
        bias_f = torch.full((Vp,), float("-inf"), device=dev)
        bias_f[:V] = bias

    def fused():
        logits, den = ext.joiner_project(x=x, weight=wt_f, bias=bias_f, float32_logits=f32_logits)
        logits.requires_grad_(True)
        loss = ot.transducer_loss(logits, targets, T, U, w.blank, False, w.one_sym_per_frame,
                                  "sum", denominators=den)
        loss.backward()

    bias_act = bias.to(act)

    def unfused():
        if f32_logits:
            logits = torch.mm(x, wt.t(), out_dtype=torch.float32).add_(bias)
        else:
            logits = torch.addmm(bias_act, x, wt.t())
        logits.requires_grad_(True)
        loss = ot.transducer_loss(logits, targets, T, U, w.blank, False, w.one_sym_per_frame, "sum")
        loss.backward()

    elapsed, spread = timed_steps(torch, fused, K, W)
    elapsed_unfused, spread_unfused = timed_steps(torch, unfused, K, W)

    # The whole training step of the joiner's tail: projection + loss forward and backward
    # down to the gradients of x, weight and bias (the backward products are torch's own
    # in both arrangements).
    xg = x.clone().requires_grad_(True)
    wg = wt.clone().requires_grad_(True)
    bg = bias.clone().requires_grad_(True)

    def whole_fused():
        xg.grad = wg.grad = bg.grad = None
        loss = ot.joiner_transducer_loss(xg, wg, bg, targets, T, U, w.blank, w.one_sym_per_frame,
                                         "sum", float32_logits=f32_logits)
        loss.backward()

    def whole_unfused():
        xg.grad = wg.grad = bg.grad = None
        if f32_logits:
            logits = torch.nn.functional.linear(xg.float(), wg.float(), bg)
        else:
            logits = torch.nn.functional.linear(xg, wg, bg.to(act))
        loss = ot.transducer_loss(logits, targets, T, U, w.blank, False, w.one_sym_per_frame, "sum")
        loss.backward()

    elapsed_whole, spread_whole = timed_steps(torch, whole_fused, K, W)
    elapsed_whole_unfused, spread_whole_unfused = timed_steps(torch, whole_unfused, K, W)
    flops = 2.0 * R * D * V  # of the real columns, padded or not
    out = {
        "metric": "utterances/sec joiner output projection (fused denominators) + transducer loss "
                  "fwd+bwd; achieved MFMA TFLOP/s of the projection vs peak",
        "value": N * K / elapsed, "unit": "utterances/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": 1e3 * elapsed / K, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "step_ms": spread,
        "dtype": args.logits_dtype if not f32_logits else "bf16->f32",
        "data": "synthetic",
        "config": {"workload": "joiner_projection_of_" + w.name, "N": N, "D": D, "V": V,
                   "packed_rows": R, "activations": str(act).split(".")[-1],
                   "logits": "f32" if f32_logits else str(act).split(".")[-1],
                   "fused_vocabulary_columns": int(wt_f.shape[0])},
        "unfused": {"ms_per_step": 1e3 * elapsed_unfused / K, "step_ms": spread_unfused,
                    "what": "torch (hipBLASLt) projection of the same operands, then the loss with "
                            "its own denominator pass"},
        "whole_step": {
            "what": "projection + loss forward and backward down to the gradients of x, weight and "
                    "bias: joiner_transducer_loss(...).backward() against torch's linear (in float32 "
                    "for float32 logits) followed by transducer_loss",
            "fused_ms_per_step": 1e3 * elapsed_whole / K, "fused_step_ms": spread_whole,
            "unfused_ms_per_step": 1e3 * elapsed_whole_unfused / K,
            "unfused_step_ms": spread_whole_unfused},
    }
    ext.set_profiling(True)
    for _ in range(K):
        fused()
    torch.cuda.synchronize()
    ext.set_profiling(False)
    per = {}
    for name, ms in ext.take_profile():
        per.setdefault(name, []).append(ms)
    kernels = {name: {"ms_per_step": sum(ms) / K, "launches_per_step": len(ms) / K}
               for name, ms in per.items()}
    t = kernels["joiner_project"]["ms_per_step"]
    kernels["joiner_project"]["flops"] = flops
    kernels["joiner_project"]["achieved_TFLOPs"] = flops / (t * 1e-3) / 1e12
    # bytes the projection cannot avoid: read x and W once, write the logits once
    min_bytes = 2.0 * R * D + 2.0 * V * D + (4.0 if f32_logits else 2.0) * R * V
    out["roofline"] = {"bound": "mfma", "kernel": "joiner_project_kernel", "peak": 2500.0,
                       "achieved": kernels["joiner_project"]["achieved_TFLOPs"], "unit": "TFLOP/s",
                       "frac": kernels["joiner_project"]["achieved_TFLOPs"] / 2500.0, "traffic": None,
                       "kernel_ms_per_step": t, "flops_per_step": flops,
                       "hbm_bound_ms": min_bytes / (HBM_PEAK_GBPS * 1e9) * 1e3}
    out["kernels"] = kernels
    print(json.dumps(out), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="asr")
    ap.add_argument("--defer-gradient", action="store_true",
                    help="use the deferred mode of the Python API (gradient pass in backward)")
    ap.add_argument("--loss-weight", type=float, default=1.0,
                    help="multiply the loss by this before backward (a weighted or scaled loss); "
                         "the headline figure uses 1")
    ap.add_argument("--logits-dtype", default="f32", choices=["f32", "f16", "bf16"],
                    help="element type of the logits; the headline figure uses f32 (the only type "
                         "the reference accepts), f16/bf16 measure the half-precision addition")
    ap.add_argument("--op", default="loss", choices=["loss", "joiner", "project"],
                    help="loss: the headline benchmark; joiner: the packed joiner input "
                         "(pack_joiner) forward + backward for the workload's lengths; project: "
                         "the joiner's output projection fused with the denominators "
                         "(project_joiner), then the loss forward + backward")
    ap.add_argument("--joiner-dim", type=int, default=512)
    ap.add_argument("--vocab-multiple", type=int, default=0,
                    help="--op project: pad the fused variant's vocabulary with masked entries to "
                         "a multiple of this (32: whole 128-byte lines per float32 row)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-roofline", action="store_true")
    ap.add_argument("--no-weighted", action="store_true",
                    help="skip the secondary measurement of a weighted loss (default and deferred mode)")
    ap.add_argument("--no-parity", action="store_true",
                    help="skip the parity gate (the GPU's loss and gradient for the timed workload "
                         "against the CPU baseline's, outside the timed region)")
    ap.add_argument("--parity-f64", action="store_true",
                    help="also run the float64 build of the CPU restatement on the whole batch and "
                         "report how far the GPU and the float32 reference each are from it")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch the library's plain copy kernel on 1 GiB (read 1 GiB + "
                         "write 1 GiB) three times, as a known-size reference for profiler "
                         "byte counters")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py: this build measures one GPU only (got --gpus %d); "
                         "utterances are independent, so N GPUs shard the batch by utterance "
                         "and nothing here would change per GPU." % args.gpus)

    import torch
    import optimized_transducer_amd as ot
    from optimized_transducer_amd import _optimized_transducer as ext

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    if args.op == "joiner":
        return bench_joiner(args)
    if args.op == "project":
        return bench_project(args)
    dev = torch.device("cuda", 0)
    w = make_workload(args.workload)
    K, W = args.steps, args.warmup

    pristine = w.logits_torch(dev)
    esize = 4
    if args.logits_dtype != "f32":
        pristine = pristine.to(torch.float16 if args.logits_dtype == "f16" else torch.bfloat16)
        esize = 2
    targets = torch.from_numpy(w.targets).to(dev)
    T = torch.from_numpy(w.logit_lengths).to(dev)
    U = torch.from_numpy(w.target_lengths).to(dev)

    def step(buf, defer=args.defer_gradient, weight=args.loss_weight):
        buf.requires_grad_(True)
        loss = ot.transducer_loss(buf, targets, T, U, w.blank, w.from_log_softmax,
                                  w.one_sym_per_frame, w.reduction, defer_gradient=defer)
        if weight != 1.0:
            loss = loss * weight
        loss.backward()
        # what a training loop's zero_grad(set_to_none=True) does: with log-softmax
        # input the gradient is a tensor of its own, and K of them kept alive would
        # put K device allocations of (rows, V) floats into the timed region
        # (with logits input the gradient is the buffer itself, and this frees nothing)
        buf.grad = None
        return loss

    def wall_ms_per_step(**mode):
        """W warm-up steps, then K steps between two synchronisations, each on its own
        pristine copy of the logits (cloned outside the timed region)."""
        for _ in range(W):
            step(pristine.clone(), **mode)
        bufs = [pristine.clone() for _ in range(K)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for b in bufs:
            step(b, **mode)
        torch.cuda.synchronize()
        return 1e3 * (time.perf_counter() - t0) / K

    if args.calibrate_copy:
        import ctypes
        lib = ctypes.CDLL(os.path.join(ROOT, "optimized_transducer_amd", "libot_transducer.so"))
        src = torch.ones(1 << 28, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            rc = lib.ot_copy_floats(ctypes.c_void_p(src.data_ptr()), ctypes.c_void_p(dst.data_ptr()),
                                    ctypes.c_int64(src.numel()),
                                    ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
            assert rc == 0, rc
        torch.cuda.synchronize()
        del src, dst

    for _ in range(W):
        step(pristine.clone())
    torch.cuda.synchronize()

    bufs = [pristine.clone() for _ in range(K)]
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(K + 1)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    marks[0].record()
    for i, b in enumerate(bufs):
        step(b)
        marks[i + 1].record()  # on the stream the step's kernels were launched on
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    del bufs
    per_step_ms = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(K))

    out = {
        # the headline metric's name on the headline workload (N=32, V=500)
        "metric": "utterances/sec fwd+bwd loss at N=%d,V=%d fp32; achieved HBM GB/s vs peak" % (w.N, w.V),
        "value": w.N * K / elapsed, "unit": "utterances/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": 1e3 * elapsed / K, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None,
        # spread of the K timed steps, each between two events on the launch stream
        "step_ms": {"median": per_step_ms[K // 2] if K % 2 else
                    0.5 * (per_step_ms[K // 2 - 1] + per_step_ms[K // 2]),
                    "min": per_step_ms[0], "max": per_step_ms[-1]},
        "dtype": "f32" if esize == 4 else "f32 arithmetic on %s logits" % args.logits_dtype,
        "data": "synthetic",
        "config": {"workload": w.name, "N": w.N, "V": w.V, "packed_rows": w.rows,
                   "from_log_softmax": w.from_log_softmax,
                   "one_sym_per_frame": w.one_sym_per_frame, "reduction": w.reduction,
                   "logits_bytes": esize * w.rows * w.V, "seed": w.seed},
    }
    if args.defer_gradient or args.loss_weight != 1.0:
        out["config"]["defer_gradient"] = args.defer_gradient
        out["config"]["loss_weight"] = args.loss_weight

    if not args.no_roofline:
        # second pass, per-kernel hipEvent timing on the launch stream
        bufs = [pristine.clone() for _ in range(K)]
        torch.cuda.synchronize()
        ext.set_profiling(True)
        for b in bufs:
            step(b)
        torch.cuda.synchronize()
        ext.set_profiling(False)
        del bufs
        per = {}
        for name, ms in ext.take_profile():
            per.setdefault(name, []).append(ms)
        alg = algorithmic_bytes(w, esize)
        kernels = {}
        for name, ms in per.items():
            # a large batch is processed in two parts (two launches per step of the
            # same kernel, each on its share of the rows): durations add up per step
            per_step = sum(ms) / K
            kernels[name] = {"ms_per_step": per_step, "launches_per_step": len(ms) / K}
            if name in alg and per_step > 0:
                kernels[name]["algorithmic_bytes"] = alg[name]
                kernels[name]["achieved_GBps"] = alg[name] / (per_step * 1e-3) / 1e9
        dom = "grad_logsoftmax" if w.from_log_softmax else "grad_logits"
        achieved = kernels[dom]["achieved_GBps"]
        kernel_name = "grad_flat_kernel<%d,%s>" % (4 if w.V % 4 == 0 else 1,
                                                    "true" if w.from_log_softmax else "false")
        if esize == 2:
            kernel_name = "grad_flat_half_kernel"
        traffic, traffic_source = measured_traffic(w.name, dom) if esize == 4 else (None, None)
        out["roofline"] = {"bound": "hbm", "kernel": kernel_name, "achieved": achieved,
                           "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                           "frac": achieved / HBM_PEAK_GBPS,
                           "traffic": traffic, "traffic_source": traffic_source,
                           "kernel_ms_per_step": kernels[dom]["ms_per_step"],
                           "launches_per_step": kernels[dom]["launches_per_step"],
                           "algorithmic_bytes_per_step": alg[dom]}
        out["kernels"] = kernels

    if not args.defer_gradient and args.loss_weight == 1.0 and not args.no_weighted:
        # secondary: a loss that is multiplied by a weight before backward() (a weighted sum of
        # losses, loss scaling).  The reference's order of operations, kept by default, makes a
        # second pass over the gradient (transducer_loss.py:162); defer_gradient=True folds the
        # factor into the one gradient pass.  Not the headline figure.
        out["weighted_loss"] = {
            "loss_weight": 0.5,
            "default_ms_per_step": wall_ms_per_step(defer=False, weight=0.5),
            "deferred_ms_per_step": wall_ms_per_step(defer=True, weight=0.5),
            "deferred_ms_per_step_weight_1": wall_ms_per_step(defer=True, weight=1.0),
        }

    if not args.no_cpu_baseline:
        out["cpu_baseline"], ref = cpu_baseline(w, pristine.float().cpu())
        out["speedup_vs_cpu"] = out["value"] / out["cpu_baseline"]["value"]
        if not args.no_parity:
            out["parity"] = parity_record(w, args, pristine, targets, T, U, ref, args.parity_f64)
            out["parity_ok"] = out["parity"]["parity_ok"]

    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
