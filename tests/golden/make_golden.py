#!/usr/bin/env python3
"""Writes the golden vectors of tests/golden/*.npz.

Run in the build container only:  python tests/golden/make_golden.py

Inputs are generated here (seeded numpy); expected outputs come from the
reference's own CPU path, compiled by ``make -C oracle ref`` into
``oracle/_ref/_optimized_transducer.so`` (the reference ships no golden vectors
of its own: its four tests are differential).  Only numbers are stored.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

import workloads  # noqa: E402
from oracle import ref_loader  # noqa: E402


def run_ref(ref, logits, targets, T, U, blank, fls, osf):
    x = torch.from_numpy(logits.copy()).requires_grad_(True)
    scores, grad = ref.compute_transducer_loss(
        logits=x, targets=torch.from_numpy(targets), logit_lengths=torch.from_numpy(T),
        target_lengths=torch.from_numpy(U), blank=blank, from_log_softmax=fls,
        one_sym_per_frame=osf)
    return scores.detach().numpy().copy(), grad.detach().numpy().copy()


def log_softmax(x):
    m = x.max(axis=1, keepdims=True)
    z = (x - m).astype(np.float64)
    return (z - np.log(np.exp(z).sum(axis=1, keepdims=True))).astype(np.float32)


def case(ref, name, T, U, targets, V, blank, rng, sigma=1.0):
    T = np.asarray(T, np.int32)
    U = np.asarray(U, np.int32)
    targets = np.ascontiguousarray(targets, np.int32)
    rows = int((T.astype(np.int64) * (U + 1)).sum())
    logits = (rng.standard_normal((rows, V)) * sigma).astype(np.float32)
    out = dict(logit_lengths=T, target_lengths=U, targets=targets, blank=np.int32(blank),
               logits=logits)
    for osf in (0, 1):
        if osf and (U > T - 1).any():
            continue  # the modified lattice is undefined for U > T-1 (cpu.cc:279)
        for fls in (0, 1):
            x = log_softmax(logits) if fls else logits
            s, g = run_ref(ref, x, targets, T, U, blank, bool(fls), bool(osf))
            out["scores_fls%d_osf%d" % (fls, osf)] = s
            out["grad_fls%d_osf%d" % (fls, osf)] = g
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **out)
    print(name, "rows", rows, "V", V, sorted(k for k in out if k.startswith("scores")))


def main():
    ref = ref_loader.load()
    assert ref is not None, "build oracle/_ref first: make -C oracle ref"
    torch.set_num_threads(1)

    # configuration 1: N=4, T~U{20..50}, U~U{5..15}, V=32, seed 1
    w = workloads.tiny()
    case(ref, "tiny_N4_V32", w.logit_lengths, w.target_lengths, w.targets, w.V, w.blank,
         np.random.default_rng(101))

    # edge lattices: T=1, U=0, single cells, a target equal to blank, blank != 0
    rng = np.random.default_rng(102)
    T = [1, 1, 5, 7, 2, 9, 4]
    U = [0, 3, 0, 6, 1, 4, 3]
    targets = rng.integers(0, 7, size=(7, 6))  # includes 0..6, so some targets equal blank=2
    case(ref, "edges_N7_V7_blank2", T, U, targets, 7, 2, rng)

    # the same for the one-symbol-per-frame lattice (needs U <= T-1; U == T-1 is a single path)
    rng = np.random.default_rng(105)
    T = [1, 5, 6, 2, 9, 3]
    U = [0, 4, 0, 1, 3, 2]
    case(ref, "edges_modified_N6_V5_blank1", T, U, rng.integers(0, 5, size=(6, 4)), 5, 1, rng)

    # shapes of the reference's own small tests (test_cuda.py:15-21, test_log_softmax.py:26-32)
    rng = np.random.default_rng(103)
    case(ref, "reftest_cuda_V3", [3, 4], [2, 2], rng.integers(1, 2, size=(2, 2)), 3, 0, rng)
    case(ref, "reftest_logsoftmax_V3", [8, 5], [3, 4], rng.integers(1, 2, size=(2, 4)), 3, 0, rng)

    # peaky rows (x20) and an odd vocabulary size
    rng = np.random.default_rng(104)
    T = [12, 30, 17]
    U = [11, 4, 16]
    case(ref, "peaky_N3_V37", T, U, rng.integers(1, 37, size=(3, 16)), 37, 0, rng, sigma=6.0)


if __name__ == "__main__":
    main()
