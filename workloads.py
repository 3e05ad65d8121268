"""Seeded synthetic workloads for the transducer-loss path.

Shapes follow the five benchmark configurations (tiny / typical ASR batch /
log-softmax + modified / large vocabulary / ragged stress).  Lengths and targets
come from ``numpy.random.default_rng(seed)`` so that every machine sees the
same integers; logits come from a second generator seeded from the same seed.
"""
import numpy as np


class Workload:
    def __init__(self, name, logit_lengths, target_lengths, targets, V, blank,
                 from_log_softmax, one_sym_per_frame, reduction, logits_sigma, peaky, seed):
        self.name = name
        self.logit_lengths = np.asarray(logit_lengths, dtype=np.int32)
        self.target_lengths = np.asarray(target_lengths, dtype=np.int32)
        self.targets = np.ascontiguousarray(targets, dtype=np.int32)
        self.V = int(V)
        self.blank = int(blank)
        self.from_log_softmax = bool(from_log_softmax)
        self.one_sym_per_frame = bool(one_sym_per_frame)
        self.reduction = reduction
        self.logits_sigma = float(logits_sigma)
        self.peaky = float(peaky)
        self.seed = int(seed)

    @property
    def N(self):
        return int(self.logit_lengths.size)

    @property
    def rows(self):
        return int((self.logit_lengths.astype(np.int64) * (self.target_lengths.astype(np.int64) + 1)).sum())

    def logits_numpy(self):
        """(rows, V) float32 on the host (use only for sizes that fit comfortably)."""
        rng = np.random.default_rng(self.seed + 1000003)
        x = rng.standard_normal((self.rows, self.V), dtype=np.float32)
        if self.logits_sigma != 1.0:
            x *= np.float32(self.logits_sigma)
        if self.peaky > 0:
            pick = rng.random(self.rows) < self.peaky
            x[pick] *= np.float32(20.0)
        if self.from_log_softmax:
            m = x.max(axis=1, keepdims=True)
            x = x - (m + np.log(np.exp((x - m).astype(np.float64)).sum(axis=1, keepdims=True))).astype(np.float32)
        return np.ascontiguousarray(x, dtype=np.float32)

    def logits_torch(self, device):
        """(rows, V) float32 generated on ``device`` with torch's generator (not
        bit-identical to ``logits_numpy``; used for the large benchmark shapes)."""
        import torch
        g = torch.Generator(device=device)
        g.manual_seed(self.seed + 1000003)
        x = torch.randn((self.rows, self.V), dtype=torch.float32, device=device, generator=g)
        if self.logits_sigma != 1.0:
            x.mul_(self.logits_sigma)
        if self.peaky > 0:
            pick = torch.rand((self.rows, 1), device=device, generator=g) < self.peaky
            x = torch.where(pick, x * 20.0, x)
        if self.from_log_softmax:
            x = torch.log_softmax(x, dim=1)
        return x.contiguous()


def beyond_int32(seed=6, one_sym_per_frame=False):
    """Four utterances of T=1100, U=499 at V=1000: 2.2 million packed rows, 2.2e9 logits
    (more than 2^31 elements, 8.8 GB), plus one degenerate utterance in front so that no
    offset is a round number.  The lattice has 8 waves per workgroup."""
    T = np.array([3, 1100, 1100, 1100, 1100], np.int64)
    U = np.array([1, 499, 499, 499, 499], np.int64)
    rng = np.random.default_rng(seed)
    name = "beyond_int32_N5_V1000%s" % ("_modified" if one_sym_per_frame else "")
    return Workload(name, T, U, _targets(rng, 5, U.max(), 1000), 1000, 0, False,
                    one_sym_per_frame, "mean", 1.0, 0.0, seed)


def _targets(rng, N, max_u, V, zipf=False):
    cols = max(int(max_u), 0)
    if zipf:
        t = rng.zipf(1.1, size=(N, cols))
        t = ((t - 1) % (V - 1)) + 1
    else:
        t = rng.integers(1, V, size=(N, cols))
    return t.astype(np.int32)


def tiny(seed=1, from_log_softmax=False, one_sym_per_frame=False, reduction="mean"):
    """N=4, T~U{20..50}, U~U{5..15}, V=32."""
    rng = np.random.default_rng(seed)
    T = rng.integers(20, 51, size=4)
    U = rng.integers(5, 16, size=4)
    return Workload("tiny_N4_V32", T, U, _targets(rng, 4, U.max(), 32), 32, 0,
                    from_log_softmax, one_sym_per_frame, reduction, 1.0, 0.0, seed)


def asr_batch(seed=2, from_log_softmax=False, one_sym_per_frame=False, reduction="sum",
              N=32, V=500, scale=1.0):
    """N=32, T~U{200..500}, U~U{20..100}, V=500 (``scale`` shrinks T and U for CPU-sized tests)."""
    rng = np.random.default_rng(seed)
    T = np.maximum(1, (rng.integers(200, 501, size=N) * scale).astype(np.int64))
    U = np.maximum(0, (rng.integers(20, 101, size=N) * scale).astype(np.int64))
    if one_sym_per_frame:
        U = np.minimum(U, T - 1)
    name = "asr_N%d_V%d%s%s" % (N, V, "_logsoftmax" if from_log_softmax else "",
                                "_modified" if one_sym_per_frame else "")
    return Workload(name, T, U, _targets(rng, N, U.max(), V), V, 0,
                    from_log_softmax, one_sym_per_frame, reduction, 1.0, 0.0, seed)


def asr_batch_logsoftmax_modified(seed=3, **kw):
    return asr_batch(seed=seed, from_log_softmax=True, one_sym_per_frame=True,
                     reduction="mean", **kw)


def large_vocab(seed=4, N=16, V=5000, scale=1.0):
    """N=16, T~U{100..300}, U~U{10..60}, V=5000, logits N(0, sigma=2), Zipf(1.1) targets."""
    rng = np.random.default_rng(seed)
    T = np.maximum(1, (rng.integers(100, 301, size=N) * scale).astype(np.int64))
    U = np.maximum(0, (rng.integers(10, 61, size=N) * scale).astype(np.int64))
    return Workload("largevocab_N%d_V%d" % (N, V), T, U,
                    _targets(rng, N, U.max(), V, zipf=True), V, 0,
                    False, False, "mean", 2.0, 0.0, seed)


def ragged(seed=5, one_sym_per_frame=False, N=128, V=1000, t_max=1000, u_max=200,
           mu=np.log(100.0), sigma=0.8):
    """N=128, T log-normal clipped to [1, t_max], U~U{0..min(u_max, T)}, 1 % peaky rows.

    Always contains one T=1 and one U=0 utterance.  For the modified lattice U is
    also clamped to T-1 (the recursion is undefined beyond that).
    """
    rng = np.random.default_rng(seed)
    T = np.clip(np.rint(rng.lognormal(mu, sigma, size=N)), 1, t_max).astype(np.int64)
    T[0] = 1
    U = np.array([rng.integers(0, min(u_max, int(t)) + 1) for t in T], dtype=np.int64)
    U[1] = 0
    if one_sym_per_frame:
        U = np.minimum(U, T - 1)
    if U.max() == 0:
        U[-1] = min(u_max, int(T[-1]) - (1 if one_sym_per_frame else 0))
    name = "ragged_N%d_V%d%s" % (N, V, "_modified" if one_sym_per_frame else "")
    return Workload(name, T, U, _targets(rng, N, U.max(), V), V, 0,
                    False, one_sym_per_frame, "mean", 1.0, 0.01, seed)
