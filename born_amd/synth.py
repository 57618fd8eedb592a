"""Seeded synthetic workloads of the five benchmark configurations (numpy PCG64).

Every generator returns plain numpy arrays so the same inputs can be handed to the HIP path and to
a checker.  `rows` limits how many rows are generated (tests use a slice of the big configurations).
"""
from dataclasses import dataclass, field

import numpy as np

BASE_SEED = 20251125


@dataclass
class Workload:
    name: str
    logits: np.ndarray                 # [B, V] fp32
    uniforms: np.ndarray               # [B] fp32 in [0, 1)
    temperature: float = 1.0
    top_k: int = 0
    top_p: float = 1.0
    rep: float = 1.0
    history: np.ndarray = None         # [B, H] int32 or None
    extra: dict = field(default_factory=dict)

    def algorithmic_bytes(self):
        """One read of the logits + one read of the history + uniforms in + tokens out."""
        B = self.logits.shape[0]
        n = self.logits.nbytes + 4 * B + 4 * B
        if self.history is not None:
            n += self.history.nbytes
        return n


def _rng(seed, tag):
    return np.random.Generator(np.random.PCG64([seed, tag]))


def c1(step=0, seed=BASE_SEED):
    """B=1, V=32000, N(0, 2^2); T=0.8, k=40, p=0.95, rep=1.1 over 64 uniform history ids; fresh per step."""
    r = _rng(seed, 1000 + step)
    V = 32000
    x = (r.standard_normal((1, V), dtype=np.float32) * np.float32(2.0)).astype(np.float32)
    h = r.integers(0, V, size=(1, 64), dtype=np.int32)
    u = r.random(1, dtype=np.float32)
    return Workload("C1", x, u, 0.8, 40, 0.95, 1.1, h)


def c2(rows=64, seed=BASE_SEED):
    """B=64, V=32000, N(0,1) + 8 spikes of +8 per row; greedy and T=1 full-vocab multinomial."""
    r = _rng(seed, 2)
    V = 32000
    x = r.standard_normal((rows, V), dtype=np.float32)
    for b in range(rows):
        x[b, r.choice(V, 8, replace=False)] += np.float32(8.0)
    u = r.random(rows, dtype=np.float32)
    return Workload("C2", x, u, 1.0, 0, 1.0, 1.0, None)


def c3(rows=256, seed=BASE_SEED, vocab=128256, hist=512):
    """B=256, V=128256, N(0, 1.5^2) + 20 spikes U(6,12); T=0.7, k=50, p=0.9, rep=1.15, H=512 Zipf(1.1)."""
    r = _rng(seed, 3)
    x = (r.standard_normal((rows, vocab), dtype=np.float32) * np.float32(1.5)).astype(np.float32)
    for b in range(rows):
        pos = r.choice(vocab, 20, replace=False)
        x[b, pos] += r.uniform(6.0, 12.0, size=20).astype(np.float32)
    h = ((r.zipf(1.1, size=(rows, hist)) - 1) % vocab).astype(np.int32)
    u = r.random(rows, dtype=np.float32)
    return Workload("C3", x, u, 0.7, 50, 0.9, 1.15, h)


def c4(rows=64, gamma=5, seed=BASE_SEED, vocab=32000):
    """Speculative verify: target N(0,1), draft = target + N(0, 0.5^2), T=1; draft tokens drawn from
    softmax(draft) with their own seeded uniforms."""
    r = _rng(seed, 4)
    t = r.standard_normal((rows, gamma, vocab), dtype=np.float32)
    d = (t + r.standard_normal((rows, gamma, vocab), dtype=np.float32) * np.float32(0.5)).astype(np.float32)
    ud = r.random((rows, gamma))
    q = d.astype(np.float64)
    q = np.exp(q - q.max(axis=-1, keepdims=True))
    cdf = np.cumsum(q, axis=-1)
    cdf /= cdf[..., -1:]
    toks = np.minimum((cdf <= ud[..., None]).sum(axis=-1), vocab - 1).astype(np.int32)
    u_acc = r.random((rows, gamma), dtype=np.float32)
    u_res = r.random(rows, dtype=np.float32)
    w = Workload("C4", t.reshape(rows * gamma, vocab), u_res, 1.0)
    w.extra = dict(target=t, draft=d, draft_tokens=toks, u_acc=u_acc, u_res=u_res, gamma=gamma)
    return w


def c5(rows=1024, seed=BASE_SEED, vocab=152064, hist=2048):
    """B=1024, V=152064, N(0,1); k off, p=0.99, T=1.2, rep=1.05 over 2048 uniform history ids."""
    r = _rng(seed, 5)
    x = r.standard_normal((rows, vocab), dtype=np.float32)
    h = r.integers(0, vocab, size=(rows, hist), dtype=np.int32)
    u = r.random(rows, dtype=np.float32)
    return Workload("C5", x, u, 1.2, 0, 0.99, 1.05, h)
