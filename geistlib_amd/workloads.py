"""Synthetic workloads of the sampling path: the five benchmark configurations, generated on
the host from fixed seeds so that the CPU oracle and the device see identical bits.

Uniform draws come from the reference's xorshift64* generator (src/engine/sampler.c:35-48),
restated here with Python integers.
"""
from dataclasses import dataclass, field

import numpy as np

_M64 = (1 << 64) - 1


def xorshift_units(seed, n):
    """n successive geist_rng_next_unit values for `seed` (0 is remapped as the reference does)."""
    x = seed if seed else 0x9E3779B97F4A7C15
    out = np.empty(n, dtype=np.float32)
    for i in range(n):
        x ^= x >> 12
        x = (x ^ (x << 25)) & _M64
        x ^= x >> 27
        out[i] = np.float32(((x * 0x2545F4914F6CDD1D) & _M64) >> 40) * np.float32(2.0 ** -24)
    return out, x


@dataclass
class Workload:
    name: str
    logits: np.ndarray                      # [rows, V] float32
    uniforms: np.ndarray                    # [rows] float32
    temperature: float = 1.0
    top_k: int = 0
    top_p: float = 1.0
    min_p: float = 0.0
    rep: float = 1.0
    freq: float = 0.0
    pres: float = 0.0
    history: np.ndarray = None              # [rows, H] int32
    history_len: np.ndarray = None          # [rows] int32
    extra: dict = field(default_factory=dict)

    @property
    def rows(self):
        return self.logits.shape[0]

    @property
    def n_vocab(self):
        return self.logits.shape[1]

    def algorithmic_bytes(self):
        """4V logits + 4H history ids + 8U gathered/scattered distinct ids + 4 B uniform + 4 B id,
        summed over the rows."""
        total = self.rows * (4 * self.n_vocab + 8)
        if self.history is not None:
            for r in range(self.rows):
                h = self.history[r, :self.history_len[r]]
                total += 4 * h.size + 8 * np.unique(h).size
        return int(total)


def zipf_history(g, rows, length, n_vocab, s=1.1):
    w = 1.0 / np.arange(1, n_vocab + 1, dtype=np.float64) ** s
    cdf = np.cumsum(w)
    cdf /= cdf[-1]
    ids = np.searchsorted(cdf, g.random((rows, length)), side="right")
    return np.minimum(ids, n_vocab - 1).astype(np.int32)


def config1(seed=1):
    """One row, V = 128256, logits ~ N(0, 3^2); greedy argmax, then T = 0.8 with one draw."""
    g = np.random.default_rng(seed)
    logits = (g.standard_normal((1, 128256)) * 3).astype(np.float32)
    u, _ = xorshift_units(seed, 1)
    return Workload("cfg1_b1_v128256", logits, u, temperature=0.8)


def config2(seed=2, rows=64, n_vocab=128256, with_penalties=False, history=2048):
    """B = 64 x V = 128256, N(0, 2^2) with 5 positions per row boosted by +10; T = 0.7,
    top-k 40, top-p 0.9, one seeded uniform per row. `with_penalties` adds the penalty stage
    of configuration 3 (Zipf history, rep 1.1 / freq 0.5 / pres 0.3) in front."""
    g = np.random.default_rng(seed)
    logits = (g.standard_normal((rows, n_vocab)) * 2).astype(np.float32)
    for r in range(rows):
        logits[r, g.choice(n_vocab, 5, replace=False)] += np.float32(10)
    u, _ = xorshift_units(seed, rows)
    w = Workload(f"cfg2_b{rows}_v{n_vocab}", logits, u, temperature=0.7, top_k=40, top_p=0.9)
    if with_penalties:
        w.name += f"_pen{history}"
        w.history = zipf_history(g, rows, history, n_vocab)
        w.history_len = np.full(rows, history, dtype=np.int32)
        w.rep, w.freq, w.pres = 1.1, 0.5, 0.3
    return w


def config3(seed=3, rows=128, n_vocab=151936, history=2048):
    """Penalty path: N(0, 2^2); 2048 history ids per row ~ Zipf(1.1); rep 1.1, freq 0.5,
    pres 0.3; T = 1.0, top-p 0.95, min-p 0.05."""
    g = np.random.default_rng(seed)
    logits = (g.standard_normal((rows, n_vocab)) * 2).astype(np.float32)
    u, _ = xorshift_units(seed, rows)
    w = Workload(f"cfg3_b{rows}_v{n_vocab}", logits, u, temperature=1.0, top_p=0.95, min_p=0.05,
                 rep=1.1, freq=0.5, pres=0.3)
    w.history = zipf_history(g, rows, history, n_vocab)
    w.history_len = np.full(rows, history, dtype=np.int32)
    return w


def config4(seed=4, rows=256, n_vocab=262144):
    """Heavy tail: Student-t(nu = 3) x 2.5; top-k 64 then top-p 0.9, T = 0.6; also argmax."""
    g = np.random.default_rng(seed)
    logits = (g.standard_t(3, size=(rows, n_vocab)) * 2.5).astype(np.float32)
    u, _ = xorshift_units(seed, rows)
    return Workload(f"cfg4_b{rows}_v{n_vocab}", logits, u, temperature=0.6, top_k=64, top_p=0.9)


def config5(seed=5, n_seq=32, draft_len=8, n_vocab=128256):
    """Speculative verification: target logits [n_seq, L+1, V] ~ N(0, 2^2); draft probabilities
    q = softmax(target + N(0, 0.5^2)); draft tokens drawn from q; uniforms [n_seq, L+1]."""
    g = np.random.default_rng(seed)
    target = (g.standard_normal((n_seq, draft_len + 1, n_vocab)) * 2).astype(np.float32)
    noisy = target[:, :draft_len, :] + (g.standard_normal((n_seq, draft_len, n_vocab)) * 0.5
                                        ).astype(np.float32)
    x = noisy.astype(np.float64)
    x -= x.max(axis=-1, keepdims=True)
    e = np.exp(x)
    q = (e / e.sum(axis=-1, keepdims=True)).astype(np.float32)
    cdf = np.cumsum(q.astype(np.float64), axis=-1)
    pick = g.random((n_seq, draft_len, 1)) * cdf[..., -1:]
    draft = np.minimum((cdf < pick).sum(axis=-1), n_vocab - 1).astype(np.int32)
    u, _ = xorshift_units(seed, n_seq * (draft_len + 1))
    w = Workload(f"cfg5_s{n_seq}_l{draft_len}_v{n_vocab}", target.reshape(-1, n_vocab), u,
                 temperature=1.0)
    w.extra = {"n_seq": n_seq, "draft_len": draft_len, "q": q, "draft": draft,
               "target": target, "uniforms": u.reshape(n_seq, draft_len + 1)}
    return w
