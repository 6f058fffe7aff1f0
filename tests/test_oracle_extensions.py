"""Pins for the oracle stages that have no reference counterpart (penalties, min-p, the
top-k -> top-p -> min-p chain, speculative verification, session dispatch): identities,
limiting cases, library cross-checks and brute force on tiny inputs, each chosen so that a
dropped term, a wrong sign or a swapped operand fails."""
import ctypes as C
import itertools

import numpy as np
import pytest

from oracle_lib import _fp


# ------------------------------------------------------------------------------- penalties
def test_penalties_identity_and_bincount(oracle):
    g = np.random.default_rng(0)
    n = 500
    row = (g.standard_normal(n) * 3).astype(np.float32)
    hist = g.integers(0, n, 300).astype(np.int32)
    # neutral parameters leave every bit alone
    assert np.array_equal(oracle.penalties(row, hist, 1.0, 0.0, 0.0), row)
    # empty history
    assert np.array_equal(oracle.penalties(row, np.zeros(0, np.int32), 1.3, 0.5, 0.2), row)
    # frequency only: l - f * count, counts from numpy.bincount
    cnt = np.bincount(hist, minlength=n).astype(np.float32)
    out = oracle.penalties(row, hist, 1.0, 0.5, 0.0)
    assert np.array_equal(out, (row - np.float32(0.5) * cnt).astype(np.float32))
    # presence only: applied once however often the id repeats
    out = oracle.penalties(row, hist, 1.0, 0.0, 0.3)
    assert np.array_equal(out, np.where(cnt > 0, row - np.float32(0.3), row).astype(np.float32))
    # repetition only: positive logits shrink by division, negative ones by multiplication, once
    out = oracle.penalties(row, hist, 1.1, 0.0, 0.0)
    want = np.where(cnt > 0, np.where(row > 0, row / np.float32(1.1), row * np.float32(1.1)), row)
    assert np.array_equal(out, want.astype(np.float32))
    assert np.all(out[cnt > 0] <= row[cnt > 0])  # a penalty never raises a logit (rep > 1)
    # all three, in the stated order (repetition, then frequency, then presence)
    out = oracle.penalties(row, hist, 1.2, 0.25, 0.125)
    w = np.where(row > 0, row / np.float32(1.2), row * np.float32(1.2)).astype(np.float32)
    w = (w - (np.float32(0.25) * cnt).astype(np.float32)).astype(np.float32)
    w = (w - np.float32(0.125)).astype(np.float32)
    assert np.array_equal(out, np.where(cnt > 0, w, row))
    # ids outside [0, n) are ignored
    bad = np.array([-1, n, n + 7, -2**31, 3], dtype=np.int32)
    out = oracle.penalties(row, bad, 1.0, 0.0, 1.0)
    want = row.copy()
    want[3] -= 1.0
    assert np.array_equal(out, want)


# -------------------------------------------------------------------- brute-force chain
def brute_chain(row, u, T, top_k, top_p, min_p):
    """Independent float64 statement of the chain; returns (token, distance to slot edge)."""
    n = len(row)
    if T <= 0:
        return int(np.argmax(row)), np.inf
    order = sorted(range(n), key=lambda i: (-float(row[i]), i))
    use_k = 1 < top_k < n
    use_p = 0 < top_p < 1
    use_m = min_p > 0
    x = row.astype(np.float64)
    if not use_k and not use_p and not use_m:
        w = np.exp((x - x.max()) / T)
        ids = list(range(n))
    else:
        ids = order[:min(top_k, 8192)] if use_k else order
        w = np.exp((x[ids] - x[ids].max()) / T)
        w = w / w.sum()
        keep = len(ids)
        if use_p:
            keep = min(keep, int(np.searchsorted(np.cumsum(w), top_p, side="left")) + 1)
        if use_m:
            keep = min(keep, max(1, int(np.sum(w >= min_p * w[0]))))
        ids, w = ids[:keep], w[:keep]
    cdf = np.cumsum(w)
    t = u * cdf[-1]
    j = int(np.searchsorted(cdf, t, side="right"))
    j = min(j, len(ids) - 1)
    lo = cdf[j - 1] if j else 0.0
    return ids[j], min(t - lo, cdf[j] - t) / cdf[-1]


@pytest.mark.parametrize("n", [2, 5, 17, 64, 300])
def test_chain_matches_brute_force(oracle, n):
    g = np.random.default_rng(n)
    checked = 0
    for trial in range(60):
        row = (g.standard_normal(n) * g.choice([0.5, 2.0, 4.0])).astype(np.float32)
        T = float(g.choice([0.5, 0.7, 1.0, 1.8]))
        top_k = int(g.choice([0, 1, 2, 3, n // 2, n, n + 5]))
        top_p = float(g.choice([1.0, 0.95, 0.9, 0.5, 0.1, 0.0]))
        min_p = float(g.choice([0.0, 0.02, 0.2, 0.9, 1.0]))
        for _ in range(6):
            u = float(np.float32(g.integers(0, 1 << 24)) / np.float32(1 << 24))
            want, dist = brute_chain(row, u, T, top_k, top_p, min_p)
            got, info = oracle.chain_u(row, u, temperature=T, top_k=top_k, top_p=top_p, min_p=min_p)
            if dist > 1e-5:  # away from a slot edge fp32 vs fp64 cannot change the slot
                assert got == want, (n, trial, T, top_k, top_p, min_p, u)
                checked += 1
    assert checked > 200


def test_chain_limits(oracle):
    g = np.random.default_rng(3)
    row = (g.standard_normal(200) * 2).astype(np.float32)
    for u in (0.0, 0.25, 0.5, 0.999):
        # top_p = 1 and min_p = 0 switch the filters off
        assert oracle.chain_u(row, u, temperature=0.8, top_k=10, top_p=1.0)[0] == \
            oracle.top_k_u(row, 10, 0.8, u)[0]
        # top_k >= n leaves top-p alone
        assert oracle.chain_u(row, u, temperature=0.8, top_k=200, top_p=0.7)[0] == \
            oracle.top_p_u(row, 0.7, 0.8, u)[0]
        # min_p = 1 keeps only the ties of the maximum -> argmax here
        assert oracle.chain_u(row, u, temperature=0.8, min_p=1.0)[0] == oracle.argmax(row)
        # a vanishing top_p keeps exactly one entry -> argmax
        assert oracle.chain_u(row, u, temperature=0.8, top_p=1e-9)[0] == oracle.argmax(row)
        # T -> 0+ collapses onto the argmax
        assert oracle.chain_u(row, u, temperature=1e-4, top_k=40, top_p=0.9)[0] == oracle.argmax(row)
    # greedy consumes no draw
    assert oracle.chain_u(row, 0.3, temperature=0.0, top_k=40)[1].draws == 0
    assert oracle.chain_u(row, 0.3, temperature=0.7, top_k=40)[1].draws == 1


def test_min_p_set_is_logit_threshold(oracle):
    """{i : p_i >= min_p * p_max}  <=>  l_i / T >= l_max / T + ln(min_p); the draw never leaves it."""
    g = np.random.default_rng(11)
    row = (g.standard_normal(4000) * 2).astype(np.float32)
    T, min_p = 0.9, 0.05
    thr = row.max() + T * np.log(min_p)
    allowed = set(np.nonzero(row >= thr - 1e-4)[0].tolist())
    inside = set(np.nonzero(row >= thr + 1e-4)[0].tolist())
    seen = set()
    for k in range(400):
        tok, info = oracle.chain_u(row, (k + 0.5) / 400, temperature=T, min_p=min_p)
        assert tok in allowed
        assert len(inside) <= info.n_keep <= len(allowed)
        seen.add(tok)
    assert len(seen) > 1


def test_temperature_closed_forms(oracle):
    # uniform logits: sum == n exactly and id == floor(u * n)
    for n in (5, 64, 1000):
        row = np.full(n, 0.75, dtype=np.float32)
        p, s = oracle.softmax_into(row, 1.3)
        assert s == float(n) and np.all(p == 1.0)
        for k in range(50):
            u = float(np.float32((k * 331 + 7) % 1024) / np.float32(1024))
            assert oracle.temperature_u(row, 1.3, u)[0] == int(np.floor(u * n))
    # two-point row: P(1) = 1 / (1 + e^{-d/T})
    row = np.array([0.0, 2.0], dtype=np.float32)
    p1 = 1.0 / (1.0 + np.exp(-2.0 / 0.5))
    for u in np.linspace(0.001, 0.999, 97):
        u = float(np.float32(u))
        want = 0 if u < 1 - p1 else 1
        if abs(u - (1 - p1)) > 1e-4:
            assert oracle.temperature_u(row, 0.5, u)[0] == want
    # shift invariance (values chosen so the shift is exact in fp32)
    g = np.random.default_rng(1)
    row = (np.round(g.standard_normal(300) * 64) / 64).astype(np.float32)
    for u in (0.1, 0.6, 0.93):
        assert oracle.temperature_u(row, 0.8, u)[0] == oracle.temperature_u(row + np.float32(16), 0.8, u)[0]
    # library cross-check of the normalised probabilities (float64 softmax)
    row = (g.standard_normal(5000) * 2).astype(np.float32)
    pn, _ = oracle.softmax_normalised(row, 0.7)
    x = row.astype(np.float64) / 0.7
    want = np.exp(x - x.max())
    want /= want.sum()
    assert np.allclose(pn, want, rtol=1e-5, atol=0)  # fp32 scaling of the exponent


# ---------------------------------------------------------------------- session dispatch
def test_dispatch_precedence_and_draw_counts(oracle):
    g = np.random.default_rng(21)
    row = (g.standard_normal(400) * 2).astype(np.float32)
    table = [  # (T, top_k, top_p) -> (expected mode, draws)
        ((0.0, 40, 0.9), ("argmax", 0)), ((0.0, 0, 1.0), ("argmax", 0)),
        ((0.7, 40, 0.9), ("top_k", 1)),   # top_k takes precedence; top_p ignored
        ((0.7, 40, 1.0), ("top_k", 1)), ((0.7, 1, 0.9), ("top_p", 1)), ((0.7, 0, 0.9), ("top_p", 1)),
        ((0.7, 0, 1.0), ("temperature", 1)), ((0.7, 0, 0.0), ("temperature", 1)),  # top_p <= 0 -> 1.0
        ((0.7, 0, -3.0), ("temperature", 1)), ((0.7, 400, 0.9), ("temperature", 1)),  # k >= n
        ((0.7, 100000, 0.5), ("temperature", 1)), ((0.7, 0, 1.5), ("temperature", 1)),
    ]
    for (T, k, p), (mode, draws) in table:
        s = oracle.session(T, p, k, seed=0xC0FFEE)
        shadow = oracle.rng(0xC0FFEE)
        tok = oracle.finalize_row(s, row)
        u = oracle.next_unit(shadow) if draws else None
        if mode == "argmax":
            want = oracle.argmax(row)
        elif mode == "top_k":
            want = oracle.top_k_u(row, k, T, u)[0]
        elif mode == "top_p":
            want = oracle.top_p_u(row, p, T, u)[0]
        else:
            want = oracle.temperature_u(row, T, u)[0]
        assert tok == want, (T, k, p)
        if not draws:
            shadow = oracle.rng(0xC0FFEE)
        assert int(s.rng.state) == int(shadow.state), "draw count differs"
        assert oracle.lib.oracle_session_draws(C.byref(s), row.size) == draws
    # default seed when random_seed == 0 (arch_state.c:1173), and apply_opts keeps it
    s = oracle.session(0.5, 1.0, 0, seed=0)
    assert int(s.rng.state) == 0xCAFEBABE1234


def test_batch_shares_one_rng_in_row_order(oracle):
    g = np.random.default_rng(8)
    rows = (g.standard_normal((6, 300)) * 2).astype(np.float32)
    s = oracle.session(0.8, 1.0, 20, seed=5)
    got = oracle.finalize_batch(s, rows)
    r = oracle.rng(5)
    want = [oracle.top_k_u(rows[i], 20, 0.8, oracle.next_unit(r))[0] for i in range(6)]
    assert got.tolist() == want


def test_softcap_is_monotone_and_only_for_stochastic(oracle):
    g = np.random.default_rng(2)
    row = (g.standard_normal(1000) * 20).astype(np.float32)
    capped = oracle.softcap(row, 30.0)
    assert np.allclose(capped, np.tanh(row.astype(np.float64) / 30) * 30, rtol=1e-6)
    assert oracle.argmax(capped) == oracle.argmax(row)
    s = oracle.session(0.9, 1.0, 0, seed=3)
    u = oracle.next_unit(oracle.rng(3))
    assert oracle.finalize_row(s, row, softcap=30.0) == oracle.temperature_u(capped, 0.9, u)[0]


# ------------------------------------------------------------------- speculative verify
def _softmax64(x, T):
    e = np.exp((x - x.max()) / T)
    return e / e.sum()


def test_spec_verify_special_cases(oracle):
    g = np.random.default_rng(4)
    L, n = 4, 50
    target = (g.standard_normal((L + 1, n)) * 2).astype(np.float32)
    pn = np.stack([oracle.softmax_normalised(target[j], 1.0)[0] for j in range(L)])
    draft = g.integers(0, n, L).astype(np.int32)
    u = np.array([0.999, 0.999, 0.999, 0.999, 0.4], dtype=np.float32)
    # q == p: every position is accepted whatever the uniforms; the bonus is a temperature draw
    nacc, out = oracle.spec_verify(target, pn, draft, u, 1.0)
    assert nacc == L and out[:L].tolist() == draft.tolist()
    assert out[L] == oracle.temperature_u(target[L], 1.0, 0.4)[0]
    # disjoint supports: q puts all mass on a token p gives ~nothing -> reject at 0, residual == p
    q = np.zeros((L, n), dtype=np.float32)
    tgt = target.copy()
    tgt[0, 7] = -200.0  # p(7) == 0 in fp32
    q[:, 7] = 1.0
    d2 = np.full(L, 7, dtype=np.int32)
    for uu in (0.05, 0.5, 0.95):
        u2 = np.array([0.0, 0, 0, 0, uu], dtype=np.float32)
        nacc, out = oracle.spec_verify(tgt, q, d2, u2, 1.0)
        assert nacc == 0
        p0 = oracle.softmax_normalised(tgt[0], 1.0)[0].astype(np.float64)
        cdf = np.cumsum(p0)
        assert out[0] == int(np.searchsorted(cdf, uu * cdf[-1], side="right"))
    # greedy: exact-match prefix, emitted token is the target's argmax
    am = np.array([oracle.argmax(target[j]) for j in range(L + 1)], dtype=np.int32)
    d3 = am[:L].copy()
    d3[2] = (d3[2] + 1) % n
    nacc, out = oracle.spec_verify(target, pn, d3, u, 0.0)
    assert nacc == 2 and out[:3].tolist() == [am[0], am[1], am[2]]
    nacc, out = oracle.spec_verify(target, pn, am[:L].copy(), u, 0.0)
    assert nacc == L and out.tolist() == am.tolist()


@pytest.mark.parametrize("n", [3, 6])
def test_spec_verify_preserves_target_distribution(oracle, n):
    """One draft position: sum_x q(x) * P(emit y | x) must equal p(y). Integrated on a uniform
    grid of (u_accept, u_resample); the grid resolves probabilities to ~1/G."""
    g = np.random.default_rng(n)
    G = 192
    target = (g.standard_normal((2, n)) * 1.5).astype(np.float32)
    q = _softmax64(g.standard_normal(n) * 1.5, 1.0).astype(np.float32)[None, :]
    p = _softmax64(target[0].astype(np.float64), 1.0)
    us = (np.arange(G, dtype=np.float64) + 0.5) / G
    out_mass = np.zeros(n)
    for x in range(n):
        draft = np.array([x], dtype=np.int32)
        for ua in us:
            # acceptance does not depend on the resample uniform: test once, then sweep
            nacc, out = oracle.spec_verify(target, q, draft, np.array([ua, 0.5], np.float32), 1.0)
            if nacc == 1:
                out_mass[x] += q[0, x] / G
            else:
                for ur in us:
                    _, o2 = oracle.spec_verify(target, q, draft, np.array([ua, ur], np.float32), 1.0)
                    out_mass[o2[0]] += q[0, x] / (G * G)
    assert np.allclose(out_mass, p, atol=3.0 / G), (out_mass, p)


# ------------------------------------------------------------------ log-probability scoring
def test_logprob_at_closed_forms_and_library(oracle):
    """tools/eval_geist.c:63-73. Pins: uniform logits -> -log(n) for every token; two-point rows;
    shift invariance; scipy's float64 log_softmax of the same fp32 values."""
    from scipy.special import log_softmax
    n = 1000
    assert oracle.logprob_at(np.full(n, 3.25, np.float32), 17) == pytest.approx(-np.log(n), abs=1e-13)
    row = np.array([0.0, np.log(3.0)], dtype=np.float32)      # probabilities 1/4 and 3/4
    d = float(row[1]) - float(row[0])
    assert oracle.logprob_at(row, 1) == pytest.approx(-np.log1p(np.exp(-d)), abs=1e-14)
    assert oracle.logprob_at(row, 0) == pytest.approx(-d - np.log1p(np.exp(-d)), abs=1e-14)
    g = np.random.default_rng(3)
    x = (g.standard_normal(5000) * 4).astype(np.float32)
    want = log_softmax(x.astype(np.float64))
    # the reference subtracts the maximum in fp32 before widening, so against an all-float64
    # library the differences carry fp32 rounding (~1e-7 each); with the same fp32 differences
    # fed to numpy's own exp / sum / log the agreement is to the last few bits
    d32 = (x - x.max()).astype(np.float32).astype(np.float64)
    same = d32 - np.log(np.sum(np.exp(d32)))
    for t in (0, 1, 4999, int(np.argmax(x)), int(np.argmin(x))):
        assert oracle.logprob_at(x, t) == pytest.approx(want[t], abs=2e-6)
        assert oracle.logprob_at(x, t) == pytest.approx(same[t], abs=1e-12)
    probs = np.exp([oracle.logprob_at(x[:50], t) for t in range(50)])
    assert probs.sum() == pytest.approx(1.0, abs=1e-12)
