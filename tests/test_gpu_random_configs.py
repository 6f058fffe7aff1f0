"""Differential test over random configurations: batch shape, vocabulary, sampling mode, penalties,
history, soft-cap and logit distribution are all drawn from a seeded generator and every token id
is compared with the oracle (penalties -> soft-cap -> chain), under the counted-exception rule of
the other parity tests."""
import numpy as np
import pytest

from gpu_util import compare_ids, fuzz_seeds, run_rows

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hs():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from geistlib_amd import HipSampler
    s = HipSampler(max_rows=24, max_vocab=70000)
    yield s
    s.close()


def _case(g):
    rows = int(g.integers(1, 25))
    n = int(g.choice([1, 2, 3, 7, 64, 255, 256, 257, 1000, 1024, 4097, 8192, 8193, 20000, 50257,
                      65536, 70000]))
    kind = g.choice(["normal", "wide", "peaked", "quantised", "ties", "student"])
    if kind == "normal":
        x = g.standard_normal((rows, n)) * 2
    elif kind == "wide":
        x = g.standard_normal((rows, n)) * 0.3
    elif kind == "peaked":
        x = g.standard_normal((rows, n)) * 7
    elif kind == "quantised":
        x = np.round(g.standard_normal((rows, n)) * 3 * 4) / 4
    elif kind == "ties":
        x = g.integers(-3, 4, (rows, n)).astype(np.float64)
    else:
        x = g.standard_t(3, (rows, n)) * 2.5
    x = x.astype(np.float32)
    if g.random() < 0.25 and n > 8:               # banned tokens: -inf inside the row
        x[g.random((rows, n)) < 0.1] = -np.inf
        x[:, int(g.integers(0, n))] = 1.0         # at least one finite logit per row
    mode = g.choice(["argmax", "temperature", "top_k", "top_p", "min_p", "chain", "k_p"])
    prm = dict(temperature=float(g.choice([0.5, 0.7, 1.0, 1.3])), top_k=0, top_p=1.0, min_p=0.0)
    if mode == "argmax":
        prm["temperature"] = 0.0
    if mode in ("top_k", "chain", "k_p"):
        prm["top_k"] = int(g.choice([2, 5, 40, 64, 128, 129, 300, 1000]))
    if mode in ("top_p", "chain", "k_p"):
        prm["top_p"] = float(g.choice([0.3, 0.8, 0.9, 0.95, 0.99]))
    if mode in ("min_p", "chain"):
        prm["min_p"] = float(g.choice([0.001, 0.02, 0.05, 0.3]))
    pen = None
    if g.random() < 0.5 and n > 1:
        H = int(g.choice([1, 17, 300, 2048]))
        hist = g.integers(0, n, (rows, H)).astype(np.int32)
        hl = g.integers(0, H + 1, rows).astype(np.int32)
        lowering = g.random() < 0.7            # the common case has its own (lazy) code path
        pen = dict(hist=hist, hl=hl,
                   rep=float(g.choice([1.0, 1.1, 1.5]) if lowering else g.choice([0.8, 1.2])),
                   freq=float(g.choice([0.0, 0.3, 0.5]) if lowering else g.choice([-0.2, 0.4])),
                   pres=float(g.choice([0.0, 0.3]) if lowering else g.choice([-0.1, 0.2])))
    cap = float(g.choice([0.0, 0.0, 30.0, 5.0]))
    u = (g.integers(0, 1 << 24, rows) / np.float32(1 << 24)).astype(np.float32)
    pad, lead = int(g.choice([0, 0, 1, 3, 4, 64])), int(g.choice([0, 0, 1, 2, 4]))
    allowed = None
    if g.random() < 0.35:                         # a grammar mask: from a handful to most tokens
        density = float(g.choice([0.001, 0.05, 0.5, 0.97]))
        shared = g.random() < 0.3
        allowed = g.random((1 if shared else rows, n)) < density
        allowed[:, int(g.integers(0, n))] = True
        dens = density
    else:
        dens = None
    return x, u, prm, pen, cap, pad, lead, allowed, (
        f"{kind} rows={rows} n={n} {mode} {prm} pen={pen is not None} cap={cap} pad={pad} "
        f"lead={lead} mask={dens}")


@pytest.mark.parametrize("seed", fuzz_seeds(16))
def test_random_configurations_match_oracle(hs, oracle, seed):
    from geistlib_amd import SampleParams
    g = np.random.default_rng(1000 + seed)
    near_total = 0
    for case in range(14):
        x, u, prm, pen, cap, pad, lead, allowed, what = _case(g)
        print(f"seed {seed} case {case}: {what}", flush=True)
        kw = dict(prm)
        if pen is not None:
            kw.update(rep=pen["rep"], freq=pen["freq"], pres=pen["pres"])
        p = SampleParams.make(softcap=cap, **kw)
        hs.set_logits_hint(bool(g.random() < 0.5))     # either way of loading, the same ids
        got = run_rows(hs, torch, x, u, p, None if pen is None else pen["hist"],
                       None if pen is None else pen["hl"], pad=pad, lead=lead, allowed=allowed)
        res = []
        for r in range(x.shape[0]):
            row = x[r]
            if pen is not None:
                row = oracle.penalties(row, pen["hist"][r, :pen["hl"][r]], pen["rep"], pen["freq"],
                                       pen["pres"])
            if cap > 0 and prm["temperature"] > 0:
                row = oracle.softcap(row, cap)
            if allowed is not None:               # after the penalties and the cap
                row = np.where(allowed[r if allowed.shape[0] > 1 else 0], row, -np.inf)
                row = row.astype(np.float32)
            if prm["temperature"] <= 0:
                res.append((oracle.argmax(row), None))
            else:
                res.append(oracle.chain_u(row, float(u[r]), **prm))
        near_total += compare_ids(got, [t for t, _ in res], [i for _, i in res], what)
    assert near_total <= 2


# ------------------------------------------------------------------- speculative verify
@pytest.fixture(scope="module")
def hs_spec():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from geistlib_amd import HipSampler
    s = HipSampler(max_rows=72, max_vocab=50257)
    yield s
    s.close()


def _spec_matches(oracle, target, q, draft, u, T, nacc, out):
    want_n, want = oracle.spec_verify(target, q, draft, u, T)
    return nacc == want_n and out[:want_n + 1].tolist() == want[:want_n + 1].tolist()


@pytest.mark.parametrize("seed", fuzz_seeds(8))
def test_random_spec_verify_matches_oracle(hs_spec, oracle, seed):
    """Random draft length, batch, vocabulary, temperature, soft-cap and draft quality, dense and
    point-mass drafts. A sequence that differs must be explained by a uniform within 2e-6 of a
    decision boundary (found by nudging each uniform of that sequence); those are counted."""
    from gpu_util import to_dev
    g = np.random.default_rng(5000 + seed)
    near = 0
    for case in range(6):
        n_seq, L = int(g.integers(1, 9)), int(g.integers(1, 9))
        n = int(g.choice([2, 64, 257, 1000, 4097, 8193, 20000, 50257]))
        T = float(g.choice([0.0, 0.7, 1.0, 1.3]))
        cap = float(g.choice([0.0, 0.0, 5.0, 30.0]))
        dense = g.random() < 0.6
        sigma = float(g.choice([0.05, 0.5, 2.0]))
        what = f"seed {seed} case {case}: n_seq={n_seq} L={L} n={n} T={T} cap={cap} dense={dense}"
        print(what, flush=True)
        target = (g.standard_normal((n_seq, L + 1, n)) * 2.5).astype(np.float32)
        noisy = target[:, :L, :].astype(np.float64) + g.standard_normal((n_seq, L, n)) * sigma
        noisy -= noisy.max(axis=-1, keepdims=True)
        e = np.exp(noisy)
        q = (e / e.sum(axis=-1, keepdims=True)).astype(np.float32)
        cdf = np.cumsum(q.astype(np.float64), axis=-1)
        pick = g.random((n_seq, L, 1)) * cdf[..., -1:]
        draft = np.minimum((cdf < pick).sum(axis=-1), n - 1).astype(np.int32)
        if not dense:
            q = np.zeros_like(q)
            np.put_along_axis(q, draft[..., None].astype(np.int64), 1.0, axis=-1)
        u = (g.integers(0, 1 << 24, (n_seq, L + 1)) / np.float32(1 << 24)).astype(np.float32)
        out = torch.full((n_seq, L + 1), -9, dtype=torch.int32, device="cuda")
        nacc = torch.full((n_seq,), -9, dtype=torch.int32, device="cuda")
        hs_spec.spec_verify(to_dev(target, torch), to_dev(q, torch) if dense else None,
                            to_dev(draft, torch), to_dev(u, torch), T, out, nacc, softcap=cap)
        hs_spec.sync()
        out, nacc = out.cpu().numpy(), nacc.cpu().numpy()
        for s in range(n_seq):
            tg = target[s]
            if cap > 0 and T > 0:
                tg = np.stack([oracle.softcap(tg[j], cap) for j in range(L + 1)])
            if _spec_matches(oracle, tg, q[s], draft[s], u[s], T, nacc[s], out[s]):
                continue
            explained = False
            for j in range(L + 1):
                for d in (-2e-6, 2e-6):
                    u2 = u[s].copy()
                    u2[j] = np.float32(min(max(float(u2[j]) + d, 0.0), 1 - 2.0 ** -24))
                    explained |= _spec_matches(oracle, tg, q[s], draft[s], u2, T, nacc[s], out[s])
            assert explained, (what, s, nacc[s], out[s])
            near += 1
    assert near <= 2


# --------------------------------------------------------- probabilities and log-probabilities
@pytest.mark.parametrize("seed", fuzz_seeds(6))
def test_random_softmax_and_logprob_rows(hs, oracle, seed):
    """geist_hip_softmax_rows and geist_hip_logprob_rows over random shapes, strides, penalties,
    temperatures and caps: probabilities within 2e-7 relative of the oracle's (the contract is
    1e-5), log-probabilities within 1e-9 absolute."""
    from geistlib_amd import HipSampler, SampleParams
    from gpu_util import to_dev
    g = np.random.default_rng(9000 + seed)
    for case in range(8):
        rows = int(g.integers(1, 13))
        n = int(g.choice([1, 2, 5, 64, 257, 1000, 4097, 8193, 20000, 65536, 70000]))
        pad = int(g.choice([0, 0, 1, 4, 7]))
        T = float(g.choice([0.5, 1.0, 1.7]))
        cap = float(g.choice([0.0, 0.0, 5.0, 30.0]))
        scale = float(g.choice([0.3, 2.0, 8.0]))
        with_pen = g.random() < 0.4 and n > 1
        what = f"seed {seed} case {case}: rows={rows} n={n} pad={pad} T={T} cap={cap} pen={with_pen}"
        print(what, flush=True)
        x = (g.standard_normal((rows, n)) * scale).astype(np.float32)
        buf = np.full((rows, n + pad), 3e38, dtype=np.float32)
        buf[:, :n] = x
        d = to_dev(buf, torch)[:, :n]
        kw, hist, hl, d_h, d_hl = {}, None, None, None, None
        if with_pen:
            H = int(g.choice([3, 200, 2048]))
            hist = g.integers(0, n, (rows, H)).astype(np.int32)
            hl = g.integers(0, H + 1, rows).astype(np.int32)
            d_h, d_hl = to_dev(hist, torch), to_dev(hl, torch)
            kw = dict(rep=1.2, freq=0.25, pres=0.5)
        probs = torch.full((rows, n + pad), -1.0, dtype=torch.float32, device="cuda")
        hs.softmax(HipSampler.rows(d, d_h, d_hl), SampleParams.make(temperature=T, softcap=cap, **kw),
                   probs[:, :n])
        hs.sync()
        got = probs.cpu().numpy()
        assert np.all(got[:, n:] == -1.0), what        # nothing written between the rows
        K = 5
        tok = g.integers(0, n, (rows, K)).astype(np.int32)
        lp = torch.zeros((rows, K), dtype=torch.float64, device="cuda")
        hs.logprob(d, to_dev(tok, torch), lp, softcap=cap)
        hs.sync()
        lp = lp.cpu().numpy()
        for r in range(rows):
            row = x[r]
            if with_pen:
                row = oracle.penalties(row, hist[r, :hl[r]], 1.2, 0.25, 0.5)
            if cap > 0:
                row = oracle.softcap(row, cap)
            want, _ = oracle.softmax_normalised(row, T)
            err = np.max(np.abs(got[r, :n] - want) / np.maximum(want, 1e-38))
            assert err < 2e-7, (what, r, err)
            plain = oracle.softcap(x[r], cap) if cap > 0 else x[r]
            for j in range(K):
                assert abs(lp[r, j] - oracle.logprob_at(plain, int(tok[r, j]))) < 1e-9, (what, r, j)
