"""geist_hip_sampler_set_sums(GEIST_HIP_SUMS_FAST): the sums of exponentials from the hardware's
2^z (relative error about 1e-7) instead of the bit-exact expf, every weight that is compared with
a share of a sum still exact. Ids are the oracle's except where the oracle's own decision lies
within the contract's tolerance of an edge (compare_ids counts those rows; the counts are printed
and bounded), normalised probabilities are within 1e-6 relative, and switching back to the exact
mode gives the exact results again."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")

from gpu_util import compare_ids, run_rows, to_dev  # noqa: E402


@pytest.fixture()
def hs():
    from geistlib_amd import HipSampler
    s = HipSampler(max_rows=128, max_vocab=160000)
    yield s
    s.close()


def P(**kw):
    from geistlib_amd import SampleParams
    return SampleParams.make(**kw)


CASES = [
    # (rows, n, logit scale, sampling parameters, penalties)
    (64, 60000, 2.5, dict(temperature=0.8), False),                      # exp-sum pass + walk
    (96, 128256, 0.7, dict(temperature=1.3), False),                     # flat rows
    (32, 151936, 2.0, dict(temperature=1.0, top_p=0.95, min_p=0.05), True),
    (32, 100000, 2.0, dict(temperature=1.0, top_p=0.9), False),
    (16, 128256, 0.5, dict(temperature=1.0, top_p=0.9), False),          # whole-row walks
    (8, 128256, 2.0, dict(temperature=0.9), False),      # chunks of 2048, more than one kernel
    (24, 50001, 2.0, dict(temperature=0.9), False),      # ragged rows: no float4 loads
    (64, 60000, 2.5, dict(temperature=0.8), True),       # penalties: the workgroups meet
]


@pytest.mark.parametrize("rows,n,scale,kw,pen", CASES)
def test_ids_with_fast_sums(hs, oracle, rows, n, scale, kw, pen):
    print(f"fast sums rows={rows} n={n} scale={scale} {kw} pen={pen}", flush=True)
    g = np.random.default_rng(rows + n)
    x = (g.standard_normal((rows, n)) * scale).astype(np.float32)
    hist = hl = None
    pk = {}
    if pen:
        hist = g.integers(0, n, (rows, 300)).astype(np.int32)
        hl = np.full(rows, 300, dtype=np.int32)
        pk = dict(rep=1.2, freq=0.4, pres=0.2)
    near_total = 0
    for call in range(3):
        u = g.random(rows).astype(np.float32)
        res = []
        for r in range(rows):
            row = oracle.penalties(x[r], hist[r], 1.2, 0.4, 0.2) if pen else x[r]
            res.append(oracle.chain_u(row, float(u[r]), **kw))
        want, infos = [t for t, _ in res], [i for _, i in res]
        hs.set_sums(fast=True)
        got = run_rows(hs, torch, x, u, P(**kw, **pk), history=hist, history_len=hl)
        near_total += compare_ids(got, want, infos, f"fast sums, call {call}")
        hs.set_sums(fast=False)
        exact = run_rows(hs, torch, x, u, P(**kw, **pk), history=hist, history_len=hl)
        assert compare_ids(exact, want, infos, f"exact sums, call {call}") == 0
    print(f"  rows within the tolerance of an edge that differ: {near_total} of {3 * rows}", flush=True)
    assert near_total <= 2


def test_probabilities_with_fast_sums(hs, oracle):
    from geistlib_amd import HipSampler
    rows, n, T = 4, 70001, 0.9
    g = np.random.default_rng(9)
    x = (g.standard_normal((rows, n)) * 3).astype(np.float32)
    d = to_dev(x, torch)
    probs = torch.empty((rows, n), dtype=torch.float32, device="cuda")
    hs.set_sums(fast=True)
    hs.softmax(HipSampler.rows(d), P(temperature=T), probs)
    hs.sync()
    got = probs.cpu().numpy()
    for r in range(rows):
        want, _ = oracle.softmax_normalised(x[r], T)
        big = want > 1e-30
        assert np.max(np.abs(got[r][big] / want[big] - 1.0)) < 1e-6, r   # the tolerance: 1e-6 relative
        assert abs(float(got[r].astype(np.float64).sum()) - 1.0) < 1e-5
    hs.set_sums(fast=False)
    hs.softmax(HipSampler.rows(d), P(temperature=T), probs)
    hs.sync()
    for r in range(rows):
        assert np.array_equal(probs[r].cpu().numpy(), oracle.softmax_normalised(x[r], T)[0]), r


def test_spec_verify_with_fast_sums(hs, oracle):
    from test_gpu_sampling import _run_spec, _spec_case
    n_seq, L, n, T = 12, 6, 60000, 0.9
    target, q, draft, u = _spec_case(123, n_seq, L, n)
    hs.set_sums(fast=True)
    differ = 0
    for call in range(2):
        nacc, out = _run_spec(hs, target, q, draft, u, T)
        for s in range(n_seq):
            want_n, want = oracle.spec_verify(target[s], q[s], draft[s], u[s], T)
            same = nacc[s] == want_n and out[s, :want_n + 1].tolist() == want[:want_n + 1].tolist()
            differ += 0 if same else 1
    print(f"  sequences that differ from the oracle's with fast sums: {differ} of {2 * n_seq}", flush=True)
    assert differ <= 1      # (an acceptance or a residual draw within 1e-7 of its edge)
    hs.set_sums(fast=False)
    nacc, out = _run_spec(hs, target, q, draft, u, T)
    for s in range(n_seq):
        want_n, want = oracle.spec_verify(target[s], q[s], draft[s], u[s], T)
        assert nacc[s] == want_n and out[s, :want_n + 1].tolist() == want[:want_n + 1].tolist()


def test_sums_argument_errors(hs):
    from geistlib_amd.binding import GeistHipError
    with pytest.raises(GeistHipError):
        hs._check(hs.lib.geist_hip_sampler_set_sums(hs.h, 7))


def test_rows_of_infinities_and_nan_with_fast_sums(hs, oracle):
    """-inf regions (a chunk of nothing but -inf weighs nothing), +inf and NaN logits: the ids of
    the exact mode."""
    rows, n = 6, 70000
    g = np.random.default_rng(5)
    x = (g.standard_normal((rows, n)) * 2).astype(np.float32)
    x[0, 8192:24576] = -np.inf        # two whole chunks
    x[1, :60000] = -np.inf
    x[2, 100] = np.inf
    x[3, 200] = np.nan
    x[4, :] = -np.inf
    u = g.random(rows).astype(np.float32)
    prm = P(temperature=0.9)
    hs.set_sums(fast=False)
    exact = run_rows(hs, torch, np.repeat(x, 16, axis=0), np.repeat(u, 16), prm)
    hs.set_sums(fast=True)
    fast = run_rows(hs, torch, np.repeat(x, 16, axis=0), np.repeat(u, 16), prm)
    hs.set_sums(fast=False)
    assert fast.tolist() == exact.tolist()


@pytest.mark.parametrize("extra", ["softcap", "mask", "ragged"])
def test_fast_sums_on_rows_that_are_not_plain(hs, oracle, extra):
    """Soft-capped rows, rows under an allowed-token mask and rows that allow no float4 loads
    take the pass's general form: the same ids as the exact mode (and the oracle's)."""
    rows, n = 16, 70001 if extra == "ragged" else 70000
    g = np.random.default_rng(len(extra))
    x = (g.standard_normal((rows, n)) * 3).astype(np.float32)
    u = g.random(rows).astype(np.float32)
    cap = 6.0 if extra == "softcap" else 0.0
    allowed = (g.random((rows, n)) < 0.4) if extra == "mask" else None
    if allowed is not None:
        allowed[:, 0] = True
    prm = P(temperature=0.9, softcap=cap)
    want = []
    for r in range(rows):
        row = oracle.softcap(x[r], cap) if cap else x[r]
        if allowed is not None:
            row = np.where(allowed[r], row, -np.inf).astype(np.float32)
        want.append(oracle.chain_u(row, float(u[r]), temperature=0.9))
    hs.set_sums(fast=True)
    fast = run_rows(hs, torch, x, u, prm, allowed=allowed)
    hs.set_sums(fast=False)
    exact = run_rows(hs, torch, x, u, prm, allowed=allowed)
    assert compare_ids(exact, [t for t, _ in want], [i for _, i in want], "exact") == 0
    assert compare_ids(fast, [t for t, _ in want], [i for _, i in want], "fast") <= 1
