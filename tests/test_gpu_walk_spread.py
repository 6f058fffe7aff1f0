"""The whole-row walk of the top-p / min-p modes spread over the workgroups of the row's chunks
(geist_hip_sampler_set_whole_row_walk): the same tokens as the oracle's sorted walk
(sampler.c:246-304) in every mode of sending it -- always, never, and following the rows that
turn up --, with penalties, soft-cap and mask, on rows of equal values, and when the waits
between its steps run out and a row's first workgroup has to walk it alone."""
import numpy as np
import pytest

from gpu_util import compare_ids, run_rows

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")

ADAPTIVE, SPREAD, ONE = 0, 1, 2


@pytest.fixture(scope="module")
def P():
    from geistlib_amd import SampleParams
    return SampleParams.make


def flat_rows(g, rows, n):
    x = (g.standard_normal((rows, n)) * 0.4).astype(np.float32)
    x[1] = np.round(x[1] * 4) / 4             # many equal probabilities: index order decides
    x[2, g.integers(0, n, 50)] = -90.0        # a few tiny probabilities
    if rows > 3:
        x[3] = 1.0                            # all equal
    return x


def want_of(oracle, x, u, **kw):
    res = [oracle.chain_u(x[r], float(u[r]), **kw) for r in range(x.shape[0])]
    return [t for t, _ in res], [i for _, i in res]


@pytest.mark.parametrize("n", [128256, 50001, 20000, 8192, 151936])
def test_spread_walk_gives_the_oracles_tokens(oracle, P, n):
    from geistlib_amd import HipSampler
    print(f"spread walk n={n}", flush=True)
    g = np.random.default_rng(n)
    rows = 6
    hs = HipSampler(max_rows=8, max_vocab=n)
    try:
        hs.set_whole_row_walk(SPREAD)
        for kw in (dict(temperature=1.0, top_p=0.9), dict(temperature=0.8, top_p=0.95, min_p=1e-4),
                   dict(temperature=1.3, min_p=1e-5), dict(temperature=1.0, top_p=0.5)):
            x = flat_rows(g, rows, n)
            u = g.random(rows).astype(np.float32)
            u[4] = 0.0
            u[5] = np.float32(1.0 - 2.0 ** -24)
            got = run_rows(hs, torch, x, u, P(**kw))
            paths = hs.row_paths(rows).tolist()
            want, infos = want_of(oracle, x, u, **kw)
            near = compare_ids(got, want, infos, f"spread walk n={n} {kw}")
            assert near <= 1
            # (short rows and narrow nuclei are within the list's reach: path 2)
            assert set(paths) <= {2, 4}, (paths, kw)
            if n >= 50001 and kw.get("top_p", 1.0) >= 0.9:
                assert paths == [4] * rows, (paths, kw)
    finally:
        hs.close()


def test_spread_walk_with_penalties_cap_and_mask(oracle, P):
    from geistlib_amd import HipSampler
    n, rows = 70001, 5
    g = np.random.default_rng(7)
    x = flat_rows(g, rows, n)
    u = g.random(rows).astype(np.float32)
    hist = g.integers(0, n, (rows, 300)).astype(np.int32)
    hlen = np.array([300, 0, 17, 300, 128], dtype=np.int32)
    allowed = g.random((rows, n)) < 0.8
    allowed[3] = True
    rep, freq, pres, cap = 1.3, 0.05, 0.1, 4.0
    hs = HipSampler(max_rows=8, max_vocab=n)
    try:
        hs.set_whole_row_walk(SPREAD)
        for lead, pad in ((0, 0), (1, 2)):
            for kw in (dict(temperature=1.0, top_p=0.9), dict(temperature=0.8, top_p=0.95, min_p=1e-4)):
                got = run_rows(hs, torch, x, u, P(rep=rep, freq=freq, pres=pres, softcap=cap, **kw),
                               history=hist, history_len=hlen, lead=lead, pad=pad, allowed=allowed)
                paths = hs.row_paths(rows).tolist()
                want, infos = [], []
                for r in range(rows):
                    row = oracle.penalties(x[r], hist[r, :hlen[r]], rep, freq, pres)
                    row = oracle.softcap(row, cap)
                    row[~allowed[r]] = -np.inf
                    t, i = oracle.chain_u(row, float(u[r]), **kw)
                    want.append(t)
                    infos.append(i)
                near = compare_ids(got, want, infos, f"spread walk, transforms, {kw} lead {lead}")
                assert near <= 1
                assert paths == [4] * rows, paths
    finally:
        hs.close()


def test_modes_agree_and_the_adaptive_one_follows_the_rows(oracle, P):
    """One workgroup, spread, adaptive: the same ids. In the adaptive mode the first call with
    such rows is served by one workgroup per row (path 3) and says so; the following calls are
    spread (path 4), until 64 calls in a row have had no such row."""
    from geistlib_amd import HipSampler
    n, rows = 100000, 8
    g = np.random.default_rng(3)
    kw = dict(temperature=1.0, top_p=0.9, precedence=0)
    hs = HipSampler(max_rows=8, max_vocab=n)
    try:
        flat = [flat_rows(g, rows, n) for _ in range(3)]
        peaked = (g.standard_normal((rows, n)) * 6).astype(np.float32)
        u = g.random(rows).astype(np.float32)
        ids = {}
        for mode in (ONE, SPREAD):
            hs.set_whole_row_walk(mode)
            ids[mode] = [run_rows(hs, torch, x, u, P(**kw)).tolist() for x in flat]
            assert hs.row_paths(rows).tolist() == [3 if mode == ONE else 4] * rows
        assert ids[ONE] == ids[SPREAD]
        for x, got in zip(flat, ids[SPREAD]):
            res = [oracle.top_p_u(x[r], 0.9, 1.0, float(u[r])) for r in range(rows)]
            assert compare_ids(np.array(got), [t for t, _ in res], [i for _, i in res], "modes") <= 1
        hs.set_whole_row_walk(ADAPTIVE)
        seen = []
        for x in [peaked] * 65 + [flat[0], flat[1], flat[2], peaked, flat[0]] + [peaked] * 65 + [flat[1], flat[2]]:
            got = run_rows(hs, torch, x, u, P(**kw)).tolist()
            seen.append(sorted(set(hs.row_paths(rows).tolist())))
            if x is not peaked:
                k = [i for i, f in enumerate(flat) if f is x][0]
                assert got == ids[ONE][k]
        # a call counts for the 64 that follow it
        assert seen == [[1]] * 65 + [[3], [4], [4], [1], [4]] + [[1]] * 65 + [[3], [4]], seen
    finally:
        hs.close()


def test_waits_that_run_out(oracle, P):
    """With a wait limit of zero no workgroup waits for a step's result: the workgroups that did
    not arrive last leave, the row's first one walks the row alone, and the following call (with
    the default limit again) finds its workspace cleared."""
    from geistlib_amd import HipSampler
    n, rows = 60000, 8
    g = np.random.default_rng(11)
    kw = dict(temperature=1.0, top_p=0.9)
    hs = HipSampler(max_rows=8, max_vocab=n)
    try:
        hs.set_whole_row_walk(SPREAD)
        x = flat_rows(g, rows, n)
        u = g.random(rows).astype(np.float32)
        want, infos = want_of(oracle, x, u, **kw)
        hs.set_wait_limit(0)
        for _ in range(2):
            got = run_rows(hs, torch, x, u, P(**kw))
            assert compare_ids(got, want, infos, "no waiting") <= 1
            assert set(hs.row_paths(rows).tolist()) <= {3, 4}
        hs.set_wait_limit(65536)
        for _ in range(2):
            got = run_rows(hs, torch, x, u, P(**kw))
            assert compare_ids(got, want, infos, "after the waits that ran out") <= 1
            assert hs.row_paths(rows).tolist() == [4] * rows
    finally:
        hs.close()
