"""The one-pass form of the modes that need a row's maximum before its exponentials (temperature,
top-p / min-p, softmax, speculative verification): the workgroups of a row wait for one another
inside the kernel, and one that stops waiting reads the row for itself. Both ways must give the
oracle's ids; the second is forced from the host with a wait limit of 0 polls, so every workgroup
still ends normally."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")

from gpu_util import compare_ids, run_rows, to_dev  # noqa: E402


@pytest.fixture()
def hs():
    from geistlib_amd import HipSampler
    s = HipSampler(max_rows=256, max_vocab=160000)
    yield s
    s.close()


def P(**kw):
    from geistlib_amd import SampleParams
    return SampleParams.make(**kw)


def history_for(g, rows, n, length=300):
    hist = g.integers(0, n, (rows, length)).astype(np.int32)
    hist[:, :40] = hist[:, 40:80]          # repeated ids: counts above 1
    hl = np.full(rows, length, dtype=np.int32)
    hl[1] = 0
    return hist, hl


CASES = [
    # (rows, n, sampling parameters, penalties)
    (3, 5000, dict(temperature=0.8), False),
    (8, 50000, dict(temperature=1.0), True),
    (16, 128256, dict(temperature=0.7), False),
    (8, 60000, dict(temperature=1.0, top_p=0.9), False),
    (8, 60000, dict(temperature=1.0, top_p=0.95, min_p=0.05), True),
    (5, 151936, dict(temperature=1.0, top_p=0.95, min_p=0.05), True),
    (1, 128256, dict(temperature=0.8), False),
]


@pytest.mark.parametrize("wait_limit", [None, 0, 3])
@pytest.mark.parametrize("rows,n,kw,pen", CASES)
def test_waiting_and_not_waiting_give_the_oracles_ids(hs, oracle, rows, n, kw, pen, wait_limit):
    print(f"one pass rows={rows} n={n} {kw} pen={pen} wait_limit={wait_limit}", flush=True)
    g = np.random.default_rng(rows * 7 + n)
    x = (g.standard_normal((rows, n)) * 2.5).astype(np.float32)
    x[0, n // 3] = x[0].max()              # the maximum twice: the first index counts
    u = g.random(rows).astype(np.float32)
    hist = hl = None
    pk = {}
    if pen:
        hist, hl = history_for(g, rows, n)
        pk = dict(rep=1.2, freq=0.4, pres=0.2)
    if wait_limit is not None:
        hs.set_wait_limit(wait_limit)
    for call in range(2):                  # the second call finds the meeting words as the first left them
        got = run_rows(hs, torch, x, u, P(**kw, **pk), history=hist, history_len=hl)
        res = []
        for r in range(rows):
            row = oracle.penalties(x[r], hist[r, :hl[r]], 1.2, 0.4, 0.2) if pen else x[r]
            res.append(oracle.chain_u(row, float(u[r]), **kw))
        near = compare_ids(got, [t for t, _ in res], [i for _, i in res], f"call {call}")
        assert near <= 1


@pytest.mark.parametrize("far", [False, True])
@pytest.mark.parametrize("rows,n,kw,pen", [CASES[1], CASES[2], CASES[4], CASES[6], (4, 128256, dict(temperature=0.9), True)])
def test_meeting_in_the_shared_l2_or_through_memory(hs, oracle, rows, n, kw, pen, far):
    """Where a launch deals the workgroups of a row to one XCD they write their meeting slots
    with plain stores, which that XCD's L2 serves to the polls; geist_hip_sampler_handoff_scope
    (1) makes them store through to memory as launches of other shapes do. The ids are the
    oracle's both ways, on two calls in a row (the slot arrays take turns)."""
    print(f"meeting rows={rows} n={n} {kw} pen={pen} far={far}", flush=True)
    g = np.random.default_rng(rows * 11 + n)
    x = (g.standard_normal((rows, n)) * 2.5).astype(np.float32)
    hist = hl = None
    pk = {}
    if pen:
        hist, hl = history_for(g, max(rows, 2), n)
        hist, hl = hist[:rows], hl[:rows]
        pk = dict(rep=1.2, freq=0.4, pres=0.2)
    hs.handoff_scope(far)
    try:
        for call in range(2):
            u = g.random(rows).astype(np.float32)
            got = run_rows(hs, torch, x, u, P(**kw, **pk), history=hist, history_len=hl)
            res = []
            for r in range(rows):
                row = oracle.penalties(x[r], hist[r, :hl[r]], 1.2, 0.4, 0.2) if pen else x[r]
                res.append(oracle.chain_u(row, float(u[r]), **kw))
            near = compare_ids(got, [t for t, _ in res], [i for _, i in res], f"call {call}")
            assert near <= 1
    finally:
        hs.handoff_scope(False)


@pytest.mark.parametrize("wait_limit", [None, 0])
def test_normalised_probabilities_one_pass(hs, oracle, wait_limit):
    rows, n, T = 4, 70001, 0.9
    g = np.random.default_rng(9)
    x = (g.standard_normal((rows, n)) * 3).astype(np.float32)
    if wait_limit is not None:
        hs.set_wait_limit(wait_limit)
    d = to_dev(x, torch)
    probs = torch.empty((rows, n), dtype=torch.float32, device="cuda")
    from geistlib_amd import HipSampler
    hs.softmax(HipSampler.rows(d), P(temperature=T), probs)
    hs.sync()
    got = probs.cpu().numpy()
    for r in range(rows):
        want, _ = oracle.softmax_normalised(x[r], T)
        assert np.array_equal(got[r], want), r


@pytest.mark.parametrize("wait_limit", [None, 0])
def test_spec_verify_one_pass(hs, oracle, wait_limit):
    from test_gpu_sampling import _run_spec, _spec_case
    n_seq, L, n, T = 5, 6, 40000, 0.9
    if wait_limit is not None:
        hs.set_wait_limit(wait_limit)
    target, q, draft, u = _spec_case(77, n_seq, L, n)
    for call in range(2):
        nacc, out = _run_spec(hs, target, q, draft, u, T)
        for s in range(n_seq):
            want_n, want = oracle.spec_verify(target[s], q[s], draft[s], u[s], T)
            assert nacc[s] == want_n, (call, s)
            assert out[s, :want_n + 1].tolist() == want[:want_n + 1].tolist(), (call, s)


@pytest.mark.parametrize("n_seq,L,n,T", [(28, 8, 128256, 1.0), (7, 5, 50001, 0.8), (3, 63, 9000, 1.2),
                                         (1, 4, 128256, 1.0), (40, 2, 20000, 1.0)])
def test_spec_verify_one_launch_and_two_launches_agree(hs, oracle, n_seq, L, n, T):
    """The residual sums and the draw in one launch (the workgroups of a sequence meet for their
    sums and one of them walks its chunk from registers), in two launches, and in one launch
    with every wait given up at once (each workgroup then forms the other chunks' sums itself):
    the same accepted counts and tokens, equal to the oracle's. One sequence accepts every draft
    (the bonus token), one is rejected where the residual is empty (the token is drawn from p)."""
    from test_gpu_sampling import _run_spec, _spec_case
    print(f"spec one launch n_seq={n_seq} L={L} n={n}", flush=True)
    target, q, draft, u = _spec_case(n_seq * 31 + L, n_seq, L, n)
    if n_seq >= 3:
        # sequence 1: q == p on every row, so every draft is accepted whatever the draws
        q[1] = np.stack([oracle.softmax_normalised(target[1, j], T)[0] for j in range(L)])
        # sequence 2: at row 0 every q is one step above p and the draw is the largest there
        # is, so the draft is rejected there and the residual max(0, p - q) is empty
        q[2, 0] = np.nextafter(oracle.softmax_normalised(target[2, 0], T)[0], np.float32(2.0))
        u[2, 0] = np.float32(1 - 2.0 ** -24)
    results = []
    try:
        for one_launch, wait_limit in ((True, None), (False, None), (True, 0)):
            hs.one_launch_spec(one_launch)
            if wait_limit is not None:
                hs.set_wait_limit(wait_limit)
            results.append(_run_spec(hs, target, q, draft, u, T))
    finally:
        hs.one_launch_spec(True)
        hs.set_wait_limit(65536)
    for nacc, out in results[1:]:
        assert np.array_equal(nacc, results[0][0]) and np.array_equal(out, results[0][1])
    nacc, out = results[0]
    seen = set()
    for s in range(n_seq):
        want_n, want = oracle.spec_verify(target[s], q[s], draft[s], u[s], T)
        assert nacc[s] == want_n, (s, nacc[s], want_n)
        assert out[s, :want_n + 1].tolist() == want[:want_n + 1].tolist(), (s, out[s], want)
        seen.add(int(want_n))
    print("  accepted lengths seen:", sorted(seen))
    if n_seq >= 3:
        assert nacc[1] == L and nacc[2] == 0


@pytest.mark.parametrize("pen", [False, True])
def test_min_p_lists_of_every_size(hs, oracle, pen):
    """The exp-sum pass stages a chunk's min-p candidates in LDS (2048 places per chunk): rows whose
    candidates are a handful per chunk, rows with about a thousand in one chunk, and rows with more
    than a chunk can stage (which the pass must report as not listed, so that the whole row is
    walked) all give the oracle's ids."""
    rows, n = 6, 40000
    g = np.random.default_rng(31 + pen)
    x = (g.standard_normal((rows, n)) * 2.0).astype(np.float32)
    x[1, 9000:10000] = x[1].max() - 0.01 * g.random(1000).astype(np.float32)   # ~1000 in one chunk
    x[2, 17000:20000] = x[2].max() + 0.5                                       # 3000 equal leaders
    x[3, :] = np.float32(0.25)                                                 # every element
    x[4, 8190:8194] = x[4].max() + 1.0                                         # across a chunk edge
    u = g.random(rows).astype(np.float32)
    kw = dict(temperature=1.0, top_p=0.95, min_p=0.05)
    hist = hl = None
    pk = {}
    if pen:
        hist, hl = history_for(g, rows, n)
        pk = dict(rep=1.2, freq=0.4, pres=0.2)
    for call in range(2):
        got = run_rows(hs, torch, x, u, P(**kw, **pk), history=hist, history_len=hl)
        res = []
        for r in range(rows):
            row = oracle.penalties(x[r], hist[r, :hl[r]], 1.2, 0.4, 0.2) if pen else x[r]
            res.append(oracle.chain_u(row, float(u[r]), **kw))
        near = compare_ids(got, [t for t, _ in res], [i for _, i in res], f"call {call}")
        assert near <= 1
        paths = hs.row_paths(rows)
        assert paths[0] == 2 and paths[1] == 2, paths     # listed
        assert paths[2] in (3, 4) and paths[3] in (3, 4), paths   # more than a chunk stages: whole row


@pytest.mark.parametrize("wait_limit", [None, 0, 3])
@pytest.mark.parametrize("rows,n,pen,extra", [
    (1, 128256, False, ""),
    (1, 2049, False, ""),            # two chunks, the second with one element
    (2, 50001, True, ""),            # ragged rows (not a multiple of four), penalties
    (4, 32000, False, "softcap"),
    (3, 32003, True, "mask"),
    (2, 10000, False, "nan"),
    (1, 7, False, ""),               # one workgroup: nobody to meet
])
def test_temperature_draw_in_one_kernel(hs, oracle, rows, n, pen, extra, wait_limit):
    """A few rows draw by temperature in a single kernel whose workgroups meet twice (for the
    row's maximum, then for the chunks' sums) and whose draw is walked from the registers of
    the workgroup it falls to. Ids equal the oracle's, also when every wait is given up at once
    (wait limit 0: every workgroup forms maximum and sums from the row itself) or early (3)."""
    from gpu_util import pack_allowed  # noqa: F401  (run_rows packs the mask)
    print(f"one kernel rows={rows} n={n} pen={pen} {extra} wait_limit={wait_limit}", flush=True)
    g = np.random.default_rng(rows * 131 + n)
    x = (g.standard_normal((rows, n)) * 2.5).astype(np.float32)
    x[0, n // 2] = x[0].max()
    if extra == "nan":
        x[1, 17] = np.nan
        x[0, 5] = -np.inf
    cap = 5.0 if extra == "softcap" else 0.0
    allowed = (g.random((rows, n)) < 0.3) if extra == "mask" else None
    if allowed is not None:
        allowed[:, 0] = True
    hist = hl = None
    pk = {}
    if pen:
        hist, hl = history_for(g, max(rows, 2), n)
        hist, hl = hist[:rows], hl[:rows]
        pk = dict(rep=1.2, freq=0.4, pres=0.2)
    if wait_limit is not None:
        hs.set_wait_limit(wait_limit)
    T = 0.8
    for call in range(3):                  # meeting words alternate between two arrays
        u = g.random(rows).astype(np.float32)
        if call == 1:
            u[0] = np.float32(0.99999994)  # the last float below one: the end of the row
        got = run_rows(hs, torch, x, u, P(temperature=T, softcap=cap, **pk), history=hist,
                       history_len=hl, allowed=allowed)
        res = []
        for r in range(rows):
            row = oracle.penalties(x[r], hist[r, :hl[r]], 1.2, 0.4, 0.2) if pen else x[r]
            if cap:
                row = oracle.softcap(row, cap)
            if allowed is not None:
                row = np.where(allowed[r], row, -np.inf).astype(np.float32)
            res.append(oracle.chain_u(row, float(u[r]), temperature=T))
        near = compare_ids(got, [t for t, _ in res], [i for _, i in res], f"call {call}")
        assert near <= 1
