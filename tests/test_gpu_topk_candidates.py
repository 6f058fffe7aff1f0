"""The candidate path of top-k (the scan's wavefronts hand their leading groups on, the row-final
kernel gathers nothing) against the oracle, on the rows it was built for and on the rows it has to
pass on to the thread-maxima path and the whole-row selection. Token ids bit for bit; which path
served each row is read back and asserted, so that every branch is known to have run."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

from gpu_util import compare_ids, run_rows  # noqa: E402


@pytest.fixture(scope="module")
def hs():
    from geistlib_amd import HipSampler
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need a device; the sampling path has no CPU fallback")
    s = HipSampler(max_rows=256, max_vocab=262144)
    yield s
    s.close()


def P(**kw):
    from geistlib_amd import SampleParams
    return SampleParams.make(**kw)


def units(g, rows):
    return (g.integers(0, 1 << 24, rows).astype(np.float32) / np.float32(1 << 24)).astype(np.float32)


def want_rows(oracle, x, u, hist=None, pen=None, hist_len=None, **kw):
    res = []
    for r in range(x.shape[0]):
        h = None if hist is None else (hist[r] if hist_len is None else hist[r][:hist_len[r]])
        row = x[r] if hist is None else oracle.penalties(x[r], h, *pen)
        res.append(oracle.chain_u(row, float(u[r]), **kw))
    return [t for t, _ in res], [i for _, i in res]


@pytest.mark.parametrize("n,k", [(128256, 40), (151936, 40), (262144, 64), (32000, 2), (70000, 64),
                                 (8192 * 3, 17)])
def test_plain_rows_take_the_candidate_path(hs, oracle, n, k):
    print(f"candidates n={n} k={k}", flush=True)
    g = np.random.default_rng(n + k)
    rows = 24
    x = (g.standard_normal((rows, n)) * 2).astype(np.float32)
    x[1, g.integers(0, n, 5)] += 10        # a few leaders far above the rest
    x[2] = (g.standard_t(3, n) * 2.5).astype(np.float32)
    u = units(g, rows)
    got = run_rows(hs, torch, x, u, P(temperature=0.7, top_k=k, top_p=0.9))
    paths = hs.topk_paths(rows).tolist()
    want, infos = want_rows(oracle, x, u, temperature=0.7, top_k=k, top_p=0.9)
    compare_ids(got, want, infos, f"candidates n={n} k={k}")
    assert paths == [0] * rows, paths


def test_rows_the_candidates_cannot_certify(hs, oracle):
    """Leading logits crowded into one wavefront's elements (a sorted row, a cluster of
    consecutive ids), runs of equal values across the cut, rows with fewer than k finite logits:
    each falls back inside the same launch and still gives the oracle's token."""
    g = np.random.default_rng(5)
    n, k, rows = 128256, 40, 16
    x = (g.standard_normal((rows, n)) * 2).astype(np.float32)
    x[0] = -np.sort(-x[0])                          # sorted: the top 40 sit in 10 threads
    x[1, 70000:70040] = x[1].max() + 1 + g.random(40).astype(np.float32)   # a cluster
    x[2, :] = np.round(x[2])                        # long runs of equal values
    x[3, :] = 1.5                                   # all equal
    x[4, :] = -np.inf
    x[4, g.integers(0, n, 25)] = g.standard_normal(25).astype(np.float32)  # < k finite
    x[5, ::2] = -np.inf                             # half the row forbidden by value
    x[6, :1000] = 9.0                               # 1000 equal leaders in the first chunk
    x[7, n - 3:] = 50.0                             # leaders in the ragged last chunk
    u = units(g, rows)
    got = run_rows(hs, torch, x, u, P(temperature=0.8, top_k=k, top_p=0.95))
    paths = hs.topk_paths(rows).tolist()
    want, infos = want_rows(oracle, x, u, temperature=0.8, top_k=k, top_p=0.95)
    compare_ids(got, want, infos, "rows passed on")
    print("paths:", paths)
    # (the cluster of row 1 and the short runs of equal values of row 2 are within what some forms
    # of the path hand on and beyond others)
    assert paths[0] != 0 and paths[3] != 0 and paths[4] != 0
    assert paths[5] == 0 and paths[7] == 0 and all(p == 0 for p in paths[8:])


@pytest.mark.parametrize("H,dup", [(2048, True), (2048, False), (300, True), (1, False), (0, False)])
def test_penalties_from_the_history_table(hs, oracle, H, dup):
    """Penalties on the candidate path: the history goes into a table in LDS. Heavily repeated
    ids, ids outside the vocabulary, rows with shorter histories, leaders penalised away."""
    g = np.random.default_rng(100 + H + dup)
    n, k, rows = 128256, 40, 32
    Hl = max(H, 4)
    x = (g.standard_normal((rows, n)) * 2).astype(np.float32)
    hist = (g.zipf(1.1, (rows, Hl)) % n if dup else g.integers(0, n, (rows, Hl))).astype(np.int32)
    lead = np.argsort(-x, axis=1)[:, :60]
    m = min(Hl, 30)
    hist[::2, :m] = lead[::2, :m]                   # every other row: its leaders are in the history
    hist[3, : min(Hl, 3)] = [-1, n, n + 5][: min(Hl, 3)]   # ids outside the vocabulary: ignored
    hl = np.full(rows, H, dtype=np.int32)
    hl[5] = H // 2
    hl[6] = 0
    u = units(g, rows)
    for pen in [(1.1, 0.5, 0.3), (1.0, 0.0, 4.0), (3.0, 0.0, 0.0)]:
        got = run_rows(hs, torch, x, u, P(temperature=0.7, top_k=k, top_p=0.9, rep=pen[0],
                                          freq=pen[1], pres=pen[2]), hist, hl)
        paths = hs.topk_paths(rows).tolist()
        hh = [hist[r, :hl[r]] for r in range(rows)]
        want, infos = want_rows(oracle, x, u, hist=hh, pen=pen, temperature=0.7, top_k=k, top_p=0.9)
        compare_ids(got, want, infos, f"history table H={H} dup={dup} pen={pen}")
        assert set(paths) <= {0, 1, 2} and paths.count(0) >= rows // 2, paths


def test_penalties_that_empty_the_candidates(hs, oracle):
    """The 500 leading logits of a row are all penalised far down: fewer than k of the candidates
    still reach the bound, which then certifies nothing, and the row is passed on."""
    g = np.random.default_rng(77)
    n, k, rows, H = 128256, 40, 8, 512
    x = (g.standard_normal((rows, n)) * 2).astype(np.float32)
    hist = g.integers(0, n, (rows, H)).astype(np.int32)
    hist[:4, :500] = np.argsort(-x[:4], axis=1)[:, :500]
    hl = np.full(rows, H, dtype=np.int32)
    u = units(g, rows)
    got = run_rows(hs, torch, x, u, P(temperature=0.7, top_k=k, top_p=0.9, rep=1.0, freq=0.0, pres=8.0),
                   hist, hl)
    paths = hs.topk_paths(rows).tolist()
    want, infos = want_rows(oracle, x, u, hist=hist, pen=(1.0, 0.0, 8.0), temperature=0.7, top_k=k,
                            top_p=0.9)
    compare_ids(got, want, infos, "emptied candidates")
    assert all(p != 0 for p in paths[:4]) and paths[4:] == [0] * 4, paths


def test_calls_that_stay_off_the_candidate_path(hs, oracle):
    """k above 64 and penalties that can raise a logit: the thread-maxima path serves the whole
    call, and says so."""
    g = np.random.default_rng(9)
    n, rows = 60000, 8
    x = (g.standard_normal((rows, n)) * 2).astype(np.float32)
    u = units(g, rows)
    hist = g.integers(0, n, (rows, 2500)).astype(np.int32)
    hl = np.full(rows, 2500, dtype=np.int32)
    cases = [(dict(temperature=0.7, top_k=100), None, None),
             (dict(temperature=0.7, top_k=40, rep=0.8), hist[:, :100].copy(), (0.8, 0.0, 0.0))]
    for kw, h, pen in cases:
        hlen = None if h is None else np.full(rows, h.shape[1], dtype=np.int32)
        got = run_rows(hs, torch, x, u, P(**kw), h, hlen)
        assert hs.topk_paths(rows).tolist() == [-1] * rows
        okw = {k_: v for k_, v in kw.items() if k_ in ("temperature", "top_k", "top_p", "min_p")}
        want, infos = want_rows(oracle, x, u, hist=h, pen=pen, **okw)
        compare_ids(got, want, infos, f"off the candidate path {kw}")


@pytest.mark.parametrize("H", [2500, 9000, 40000])
def test_histories_of_any_length_on_the_candidate_path(hs, oracle, H):
    """The final stage keeps its candidates in a table and looks the history up in it, so the
    history's length does not matter: thousands of ids, many of them repeated and many of them
    among the leading logits, still on the candidate path."""
    g = np.random.default_rng(H)
    n, rows, k = 128256, 16, 40
    x = (g.standard_normal((rows, n)) * 2).astype(np.float32)
    hist = g.integers(0, n, (rows, H)).astype(np.int32)
    for r in range(rows):                       # the row's leaders, over and over
        top = np.argsort(-x[r])[:60]
        hist[r, : H // 2] = g.choice(top, H // 2)
    hist[0, :] = int(np.argmax(x[0]))           # one id H times
    hl = np.full(rows, H, dtype=np.int32)
    hl[1] = H - 777
    u = units(g, rows)
    pen = (1.3, 0.02, 0.1)
    got = run_rows(hs, torch, x, u, P(temperature=0.7, top_k=k, top_p=0.9, rep=pen[0], freq=pen[1],
                                      pres=pen[2]), hist, hl)
    paths = hs.topk_paths(rows).tolist()
    want, infos = want_rows(oracle, x, u, hist=[hist[r, :hl[r]] for r in range(rows)], pen=pen,
                            temperature=0.7, top_k=k, top_p=0.9)
    compare_ids(got, want, infos, f"history of {H}")
    assert all(p_ >= 0 for p_ in paths), paths   # the candidate path served the call


def test_soft_capped_rows_select_on_raw_logits_and_cap_what_they_keep(hs, oracle):
    """The soft-cap (head.c:148-159) keeps the order of the logits, so the scan hands on raw
    values and the row-final kernel caps its candidates. Ordinary rows stay on the candidate
    path; rows whose leaders the cap presses into one value (logits far beyond the cap) cannot
    be certified from candidates -- ties are broken by index over the whole row -- and are passed
    on. Penalties come before the cap, as in the exact scan."""
    g = np.random.default_rng(314)
    n, k, rows, cap = 128256, 40, 12, 30.0
    x = (g.standard_normal((rows, n)) * 4).astype(np.float32)
    x[1] *= 2                                        # bent by the cap, still distinct
    x[2] = (g.standard_normal(n) * 400).astype(np.float32)     # thousands saturate at +-cap
    x[3, g.integers(0, n, 60)] = 1e4                 # 60 equal leaders: all of them candidates
    x[4, :7] = [np.inf, 500.0, 499.0, 200.0, 30.0, 29.999, -np.inf]
    u = units(g, rows)
    kw = dict(temperature=0.8, top_k=k, top_p=0.95)
    got = run_rows(hs, torch, x, u, P(softcap=cap, **kw))
    paths = hs.topk_paths(rows).tolist()
    res = [oracle.chain_u(oracle.softcap(x[r], cap), float(u[r]), **kw) for r in range(rows)]
    compare_ids(got, [t for t, _ in res], [i for _, i in res], "soft-capped candidates")
    print("paths:", paths)
    assert paths[0] == 0 and paths[1] == 0 and all(p == 0 for p in paths[5:]), paths
    assert paths[2] != 0, paths
    # with penalties in front of the cap
    H = 300
    hist = g.integers(0, n, (rows, H)).astype(np.int32)
    top = np.argsort(-x, axis=1)[:, :10].astype(np.int32)
    hist[:, :10] = top
    hl = np.full(rows, H, dtype=np.int32)
    pen = (1.2, 0.3, 0.1)
    got = run_rows(hs, torch, x, u, P(softcap=cap, rep=pen[0], freq=pen[1], pres=pen[2], **kw),
                   hist, hl)
    res = [oracle.chain_u(oracle.softcap(oracle.penalties(x[r], hist[r], *pen), cap), float(u[r]),
                          **kw) for r in range(rows)]
    compare_ids(got, [t for t, _ in res], [i for _, i in res], "soft-capped, penalised")


def test_soft_capped_rows_on_the_thread_maxima_path(oracle):
    """The same split of work where the candidate path does not apply (k above its limit, a mask,
    an unaligned row): thread maxima of the raw logits, the cap on what the row-final kernel
    gathers, strict comparison with the capped bound."""
    from geistlib_amd import HipSampler
    s = HipSampler(max_rows=16, max_vocab=70000)
    g = np.random.default_rng(99)
    n, rows, cap = 65537, 8, 20.0
    x = (g.standard_normal((rows, n)) * 6).astype(np.float32)
    x[1] = (g.standard_normal(n) * 300).astype(np.float32)     # saturated leaders: passed on
    x[2, g.integers(0, n, 200)] = 77.0
    u = units(g, rows)
    for k in (100, 40):
        kw = dict(temperature=0.9, top_k=k, top_p=0.9)
        got = run_rows(s, torch, x, u, P(softcap=cap, **kw))
        res = [oracle.chain_u(oracle.softcap(x[r], cap), float(u[r]), **kw) for r in range(rows)]
        compare_ids(got, [t for t, _ in res], [i for _, i in res], f"soft-capped maxima k={k}")
    s.close()


@pytest.mark.parametrize("pen", [False, True])
def test_one_launch_and_two_launches_agree(hs, oracle, pen):
    """The candidate path as one launch (the last workgroup of a row to finish scanning goes on
    as the row's final stage) and as two give the oracle's ids, call after call on changing
    rows -- what one workgroup wrote must be what another reads -- including rows that fall back
    to the thread maxima and to the whole-row selection."""
    n, k, rows = 128256, 40, 64
    g = np.random.default_rng(77 + pen)
    used = hs.one_launch_topk(True)
    print("one launch available on this device:", used, flush=True)
    hist = None
    pk = {}
    pen_t = None
    if pen:
        hist = g.integers(0, n, (rows, 1024)).astype(np.int32)
        pk = dict(rep=1.1, freq=0.5, pres=0.2)
        pen_t = (1.1, 0.5, 0.2)
    try:
        for call in range(4):
            x = (g.standard_normal((rows, n)) * 2).astype(np.float32)
            x[call] = -np.sort(-x[call])                # thread-maxima path
            x[8 + call, :] = np.round(x[8 + call])      # runs of equal values
            x[16 + call, :] = 0.5                       # all equal: whole-row selection
            u = units(g, rows)
            # every row its own history length: the slower paths read the length of THEIR row
            hl = None if hist is None else g.integers(0, hist.shape[1] + 1, rows).astype(np.int32)
            want, infos = want_rows(oracle, x, u, hist=hist, pen=pen_t, temperature=0.7, top_k=k,
                                    top_p=0.9, hist_len=hl)
            # one launch with the hand-over read from the shared second-level cache (where the
            # placement allows), one launch with every row treated as spread over XCDs, two launches
            for one, far in ((True, False), (True, True), (False, False)):
                hs.one_launch_topk(one)
                hs.handoff_scope(far)
                got = run_rows(hs, torch, x, u, P(temperature=0.7, top_k=k, top_p=0.9, **pk),
                               history=hist, history_len=hl)
                compare_ids(got, want, infos, f"call {call} one launch {one} far {far}")
                paths = hs.topk_paths(rows).tolist()
                assert paths[call] != 0 and paths[16 + call] != 0, paths
                if far:   # no row trusts what the others handed on: all served from the logits
                    assert all(p != 0 for p in paths), paths
                else:
                    assert sum(p == 0 for p in paths) >= rows - 8, paths
    finally:
        hs.one_launch_topk(True)
        hs.handoff_scope(False)
