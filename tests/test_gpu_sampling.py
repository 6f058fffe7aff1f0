"""GPU parity tests proper: the HIP path, called through the C ABI, against the CPU oracle on
identical logits and identical uniforms. Token ids are bit-exact (lowest index wins ties) except
draws within 1e-6 of a CDF boundary, which are counted and printed."""
import ctypes as C
import json
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

from gpu_util import compare_ids, fuzz_seeds, run_rows, to_dev  # noqa: E402


@pytest.fixture(scope="module")
def hs():
    from geistlib_amd import HipSampler
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need a device; the sampling path has no CPU fallback")
    s = HipSampler(max_rows=512, max_vocab=262144)
    yield s
    s.close()


def P(**kw):
    from geistlib_amd import SampleParams
    return SampleParams.make(**kw)


def rows_rng(seed, rows, n, scale=2.0, ties=False):
    g = np.random.default_rng(seed)
    x = (g.standard_normal((rows, n)) * scale).astype(np.float32)
    if ties:
        x = (np.round(x * 4) / 4).astype(np.float32)
    u = (g.integers(0, 1 << 24, rows).astype(np.float32) / np.float32(1 << 24)).astype(np.float32)
    return x, u


# ----------------------------------------------------------------------------------- argmax
@pytest.mark.parametrize("n", [1, 5, 63, 64, 65, 256, 1000, 2048, 2049, 8191, 8192, 8193, 50000,
                               128256, 262144])
def test_argmax_matches_oracle(hs, oracle, n):
    print(f"argmax n={n}", flush=True)
    x, _ = rows_rng(n, 7, n)
    x[3, :] = np.round(x[3, :])            # many exact ties
    x[4, :] = 1.5                          # all equal -> index 0
    x[5, n // 2:] = x[5].max() + 1         # tie of the maximum: first of the upper half
    got = run_rows(hs, torch, x, None, P(temperature=0.0))
    want = [oracle.argmax(x[r]) for r in range(x.shape[0])]
    assert got.tolist() == want


def test_argmax_reference_vectors(hs):
    # tests/test_sampler_unit.c:33-37 of the reference -> 3
    x = np.array([[-1, 2, .5, 3, 3, -.5]], dtype=np.float32)
    assert run_rows(hs, torch, x, None, P(temperature=0.0)).tolist() == [3]
    # tests/test_fused_probe_agreement_unit.c:147-157 -> 77, through the backend-slot entry point
    p = np.array([100.0 if i == 77 else i % 7 for i in range(256)], dtype=np.float32)
    assert hs.argmax_f32(to_dev(p, torch)) == 77


def test_argmax_special_values(hs, oracle):
    n = 5000
    x, _ = rows_rng(1, 6, n)
    x[0, 10] = np.nan                      # NaN elsewhere never wins
    x[1, 0] = np.nan                       # NaN at index 0 is never displaced
    x[2, :] = -np.inf
    x[2, 4000] = -1e30
    x[3, :] = -np.inf                      # all -inf -> 0
    x[4, 77] = np.inf
    x[4, 99] = np.inf
    x[5, :] = 0.0
    x[5, 7] = -0.0                         # -0 == +0: index 0 stays
    got = run_rows(hs, torch, x, None, P(temperature=0.0))
    want = [oracle.argmax(x[r]) for r in range(6)]
    assert got.tolist() == want
    assert want[1] == 0 and want[3] == 0 and want[4] == 77 and want[5] == 0


# ------------------------------------------------------------------------------ temperature
@pytest.mark.parametrize("n,T", [(5, 1.0), (64, 0.8), (1000, 0.1), (8192, 0.8), (8193, 1.7),
                                 (50000, 0.8), (128256, 0.8), (151936, 1.0)])
def test_temperature_matches_oracle(hs, oracle, n, T):
    print(f"temperature n={n} T={T}", flush=True)
    x, u = rows_rng(n + 1, 24, n, scale=3.0)
    x[1] = 0.25                            # uniform row: id == floor(u * n)
    got = run_rows(hs, torch, x, u, P(temperature=T))
    res = [oracle.temperature_u(x[r], T, float(u[r])) for r in range(x.shape[0])]
    near = compare_ids(got, [t for t, _ in res], [i for _, i in res], f"temperature n={n}")
    assert got[1] == int(np.floor(float(u[1]) * n))
    print(f"  rows within 1e-6 of a CDF boundary: {near}")
    assert near <= 1


# ------------------------------------------------------------------------------------ top-k
@pytest.mark.parametrize("n,k,T", [(8, 2, 1.0), (300, 3, 1.0), (1000, 40, 0.7), (5000, 64, 0.6),
                                   (8192, 128, 1.0), (8193, 5, 0.9), (50000, 40, 0.7),
                                   (128256, 40, 0.7), (262144, 64, 0.6)])
def test_top_k_matches_oracle(hs, oracle, n, k, T):
    print(f"top-k n={n} k={k}", flush=True)
    x, u = rows_rng(n + k, 16, n)
    x[2] = np.round(x[2] * 2) / 2          # ties straddling the cutoff
    got = run_rows(hs, torch, x, u, P(temperature=T, top_k=k, precedence=0))
    res = [oracle.top_k_u(x[r], k, T, float(u[r])) for r in range(x.shape[0])]
    near = compare_ids(got, [t for t, _ in res], [i for _, i in res], f"top-k n={n} k={k}")
    print(f"  rows within 1e-6 of a CDF boundary: {near}")
    assert near <= 1


@pytest.mark.parametrize("n,k,T", [(3000, 200, 10.0), (20000, 129, 1.0), (20000, 1000, 0.9),
                                   (20000, 8192, 1.2), (20000, 9000, 1.2), (128256, 4096, 1.0)])
def test_top_k_large_k_general_path(hs, oracle, n, k, T):
    """k above the candidate path (the reference caps k at 8192, sampler.c:213-215)."""
    print(f"top-k general n={n} k={k}", flush=True)
    x, u = rows_rng(n + k, 6, n)
    x[2] = np.round(x[2] * 2) / 2
    got = run_rows(hs, torch, x, u, P(temperature=T, top_k=k, precedence=0))
    res = [oracle.top_k_u(x[r], k, T, float(u[r])) for r in range(x.shape[0])]
    near = compare_ids(got, [t for t, _ in res], [i for _, i in res], f"top-k n={n} k={k}")
    assert near <= 1


def test_top_k_degenerate_rows(hs, oracle):
    """Rows that overflow the per-chunk candidate lists: all-equal logits, a masked row where only
    a few logits are finite, two-valued rows. Equal logits keep ascending index order."""
    n, k = 30000, 40
    x, u = rows_rng(12, 8, n)
    x[0] = 0.5
    x[1] = -np.inf
    x[1, [17, 2900, 29999]] = [1.0, 2.0, 0.5]
    x[2] = np.where(np.arange(n) % 2 == 0, 1.0, -1.0)
    x[3] = np.round(x[3])
    x[4, :] = 3.0
    x[4, 100:200] = 3.5
    u[5] = 0.0
    u[6] = np.float32(1.0 - 2.0 ** -24)
    for T, kk, p in [(1.0, k, 1.0), (0.7, k, 0.9), (1.0, 128, 1.0)]:
        got = run_rows(hs, torch, x, u, P(temperature=T, top_k=kk, top_p=p))
        res = [oracle.chain_u(x[r], float(u[r]), temperature=T, top_k=kk, top_p=p)
               for r in range(x.shape[0])]
        compare_ids(got, [t for t, _ in res], [i for _, i in res], "degenerate rows")


def test_top_k_reference_unit_vector(hs, oracle):
    # tests/test_sampler_unit.c:92-112: top-2 of 8 logits only ever yields ids {2, 4}
    from geistlib_amd.workloads import xorshift_units
    row = np.array([0, 1, 4, 2, 5, 1.5, 0, .5], dtype=np.float32)
    u, _ = xorshift_units(11, 256)
    x = np.tile(row, (256, 1))
    got = run_rows(hs, torch, x, u, P(temperature=1.0, top_k=2, precedence=0))
    want = [oracle.top_k_u(row, 2, 1.0, float(v))[0] for v in u]
    assert got.tolist() == want and set(got.tolist()) == {2, 4}


@pytest.mark.parametrize("n,k,p,m", [(1000, 40, 0.9, 0.0), (128256, 40, 0.9, 0.0),
                                     (128256, 40, 0.9, 0.05), (50000, 64, 0.5, 0.0),
                                     (50000, 100, 1.0, 0.1), (262144, 64, 0.9, 0.0)])
def test_chain_top_k_top_p_min_p(hs, oracle, n, k, p, m):
    print(f"chain n={n} k={k} p={p} m={m}", flush=True)
    x, u = rows_rng(n * 3 + k, 16, n)
    got = run_rows(hs, torch, x, u, P(temperature=0.7, top_k=k, top_p=p, min_p=m))
    res = [oracle.chain_u(x[r], float(u[r]), temperature=0.7, top_k=k, top_p=p, min_p=m)
           for r in range(x.shape[0])]
    near = compare_ids(got, [t for t, _ in res], [i for _, i in res], "chain")
    print(f"  rows within 1e-6 of a CDF boundary: {near}")
    assert near <= 1


def test_reference_precedence_ignores_top_p_when_top_k_set(hs, oracle):
    x, u = rows_rng(99, 8, 20000)
    got = run_rows(hs, torch, x, u, P(temperature=0.7, top_k=40, top_p=0.5, precedence=0))
    want = [oracle.top_k_u(x[r], 40, 0.7, float(u[r]))[0] for r in range(8)]
    assert got.tolist() == want


# ------------------------------------------------------------ top-p / min-p, whole vocabulary
def test_top_p_reference_unit_vector(hs, oracle):
    # tests/test_sampler_unit.c:115-131: top_p = 0.5 on {10, 0, 0, 0, 0} -> index 0 nearly always
    from geistlib_amd.workloads import xorshift_units
    row = np.array([10, 0, 0, 0, 0], dtype=np.float32)
    u, _ = xorshift_units(13, 128)
    got = run_rows(hs, torch, np.tile(row, (128, 1)), u, P(temperature=1.0, top_p=0.5, precedence=0))
    want = [oracle.top_p_u(row, 0.5, 1.0, float(v))[0] for v in u]
    assert got.tolist() == want and got.tolist().count(0) > 120


@pytest.mark.parametrize("n,scale,T,p", [(5, 3.0, 1.0, 0.5), (300, 6.0, 0.7, 0.9),
                                         (5000, 6.0, 0.7, 0.9), (128256, 5.0, 0.7, 0.9),
                                         (128256, 6.0, 0.7, 0.95), (262144, 6.0, 0.6, 0.9)])
def test_top_p_peaked_rows(hs, oracle, n, scale, T, p):
    """Small nuclei: served from the thread maxima."""
    print(f"top-p peaked n={n} p={p}", flush=True)
    x, u = rows_rng(n + 7, 12, n, scale=scale)
    got = run_rows(hs, torch, x, u, P(temperature=T, top_p=p, precedence=0))
    res = [oracle.top_p_u(x[r], p, T, float(u[r])) for r in range(x.shape[0])]
    near = compare_ids(got, [t for t, _ in res], [i for _, i in res], f"top-p n={n}")
    assert near <= 1


@pytest.mark.parametrize("n,scale,T,p", [(64, 1.0, 1.0, 0.9), (5000, 1.0, 1.0, 0.9),
                                         (40000, 2.0, 1.0, 0.95), (128256, 2.0, 0.7, 0.9),
                                         (151936, 2.0, 1.0, 0.3), (9000, 0.0, 1.0, 0.37)])
def test_top_p_wide_nucleus_general_path(hs, oracle, n, scale, T, p):
    """Nuclei of thousands of entries (flat rows, the all-equal row): the radix descent."""
    print(f"top-p wide n={n} p={p}", flush=True)
    x, u = rows_rng(n + 11, 6, n, scale=scale)
    x[1] = np.round(x[1] * 8) / 8          # many equal probabilities: index order among them
    got = run_rows(hs, torch, x, u, P(temperature=T, top_p=p, precedence=0))
    res = [oracle.top_p_u(x[r], p, T, float(u[r])) for r in range(x.shape[0])]
    near = compare_ids(got, [t for t, _ in res], [i for _, i in res], f"top-p wide n={n}")
    assert near <= 1


@pytest.mark.parametrize("n,scale,T,p,m", [(2000, 2.0, 1.0, 1.0, 0.05), (128256, 2.0, 1.0, 0.95, 0.05),
                                           (151936, 2.0, 1.0, 0.95, 0.05), (50000, 1.0, 1.0, 1.0, 0.5),
                                           (50000, 2.0, 0.8, 0.5, 0.001), (50000, 1.0, 1.0, 0.9, 1e-6)])
def test_min_p_and_top_p_chain(hs, oracle, n, scale, T, p, m):
    print(f"min-p n={n} p={p} m={m}", flush=True)
    x, u = rows_rng(n + 13, 8, n, scale=scale)
    got = run_rows(hs, torch, x, u, P(temperature=T, top_p=p, min_p=m))
    res = [oracle.chain_u(x[r], float(u[r]), temperature=T, top_p=p, min_p=m)
           for r in range(x.shape[0])]
    near = compare_ids(got, [t for t, _ in res], [i for _, i in res], f"min-p n={n}")
    assert near <= 1


@pytest.mark.parametrize("n,scale,T,p,m", [(128256, 3.0, 1.0, 0.9, 0.0), (151936, 2.0, 1.0, 0.95, 0.05),
                                           (50000, 2.5, 1.0, 0.8, 0.0), (262144, 3.6, 1.0, 0.9, 0.0),
                                           (128256, 2.0, 1.0, 1.0, 0.02), (20000, 2.0, 1.0, 0.6, 0.0)])
def test_top_p_candidate_list_path(hs, oracle, n, scale, T, p, m):
    """Kept prefixes of hundreds to thousands of entries: too many for the thread-maxima shortcut,
    few enough to be listed by a third pass and walked from the list. Row 1 is quantised, so
    many list entries share one probability and the draw has to respect index order among them."""
    print(f"top-p list n={n} p={p} m={m}", flush=True)
    x, u = rows_rng(n + 17, 10, n, scale=scale)
    x[1] = np.round(x[1] * 4) / 4
    got = run_rows(hs, torch, x, u, P(temperature=T, top_p=p, min_p=m))
    paths = hs.row_paths(x.shape[0])
    res = [oracle.chain_u(x[r], float(u[r]), temperature=T, top_p=p, min_p=m)
           for r in range(x.shape[0])]
    near = compare_ids(got, [t for t, _ in res], [i for _, i in res], f"top-p list n={n}")
    assert near <= 1
    assert set(paths.tolist()) <= {1, 2, 3, 4}     # (3 / 4: the whole row, by one workgroup / by its chunks')
    assert (paths == 2).sum() >= 6, f"paths {paths.tolist()}, kept {[i.n_keep for _, i in res]}"


def test_top_p_vocabulary_beyond_the_shortcut(oracle):
    """More than 32 chunks of 8192: the thread-maxima shortcut is not attempted at all."""
    from geistlib_amd import HipSampler
    n = 300000
    big = HipSampler(max_rows=4, max_vocab=n)
    try:
        x, u = rows_rng(321, 4, n, scale=4.0)
        x[3] *= 0.1
        got = run_rows(big, torch, x, u, P(temperature=1.0, top_p=0.9, precedence=0))
        paths = big.row_paths(4).tolist()
    finally:
        big.close()
    res = [oracle.top_p_u(x[r], 0.9, 1.0, float(u[r])) for r in range(4)]
    near = compare_ids(got, [t for t, _ in res], [i for _, i in res], "top-p n=300000")
    assert near <= 1
    assert paths[:3] == [2, 2, 2] and paths[3] in (3, 4), paths


def test_sorted_paths_all_three_in_one_batch(hs, oracle):
    """One batch whose rows need the shortcut, the list and the whole-row walk."""
    n = 100000
    g = np.random.default_rng(99)
    x = np.empty((6, n), dtype=np.float32)
    x[0] = g.standard_normal(n) * 6            # peaked: shortcut
    x[1] = g.standard_normal(n) * 6
    x[2] = g.standard_normal(n) * 3            # hundreds kept: list
    x[3] = g.standard_normal(n) * 3
    x[4] = g.standard_normal(n) * 0.5          # tens of thousands kept: whole row
    x[5] = 1.0                                 # all equal
    u = g.random(6).astype(np.float32)
    got = run_rows(hs, torch, x, u, P(temperature=1.0, top_p=0.9, precedence=0))
    paths = hs.row_paths(6).tolist()
    res = [oracle.top_p_u(x[r], 0.9, 1.0, float(u[r])) for r in range(6)]
    near = compare_ids(got, [t for t, _ in res], [i for _, i in res], "three paths")
    assert near <= 1
    assert paths[:2] == [1, 1] and paths[2:4] == [2, 2] and set(paths[4:]) <= {3, 4}, paths


@pytest.mark.parametrize("n,lead,pad", [(128256, 0, 0), (50001, 0, 0), (33333, 3, 5),
                                        (70001, 1, 2)])
def test_whole_row_walk_with_penalties_cap_and_mask(hs, oracle, n, lead, pad):
    """Rows close to uniform, so that every one of them is walked in full, with everything the
    walk's own pass over the logits has to apply: penalties from a history, the soft-cap, the
    allowed-token mask; vocabularies that are no multiple of four and rows that start off a
    16-byte boundary; nucleus and min-p. Row 1 is quantised (index order among equal
    probabilities), row 2 has a few values far below the rest (tiny probabilities)."""
    print(f"whole-row walk n={n} lead={lead} pad={pad}", flush=True)
    g = np.random.default_rng(n + lead)
    rows = 5
    x = (g.standard_normal((rows, n)) * 0.4).astype(np.float32)
    x[1] = np.round(x[1] * 4) / 4
    x[2, g.integers(0, n, 50)] = -90.0
    u = g.random(rows).astype(np.float32)
    hist = g.integers(0, n, (rows, 300)).astype(np.int32)
    hlen = np.array([300, 0, 17, 300, 128], dtype=np.int32)
    allowed = g.random((rows, n)) < 0.8
    allowed[3] = True
    rep, freq, pres, cap = 1.3, 0.05, 0.1, 4.0
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
        near = compare_ids(got, want, infos, f"whole-row walk n={n} {kw}")
        assert near <= 1
        assert set(paths) <= {3, 4}, paths


def test_ids_and_draws_in_page_locked_host_memory(hs):
    """geist_hip_host_malloc: the kernels write the ids into host memory and read the draws from
    it, in place; the ids equal those of the same call with device buffers, for every mode that
    has a kernel of its own to finish a row."""
    from geistlib_amd import HipSampler
    x, u = rows_rng(77, 24, 50000, scale=3.0)
    out_h, u_h = hs.host_buffer(24 * 4), hs.host_buffer(24 * 4)
    try:
        u_h.view(np.float32)[:] = u
        d = to_dev(x, torch)
        for prm in (P(temperature=0.0), P(temperature=0.9), P(temperature=0.7, top_k=40),
                    P(temperature=0.7, top_k=40, top_p=0.9), P(temperature=1.0, top_p=0.9),
                    P(temperature=1.0, min_p=0.05), P(temperature=1.0, top_p=0.9, precedence=0)):
            want = run_rows(hs, torch, x, u, prm)
            ids = out_h.view(np.int32)
            ids[:] = -7
            hs.sample(HipSampler.rows(d), prm, u_h, out_h)
            hs.sync()
            assert ids.tolist() == want.tolist(), prm
    finally:
        out_h.close()
        u_h.close()


def test_logits_hint_changes_nothing_but_the_loads(hs, oracle):
    """GEIST_HIP_LOGITS_STREAMED: non-temporal loads in the single-pass modes, identical ids."""
    from geistlib_amd.binding import GeistHipError
    x, u = rows_rng(91, 16, 128256, scale=2.0)
    want = {}
    for streamed in (False, True, False):
        hs.set_logits_hint(streamed)
        for name, prm in (("argmax", P(temperature=0.0)), ("top_k", P(temperature=0.7, top_k=40)),
                          ("chain", P(temperature=0.7, top_k=40, top_p=0.9))):
            got = run_rows(hs, torch, x, u, prm).tolist()
            assert want.setdefault(name, got) == got, (name, streamed)
    assert want["argmax"] == [oracle.argmax(x[r]) for r in range(16)]
    with pytest.raises(GeistHipError):
        hs.set_logits_hint(7)


def test_min_p_listed_by_the_exp_sum_pass(hs, oracle):
    """min_p of a few percent: the exp-sum pass lists the candidates and the list walk follows
    it directly. Peaked rows (a handful of candidates), ordinary rows (hundreds), and flat rows
    whose list overflows and is served by the whole-row walk; with and without top-p."""
    n = 60000
    g = np.random.default_rng(321)
    scale = np.array([8.0, 8.0, 3.0, 3.0, 2.0, 0.3, 0.3, 0.05])[:, None]
    x = (g.standard_normal((8, n)) * scale).astype(np.float32)
    u = g.random(8).astype(np.float32)
    for top_p in (1.0, 0.9):
        kw = dict(temperature=1.0, top_p=top_p, min_p=0.03)
        got = run_rows(hs, torch, x, u, P(**kw))
        paths = hs.row_paths(8).tolist()
        res = [oracle.chain_u(x[r], float(u[r]), **kw) for r in range(8)]
        near = compare_ids(got, [t for t, _ in res], [i for _, i in res], f"min-p listed {top_p}")
        assert near <= 1
        assert paths[:5] == [2] * 5 and set(paths[5:]) <= {3, 4}, paths


def test_sorted_modes_many_rows_and_one_row(hs, oracle):
    """More rows than compute units share the list walk (one workgroup per row, 100 KB of LDS
    each), and the single-row call of decode_step."""
    n = 20000
    g = np.random.default_rng(123)
    x = (g.standard_normal((400, n)) * g.choice([0.7, 2.5, 6.0], (400, 1))).astype(np.float32)
    u = g.random(400).astype(np.float32)
    got = run_rows(hs, torch, x, u, P(temperature=1.0, top_p=0.9, min_p=0.001))
    paths = hs.row_paths(400)
    res = [oracle.chain_u(x[r], float(u[r]), temperature=1.0, top_p=0.9, min_p=0.001)
           for r in range(400)]
    near = compare_ids(got, [t for t, _ in res], [i for _, i in res], "400 rows")
    assert near <= 2 and 2 in paths and set(paths.tolist()) <= {1, 2, 3, 4}
    for r in (0, 1, 2):
        one = run_rows(hs, torch, x[r:r + 1], u[r:r + 1], P(temperature=1.0, top_p=0.9, min_p=0.001))
        assert one[0] == got[r]


def test_top_p_limits_match_reference_dispatch(hs, oracle):
    x, u = rows_rng(5, 6, 3000)
    for p in (0.0, -1.0, 1.0, 1.5):        # sampler.c:238-243: <= 0 -> argmax... but the session
        got = run_rows(hs, torch, x, u, P(temperature=0.8, top_p=p, precedence=0))
        # ...maps top_p <= 0 to 1.0 (step.c:391) and the dispatch (head.c:177) sends p >= 1 to the
        # temperature sampler; the C ABI takes the session's view
        want = [oracle.temperature_u(x[r], 0.8, float(u[r]))[0] for r in range(6)]
        assert got.tolist() == want


# ------------------------------------------------------------------------------ penalties
@pytest.mark.parametrize("rep,freq,pres", [(1.1, 0.5, 0.3), (1.3, 0.3, 0.7), (0.9, 0.07, 0.011)])
def test_penalties_in_place_match_oracle(hs, oracle, rep, freq, pres):
    """Bit-exact: every step of the penalty rounds on its own (freq * count is not exact for
    most freq, so a fused multiply-subtract would show here)."""
    g = np.random.default_rng(5)
    rows, n, H = 6, 30000, 700
    x = (g.standard_normal((rows, n)) * 2).astype(np.float32)
    hist = g.integers(0, n, (rows, H)).astype(np.int32)
    hist[:, :50] = hist[:, 50:100]         # duplicates
    hist[0, :10] = [-1, n, n + 5, -7, 0, 0, 0, n - 1, n - 1, 2**31 - 1]
    hl = np.array([H, H, 0, 1, 333, H], dtype=np.int32)
    d = to_dev(x, torch)
    hs.apply_penalties(d, to_dev(hist, torch), to_dev(hl, torch), rep, freq, pres)
    hs.sync()
    got = d.cpu().numpy()
    for r in range(rows):
        want = oracle.penalties(x[r], hist[r, :hl[r]], rep, freq, pres)
        assert np.array_equal(got[r], want), f"row {r}"


def test_penalties_fused_into_sampling(hs, oracle):
    g = np.random.default_rng(6)
    rows, n, H = 16, 40000, 512
    x = (g.standard_normal((rows, n)) * 2).astype(np.float32)
    hist = g.integers(0, 2000, (rows, H)).astype(np.int32)   # concentrated -> many repeats
    top = np.argsort(-x, axis=1)[:, :20].astype(np.int32)
    hist[:, :20] = top                     # the leaders are penalised, so the outcome changes
    hl = np.full(rows, H, dtype=np.int32)
    u = (g.integers(0, 1 << 24, rows) / np.float32(1 << 24)).astype(np.float32)
    before = x.copy()
    for params, kw in [(P(temperature=0.7, top_k=40, top_p=0.9, rep=1.3, freq=0.5, pres=0.3),
                        dict(temperature=0.7, top_k=40, top_p=0.9)),
                       (P(temperature=0.0, rep=1.3, freq=0.5, pres=0.3), dict(temperature=0.0)),
                       (P(temperature=0.9, rep=1.3, freq=0.5, pres=0.3), dict(temperature=0.9))]:
        got = run_rows(hs, torch, x, u, params, hist, hl)
        res = []
        for r in range(rows):
            pen = oracle.penalties(x[r], hist[r], 1.3, 0.5, 0.3)
            res.append(oracle.chain_u(pen, float(u[r]), **kw))
        compare_ids(got, [t for t, _ in res], [i for _, i in res], "fused penalties")
    assert np.array_equal(x, before)


def test_penalties_that_push_the_leaders_out(hs, oracle):
    """Most of the leading logits are penalised far down, so the thread maxima taken before the
    penalties promise too much: the row must still come out exact (it re-selects over the whole
    row), also when a penalty RAISES logits (rep < 1, negative frequency / presence)."""
    g = np.random.default_rng(16)
    rows, n, H = 8, 60000, 400
    x = (g.standard_normal((rows, n)) * 2).astype(np.float32)
    lead = np.argsort(-x, axis=1)[:, :H].astype(np.int32)
    hist = lead.copy()
    hist[4:, 200:] = g.integers(0, n, (4, 200))
    hl = np.full(rows, H, dtype=np.int32)
    u = (g.integers(0, 1 << 24, rows) / np.float32(1 << 24)).astype(np.float32)
    for rep, freq, pres in [(1.0, 0.0, 6.0), (2.5, 1.0, 0.0), (0.7, -0.4, -0.3), (1.0, -2.0, 0.0)]:
        got = run_rows(hs, torch, x, u, P(temperature=0.8, top_k=40, top_p=0.95, rep=rep, freq=freq,
                                          pres=pres), hist, hl)
        res = []
        for r in range(rows):
            pen = oracle.penalties(x[r], hist[r], rep, freq, pres)
            res.append(oracle.chain_u(pen, float(u[r]), temperature=0.8, top_k=40, top_p=0.95))
        compare_ids(got, [t for t, _ in res], [i for _, i in res], f"penalties {rep} {freq} {pres}")


# ------------------------------------------------------------------------------ softmax
@pytest.mark.parametrize("n,T", [(1000, 1.0), (128256, 0.7)])
def test_normalised_probabilities(hs, oracle, n, T):
    from geistlib_amd import HipSampler
    x, _ = rows_rng(n, 4, n)
    d = to_dev(x, torch)
    probs = torch.empty_like(d)
    hs.softmax(HipSampler.rows(d), P(temperature=T), probs)
    hs.sync()
    got = probs.cpu().numpy()
    for r in range(4):
        want, _ = oracle.softmax_normalised(x[r], T)
        # north-star bound: 1e-5 relative in fp32 (observed: identical up to 1 ulp)
        assert np.allclose(got[r], want, rtol=1e-5, atol=0)
        assert np.max(np.abs(got[r] - want) / np.maximum(want, 1e-38)) < 2e-7


# ------------------------------------------------------------------------------ soft-cap
@pytest.mark.parametrize("mode", ["temperature", "top_k", "top_p", "min_p"])
def test_softcap_fused_matches_libm_tanhf(hs, oracle, mode):
    """head.c:148-159: tanhf(x / cap) * cap before sampling. The device evaluates glibc's tanhf
    (geistlib_amd/csrc/glibc_tanhf.h), so ids are compared as in every other mode and the
    probabilities of capped rows agree to the last bit wherever the exp-sum does."""
    from geistlib_amd import HipSampler
    cap, n = 30.0, 60000
    x, u = rows_rng(77, 12, n, scale=25.0)            # most logits are bent by the cap
    x[3, :100] = [np.float32(v) for v in np.linspace(-1e-20, 1e-20, 100)]   # tiny arguments
    x[4, :4] = [np.inf, -np.inf, 700.0, -700.0]
    kw = dict(temperature=0.9, top_k=50 if mode == "top_k" else 0,
              top_p=0.9 if mode == "top_p" else 1.0, min_p=0.02 if mode == "min_p" else 0.0)
    got = run_rows(hs, torch, x, u, P(softcap=cap, **kw))
    res = [oracle.chain_u(oracle.softcap(x[r], cap), float(u[r]), **kw) for r in range(x.shape[0])]
    near = compare_ids(got, [t for t, _ in res], [i for _, i in res], f"softcap {mode}")
    assert near <= 1
    if mode == "temperature":
        d = to_dev(x[:3], torch)
        probs = torch.empty_like(d)
        hs.softmax(HipSampler.rows(d), P(temperature=0.9, softcap=cap), probs)
        hs.sync()
        got_p = probs.cpu().numpy()
        for r in range(3):
            want, _ = oracle.softmax_normalised(oracle.softcap(x[r], cap), 0.9)
            assert np.max(np.abs(got_p[r] - want) / np.maximum(want, 1e-38)) < 2e-7
            assert np.mean(got_p[r].view(np.uint32) == want.view(np.uint32)) > 0.999


@pytest.mark.parametrize("n", [64, 4097, 20000])
@pytest.mark.parametrize("mode", ["temperature", "top_k", "top_p", "min_p"])
def test_softcap_small_cap_ragged_row(hs, oracle, mode, n):
    """A small cap on a row that ends inside a chunk: the -inf that pads the chunk must stay
    weightless after the cap (tanhf(-inf) * cap = -cap is a finite logit, and with cap = 5 a few
    thousand of them outweigh the row). Probabilities are compared too."""
    from geistlib_amd import HipSampler
    cap = 5.0
    g = np.random.default_rng(n)
    x = (g.standard_t(3, (8, n)) * 4.0).astype(np.float32)
    x[1, n // 2] = -np.inf                            # inside the row -inf does become -cap
    u = g.random(8).astype(np.float32)
    kw = dict(temperature=1.0, top_k=40 if mode == "top_k" else 0,
              top_p=0.9 if mode == "top_p" else 1.0, min_p=0.01 if mode == "min_p" else 0.0)
    got = run_rows(hs, torch, x, u, P(softcap=cap, **kw))
    res = [oracle.chain_u(oracle.softcap(x[r], cap), float(u[r]), **kw) for r in range(8)]
    near = compare_ids(got, [t for t, _ in res], [i for _, i in res], f"small cap {mode} n={n}")
    assert near <= 1
    if mode == "temperature":
        d = to_dev(x, torch)
        probs = torch.empty_like(d)
        hs.softmax(HipSampler.rows(d), P(temperature=1.0, softcap=cap), probs)
        hs.sync()
        got_p = probs.cpu().numpy()
        for r in range(8):
            want, _ = oracle.softmax_normalised(oracle.softcap(x[r], cap), 1.0)
            assert np.max(np.abs(got_p[r] - want) / np.maximum(want, 1e-38)) < 2e-7


# ------------------------------------------------------------------------------ scoring
@pytest.mark.parametrize("n,cap", [(1000, 0.0), (128256, 0.0), (128256, 30.0), (262144, 50.0)])
def test_logprob_rows_match_oracle(hs, oracle, n, cap):
    """geist_session_peek_logits + logprob_at (tools/eval_geist.c:63-73) without the copy to the
    host; tolerance 1e-9 absolute on doubles (order of the sum, last bits of exp and log)."""
    rows, K = 5, 7
    x, _ = rows_rng(n + 3, rows, n, scale=6.0)
    g = np.random.default_rng(n)
    tok = g.integers(0, n, (rows, K)).astype(np.int32)
    tok[:, 0] = np.argmax(x, axis=1)
    tok[0, 1], tok[0, 2] = -1, n                      # outside the vocabulary -> NaN
    out = torch.full((rows, K), 7.0, dtype=torch.float64, device="cuda")
    hs.logprob(to_dev(x, torch), to_dev(tok, torch), out, softcap=cap)
    hs.sync()
    got = out.cpu().numpy()
    for r in range(rows):
        row = oracle.softcap(x[r], cap) if cap > 0 else x[r]
        for j in range(K):
            if 0 <= tok[r, j] < n:
                assert abs(got[r, j] - oracle.logprob_at(row, tok[r, j])) < 1e-9, (r, j)
            else:
                assert np.isnan(got[r, j])


# ------------------------------------------------------------------- speculative verify
def _spec_case(seed, n_seq, L, n, sigma=0.5):
    g = np.random.default_rng(seed)
    target = (g.standard_normal((n_seq, L + 1, n)) * 2).astype(np.float32)
    noisy = target[:, :L, :].astype(np.float64) + g.standard_normal((n_seq, L, n)) * sigma
    noisy -= noisy.max(axis=-1, keepdims=True)
    e = np.exp(noisy)
    q = (e / e.sum(axis=-1, keepdims=True)).astype(np.float32)
    cdf = np.cumsum(q.astype(np.float64), axis=-1)
    pick = g.random((n_seq, L, 1)) * cdf[..., -1:]
    draft = np.minimum((cdf < pick).sum(axis=-1), n - 1).astype(np.int32)
    u = (g.integers(0, 1 << 24, (n_seq, L + 1)) / np.float32(1 << 24)).astype(np.float32)
    return target, q, draft, u


def _run_spec(hs, target, q, draft, u, T):
    n_seq, lp1, n = target.shape
    out = torch.full((n_seq, lp1), -9, dtype=torch.int32, device="cuda")
    nacc = torch.full((n_seq,), -9, dtype=torch.int32, device="cuda")
    hs.spec_verify(to_dev(target, torch), to_dev(q, torch), to_dev(draft, torch), to_dev(u, torch),
                   T, out, nacc)
    hs.sync()
    return nacc.cpu().numpy(), out.cpu().numpy()


@pytest.mark.parametrize("n_seq,L,n,T", [(6, 4, 5000, 1.0), (5, 8, 20000, 0.8), (4, 8, 128256, 1.0),
                                         (3, 1, 300, 1.3), (8, 3, 8193, 1.0)])
def test_spec_verify_matches_oracle(hs, oracle, n_seq, L, n, T):
    print(f"spec n_seq={n_seq} L={L} n={n}", flush=True)
    target, q, draft, u = _spec_case(n_seq * 100 + L, n_seq, L, n)
    nacc, out = _run_spec(hs, target, q, draft, u, T)
    seen = set()
    for s in range(n_seq):
        want_n, want = oracle.spec_verify(target[s], q[s], draft[s], u[s], T)
        assert nacc[s] == want_n, (s, nacc[s], want_n)
        assert out[s, :want_n + 1].tolist() == want[:want_n + 1].tolist(), (s, out[s], want)
        assert np.all(out[s, want_n + 1:] == -9)       # the rest stays untouched
        seen.add(want_n)
    print("  accepted lengths seen:", sorted(seen))


def test_spec_verify_point_mass_drafts_and_softcap(hs, oracle):
    """d_draft_q = NULL is q = one-hot at the draft token; the soft-cap is applied to the target
    rows before anything else."""
    n_seq, L, n, cap = 6, 5, 30000, 20.0
    g = np.random.default_rng(8)
    target = (g.standard_normal((n_seq, L + 1, n)) * 3).astype(np.float32)
    draft = g.integers(0, n, (n_seq, L)).astype(np.int32)
    for s in range(n_seq):
        for j in range(L):
            target[s, j, draft[s, j]] += np.float32(25.0 if (s + j) % 3 else 0.0)
    u = (g.integers(0, 1 << 24, (n_seq, L + 1)) / np.float32(1 << 24)).astype(np.float32)
    out = torch.full((n_seq, L + 1), -9, dtype=torch.int32, device="cuda")
    nacc = torch.full((n_seq,), -9, dtype=torch.int32, device="cuda")
    hs.spec_verify(to_dev(target, torch), None, to_dev(draft, torch), to_dev(u, torch), 0.8, out,
                   nacc, softcap=cap)
    hs.sync()
    out, nacc = out.cpu().numpy(), nacc.cpu().numpy()
    seen = set()
    for s in range(n_seq):
        capped = np.stack([oracle.softcap(target[s, j], cap) for j in range(L + 1)])
        q = np.zeros((L, n), dtype=np.float32)
        q[np.arange(L), draft[s]] = 1.0
        want_n, want = oracle.spec_verify(capped, q, draft[s], u[s], 0.8)
        assert nacc[s] == want_n and out[s, :want_n + 1].tolist() == want[:want_n + 1].tolist(), s
        seen.add(want_n)
    assert len(seen) >= 2


def test_spec_verify_special_cases(hs, oracle):
    n_seq, L, n = 4, 5, 7000
    target, q, draft, u = _spec_case(77, n_seq, L, n)
    # q == p: everything is accepted whatever the uniforms; the bonus is a temperature draw
    pn = np.stack([[oracle.softmax_normalised(target[s, j], 1.0)[0] for j in range(L)]
                   for s in range(n_seq)]).astype(np.float32)
    u_hi = np.full_like(u, np.float32(1 - 2.0 ** -24))
    u_hi[:, L] = u[:, L]
    nacc, out = _run_spec(hs, target, pn, draft, u_hi, 1.0)
    assert nacc.tolist() == [L] * n_seq
    for s in range(n_seq):
        assert out[s, :L].tolist() == draft[s].tolist()
        assert out[s, L] == oracle.temperature_u(target[s, L], 1.0, float(u[s, L]))[0]
    # a draft that put all its mass on a token the target gives nothing: reject at once,
    # and the residual is the target distribution itself
    q2 = np.zeros_like(q)
    t2 = target.copy()
    t2[:, 0, 11] = -300.0
    q2[:, :, 11] = 1.0
    d2 = np.full_like(draft, 11)
    nacc, out = _run_spec(hs, t2, q2, d2, u, 1.0)
    assert nacc.tolist() == [0] * n_seq
    for s in range(n_seq):
        want_n, want = oracle.spec_verify(t2[s], q2[s], d2[s], u[s], 1.0)
        assert want_n == 0 and out[s, 0] == want[0]
    # greedy: exact-match prefix (src/engine/session.c:599-606 of the reference)
    am = np.array([[oracle.argmax(target[s, j]) for j in range(L + 1)] for s in range(n_seq)],
                  dtype=np.int32)
    d3 = am[:, :L].copy()
    d3[1, 2] = (d3[1, 2] + 1) % n
    d3[2, 0] = (d3[2, 0] + 1) % n
    nacc, out = _run_spec(hs, target, q, d3, u, 0.0)
    assert nacc.tolist() == [L, 2, 0, L]
    for s in range(n_seq):
        k = nacc[s]
        assert out[s, :k].tolist() == d3[s, :k].tolist() and out[s, k] == am[s, k]


# ---------------------------------------------------------------------------------- rng
def test_device_rng_matches_reference_stream(hs, oracle):
    from geistlib_amd import HipSampler
    from geistlib_amd.workloads import xorshift_units
    rows, n = 12, 20000
    x, _ = rows_rng(17, rows, n)
    d = to_dev(x, torch)
    out = torch.empty(rows, dtype=torch.int32, device="cuda")
    # shared state: row r takes draw r + 1 (finalize_logits_batch order)
    st = torch.tensor([0xC0FFEE], dtype=torch.int64, device="cuda")
    hs.sample_rng(HipSampler.rows(d), P(temperature=0.8, top_k=40, precedence=0), st, True, out)
    hs.sync()
    u, state_after = xorshift_units(0xC0FFEE, rows)
    want = [oracle.top_k_u(x[r], 40, 0.8, float(u[r]))[0] for r in range(rows)]
    assert out.cpu().tolist() == want
    assert int(st.cpu().numpy().view(np.uint64)[0]) == state_after
    # greedy leaves the state alone
    hs.sample_rng(HipSampler.rows(d), P(temperature=0.0), st, True, out)
    hs.sync()
    assert int(st.cpu().numpy().view(np.uint64)[0]) == state_after
    # per-row states
    seeds = np.arange(1, rows + 1, dtype=np.uint64) * np.uint64(7919)
    st = torch.from_numpy(seeds.view(np.int64)).cuda()
    hs.sample_rng(HipSampler.rows(d), P(temperature=0.8), st, False, out)
    hs.sync()
    want = []
    for r in range(rows):
        ur, _ = xorshift_units(int(seeds[r]), 1)
        want.append(oracle.temperature_u(x[r], 0.8, float(ur[0]))[0])
    assert out.cpu().tolist() == want


# ------------------------------------------------------------------- strided / unaligned
def test_row_stride_and_unaligned_rows(hs, oracle):
    g = np.random.default_rng(3)
    rows, n, ld = 5, 10001, 10007          # odd stride: rows are not 16-byte aligned
    buf = (g.standard_normal((rows, ld)) * 2).astype(np.float32)
    d = to_dev(buf, torch)
    view = d[:, :n]
    u = (g.integers(0, 1 << 24, rows) / np.float32(1 << 24)).astype(np.float32)
    from geistlib_amd import HipSampler
    out = torch.empty(rows, dtype=torch.int32, device="cuda")
    r = HipSampler.rows(view)
    assert r.ld == ld and r.n_vocab == n
    hs.sample(r, P(temperature=0.7, top_k=10, precedence=0), to_dev(u, torch), out)
    hs.sync()
    want = [oracle.top_k_u(np.ascontiguousarray(buf[i, :n]), 10, 0.7, float(u[i]))[0]
            for i in range(rows)]
    assert out.cpu().tolist() == want


def test_argument_errors(hs):
    from geistlib_amd import HipSampler
    from geistlib_amd.binding import GeistHipError
    d = torch.zeros((2, 100), dtype=torch.float32, device="cuda")
    out = torch.empty(2, dtype=torch.int32, device="cuda")
    with pytest.raises(GeistHipError):     # stochastic without uniforms
        hs.sample(HipSampler.rows(d), P(temperature=0.7), None, out)
    with pytest.raises(GeistHipError):     # min_p under the reference precedence
        hs.sample(HipSampler.rows(d), P(temperature=0.7, min_p=0.1, precedence=0), out, out)
    big = HipSampler.rows(d)
    big.rows = 100000
    with pytest.raises(GeistHipError):     # beyond the workspace
        hs.sample(big, P(temperature=0.0), None, out)


# ------------------------------------------------------------------------- n-gram drafter
@pytest.mark.parametrize("seed", fuzz_seeds(4))
def test_ngram_drafter_matches_oracle(hs, oracle, seed):
    """geist_hip_propose_drafts_ngram against the restated propose_drafts_ngram
    (src/engine/session.c:437-513): drafts, their count and the matched length, exactly."""
    g = np.random.default_rng(700 + seed)
    for case in range(6):
        n_seq = int(g.integers(1, 33))
        H = int(g.choice([1, 2, 9, 300, 5000]))
        alphabet = int(g.choice([2, 4, 30, 1000]))
        k_max = int(g.integers(1, 17))
        ms = int(g.choice([0, 1, 2, 4, 8, 11]))
        pad = int(g.choice([0, 3]))
        hist = g.integers(0, alphabet, (n_seq, H + pad)).astype(np.int32)
        if alphabet == 1000 and H >= 300:          # text that repeats itself in long stretches
            for s in range(n_seq):
                period = int(g.integers(5, 60))
                hist[s] = np.resize(hist[s, :period], H + pad)
                hist[s, g.integers(0, H, 8)] = 7    # with a few edits
        hl = g.integers(0, H + 1, n_seq).astype(np.int32)
        hl[0] = H
        seeds = np.array([hist[s, g.integers(0, max(int(hl[s]), 1))] for s in range(n_seq)],
                         dtype=np.int32)
        seeds[-1] = -1                              # a seed that occurs nowhere
        print(f"drafter seed {seed} case {case}: n_seq={n_seq} H={H} alphabet={alphabet} "
              f"k_max={k_max} max_suffix={ms}", flush=True)
        out = torch.full((n_seq, k_max + 2), -9, dtype=torch.int32, device="cuda")
        cnt = torch.full((n_seq,), -9, dtype=torch.int32, device="cuda")
        mlen = torch.full((n_seq,), -9, dtype=torch.int32, device="cuda")
        hs.propose_drafts_ngram(to_dev(hist, torch), to_dev(hl, torch), to_dev(seeds, torch), k_max,
                                ms, out, cnt, mlen)
        hs.sync()
        out, cnt, mlen = out.cpu().numpy(), cnt.cpu().numpy(), mlen.cpu().numpy()
        lengths = set()
        for s in range(n_seq):
            want, wl = oracle.propose_drafts_ngram(hist[s, :hl[s]], int(seeds[s]), k_max, ms)
            assert cnt[s] == len(want) and mlen[s] == wl, (s, cnt[s], mlen[s], want, wl)
            assert out[s, :cnt[s]].tolist() == want, (s, out[s], want)
            assert np.all(out[s, cnt[s]:] == -9)    # nothing written beyond the drafts
            lengths.add(wl)
        print("  matched lengths seen:", sorted(lengths))


def test_ngram_drafter_argument_errors(hs):
    from geistlib_amd.binding import GeistHipError
    h = torch.zeros((2, 8), dtype=torch.int32, device="cuda")
    hl = torch.zeros(2, dtype=torch.int32, device="cuda")
    sd = torch.zeros(2, dtype=torch.int32, device="cuda")
    out = torch.zeros((2, 4), dtype=torch.int32, device="cuda")
    c = torch.zeros(2, dtype=torch.int32, device="cuda")
    for k_max in (0, 17, 5):                        # 5 > out_ld = 4
        with pytest.raises(GeistHipError):
            hs.propose_drafts_ngram(h, hl, sd, k_max, 4, out, c, c)


# --------------------------------------------------------------------- allowed-token mask
@pytest.mark.parametrize("mode", ["argmax", "temperature", "top_k", "top_p", "min_p", "chain"])
def test_allowed_mask_equals_minus_inf_after_the_transforms(hs, oracle, mode):
    """Constrained decoding on the device: a forbidden token weighs nothing. Equal to sampling
    from the row with -inf written over the forbidden logits AFTER penalties and soft-cap (the
    reference's runtime masks what geist_session_peek_logits hands out, which is capped)."""
    from gpu_util import pack_allowed
    rows, n, cap = 10, 50257, 8.0
    g = np.random.default_rng(41)
    x = (g.standard_normal((rows, n)) * 3).astype(np.float32)
    u = (g.integers(0, 1 << 24, rows) / np.float32(1 << 24)).astype(np.float32)
    hist = g.integers(0, n, (rows, 64)).astype(np.int32)
    hl = np.full(rows, 64, dtype=np.int32)
    allowed = g.random((rows, n)) < np.array([1e-4, 1e-3, 0.01, 0.1, 0.5, 0.9, 0.99, 1.0, 0.3,
                                              0.3])[:, None]
    allowed[np.arange(rows), g.integers(0, n, rows)] = True
    allowed[8, np.argmax(x[8])] = False               # the favourite is forbidden
    allowed[9, :] = False
    allowed[9, 12345] = True                          # a single choice
    x[7, 0] = np.nan
    allowed[6, 0] = False
    x[6, 0] = np.nan                                  # a forbidden NaN at index 0 does not win
    kw = dict(temperature=0.0 if mode == "argmax" else 0.9,
              top_k=40 if mode in ("top_k", "chain") else 0,
              top_p=0.9 if mode in ("top_p", "chain") else 1.0,
              min_p=0.02 if mode in ("min_p", "chain") else 0.0)
    if mode != "argmax":
        x[7, 0] = 0.5                                 # NaN rows are defined for argmax only
    got = run_rows(hs, torch, x, u, P(softcap=cap, rep=1.2, freq=0.1, pres=0.1, **kw), hist, hl,
                   allowed=allowed)
    res = []
    for r in range(rows):
        row = oracle.penalties(x[r], hist[r], 1.2, 0.1, 0.1)
        if mode != "argmax":
            row = oracle.softcap(row, cap)
        row = np.where(allowed[r], row, -np.inf).astype(np.float32)
        res.append((oracle.argmax(row), None) if mode == "argmax"
                   else oracle.chain_u(row, float(u[r]), **kw))
    near = compare_ids(got, [t for t, _ in res], [i for _, i in res], f"mask {mode}")
    assert near <= 1
    assert all(allowed[r, got[r]] for r in range(rows))
    assert got[9] == 12345
    # one mask shared by every row (allowed_ld = 0)
    shared = allowed[4:5]
    got = run_rows(hs, torch, x[:6], u[:6], P(**kw), allowed=shared)
    for r in range(6):
        row = np.where(shared[0], x[r], -np.inf).astype(np.float32)
        want = oracle.argmax(row) if mode == "argmax" else oracle.chain_u(row, float(u[r]), **kw)[0]
        assert got[r] == want, (mode, r)


@pytest.mark.parametrize("n", [300, 9000, 50257])
def test_rows_that_are_not_finite_follow_the_reference(hs, oracle, n):
    """Rows with a NaN, a +inf or nothing finite: the softmax sum is NaN. Temperature and top-p
    then answer with the last token as the reference does (its loops find no slot; top-p:
    sampler.c:243 is not taken, 287-303 fall through), the other modes as the oracle."""
    from geistlib_amd import SampleParams
    g = np.random.default_rng(n)
    mods = [lambda x: x.__setitem__(150, np.nan), lambda x: x.__setitem__(0, np.nan),
            lambda x: x.__setitem__(len(x) - 1, np.nan), lambda x: x.__setitem__(7, np.inf),
            lambda x: (x.__setitem__(7, np.inf), x.__setitem__(9, np.inf)),
            lambda x: x.fill(-np.inf), lambda x: x.fill(np.nan)]
    rows = []
    for mod in mods:
        r = g.standard_normal(n).astype(np.float32)
        mod(r)
        rows.append(r)
    x = np.stack(rows)
    u = g.random(len(rows)).astype(np.float32)
    for kw in (dict(temperature=1.3, top_k=0, top_p=0.3, min_p=0.0),
               dict(temperature=1.0, top_k=0, top_p=0.9, min_p=0.05),
               dict(temperature=1.0, top_k=0, top_p=1.0, min_p=0.05),
               dict(temperature=1.0, top_k=0, top_p=1.0, min_p=0.0),
               dict(temperature=1.0, top_k=40, top_p=1.0, min_p=0.0),
               dict(temperature=0.7, top_k=40, top_p=0.9, min_p=0.0)):
        want = [oracle.chain_u(x[r], float(u[r]), **kw)[0] for r in range(len(rows))]
        got = [int(v) for v in run_rows(hs, torch, x, u, SampleParams.make(**kw), None, None)]
        assert got == want, kw
        if kw["top_k"] == 0 and kw["min_p"] == 0.0:
            assert want == [n - 1] * len(rows)
