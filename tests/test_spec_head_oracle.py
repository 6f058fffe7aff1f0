"""The oracle's restatement of the reference's speculative output head
(src/archs/transformer/forward/spec_head.c), pinned by what its construction fixes: the reference
file does not compile on its own and its test needs a model file."""
import numpy as np
import pytest

from oracle_lib import Oracle


@pytest.fixture(scope="module")
def oracle():
    return Oracle()


def table(g, vocab, d_model, scale=0.05, hot=None):
    w = (g.standard_normal((vocab, d_model)) * scale).astype(np.float32)
    if hot is not None:                      # a few dimensions carry most of the variance
        w[:, hot] *= 6.0
    return w.astype(np.float16)


def test_geometry_follows_the_reference_rules(oracle):
    """spec_head.c:431-452: stride d_model / 640 lowered to a divisor, 1024 finalists (4096 from
    200000 tokens on), no sketch below 8192 tokens or where a row shrinks less than 3x."""
    assert oracle.spec_head_geometry(128256, 2560) == (640, 1024)      # BitNet 2B-4T
    assert oracle.spec_head_geometry(262144, 1536) == (768, 4096)
    assert oracle.spec_head_geometry(32000, 4096) == (1024, 1024)      # 4096 / 6 -> stride 4
    assert oracle.spec_head_geometry(8191, 2560) is None
    assert oracle.spec_head_geometry(50000, 512) is None               # stride 1: 2x < 3x
    assert oracle.spec_head_geometry(50000, 2560, stride=8) == (320, 1024)
    assert oracle.spec_head_geometry(50000, 2560, stride=7) == (512, 1024)   # 7, 6 do not divide
    assert oracle.spec_head_geometry(50000, 2560, topk=3) == (640, 16)
    assert oracle.spec_head_geometry(50000, 2560, topk=10 ** 9) == (640, 50000)


def test_build_against_numpy(oracle):
    g = np.random.default_rng(1)
    vocab, d_model = 9000, 1280
    hot = g.choice(d_model, 300, replace=False)
    w16 = table(g, vocab, d_model, hot=hot)
    sh = oracle.spec_head_build(w16.view(np.uint16))
    assert sh is not None and sh.sketch_dim == 640 and sh.topk == 1024
    w = w16.astype(np.float64)
    # kept dimensions: the 640 largest sampled variances (every (vocab // 512)-th row)
    sample = w[:: vocab // 512]
    var = (sample ** 2).mean(0) - sample.mean(0) ** 2
    want_dims = np.sort(np.argsort(-var, kind="stable")[:640])
    order = np.sort(var)[::-1]
    assert order[639] - order[640] > 1e-9            # the edge is not a float32 near-tie here
    assert (sh.dims == want_dims).all()
    assert set(hot) <= set(sh.dims.tolist())
    # sketch rows and scales: max and rint are order-free, so float32 numpy reproduces them
    kept = w16.astype(np.float32)[:, sh.dims]
    amax = np.maximum(np.abs(kept).max(1), np.float32(1e-8))
    assert (sh.row_scale.view(np.uint32) == (amax / np.float32(127.0)).view(np.uint32)).all()
    q = np.clip(np.rint(kept * (np.float32(127.0) / amax)[:, None]), -127, 127).astype(np.int8)
    assert (sh.sketch == q).all()
    # the two row norms of the bound, against float64
    dropped = np.ones(d_model, bool)
    dropped[sh.dims] = False
    assert np.allclose(sh.w_l1, np.abs(w[:, sh.dims]).sum(1), rtol=1e-5)
    assert np.allclose(sh.w_drop, np.sqrt((w[:, dropped] ** 2).sum(1)), rtol=1e-5)


def test_rough_scores_and_finalists_against_numpy(oracle):
    g = np.random.default_rng(2)
    vocab, d_model = 12000, 1280
    w16 = table(g, vocab, d_model)
    sh = oracle.spec_head_build(w16.view(np.uint16), topk=200)
    h = (g.standard_normal(d_model) * 2).astype(np.float32)
    r = sh.try_row(h)
    amax = max(np.abs(h).max(), np.float32(1e-8))
    x_i8 = np.clip(np.rint(h * (np.float32(127.0) / amax)), -127, 127).astype(np.int64)
    d = sh.sketch.astype(np.int64) @ x_i8[sh.dims]
    want = d.astype(np.float32) * sh.row_scale
    assert (r["rough"].view(np.uint32) == want.view(np.uint32)).all()
    srt = np.sort(want)[::-1]
    assert r["n_finalists"] == 200 and r["cutoff"] == srt[199]
    # the token is the best exact logit among the 200 best rough scores
    assert srt[199] > srt[200]
    finalists = np.flatnonzero(want >= srt[199])
    exact = oracle.f16_gemv(w16.view(np.uint16)[finalists], h)
    assert r["token"] == finalists[np.flatnonzero(exact == exact.max())[0]]


def test_the_bound_holds_for_every_row(oracle):
    """spec_head.c:831-872: rough / x_q + the three error terms is an upper bound of the exact
    logit of every row; checked in float64 on a table with heavy dropped dimensions."""
    g = np.random.default_rng(3)
    vocab, d_model = 9000, 1280
    w16 = table(g, vocab, d_model, scale=0.2)
    w16[::7, g.choice(d_model, 40)] *= np.float16(3.0)
    sh = oracle.spec_head_build(w16.view(np.uint16))
    for scale in (0.5, 4.0):
        h = (g.standard_normal(d_model) * scale).astype(np.float32)
        r = sh.try_row(h)
        amax = np.abs(h).max()
        inv_xq = np.float64(amax) / 127.0
        kept = np.zeros(d_model, bool)
        kept[sh.dims] = True
        h64 = h.astype(np.float64)
        ub = (r["rough"].astype(np.float64) * inv_xq + 0.5 * sh.row_scale * np.abs(h64[kept]).sum()
              + 0.5 * sh.w_l1 * inv_xq + sh.w_drop * np.sqrt((h64[~kept] ** 2).sum()))
        exact = w16.astype(np.float64) @ h64
        assert (exact <= ub * (1 + 1e-6) + 1e-6).all()


def test_verified_answers_are_the_dense_heads(oracle):
    """The contract of tests/test_spec_head_sampling_int.c: with the bound on, an answer is the
    dense head's argmax. Tables whose decisive weight sits in dropped dimensions make the sketch
    misrank: without the bound the head then answers wrongly (so this check can fail), with it the
    head declines."""
    g = np.random.default_rng(4)
    vocab, d_model = 9000, 1280
    hot = np.arange(0, d_model, 2)
    w16 = table(g, vocab, d_model, hot=hot)                  # the sketch keeps the even dimensions
    sh = oracle.spec_head_build(w16.view(np.uint16), topk=16)
    assert (sh.dims == hot).all()
    answered = wrong_unverified = 0
    for trial in range(40):
        h = (g.standard_normal(d_model)).astype(np.float32)
        if trial % 2:                                        # all the signal in dropped dimensions
            h[hot] *= 0.01
        dense = oracle.f16_gemv(w16.view(np.uint16), h)
        want = int(np.flatnonzero(dense == dense.max())[0])
        r = sh.try_row(h, verify=True)
        if r["certain"]:
            answered += 1
            assert r["token"] == want, trial
        wrong_unverified += sh.try_row(h, verify=False)["token"] != want
    assert wrong_unverified > 0
    # an easy case the bound does certify: one row far above the rest in the kept dimensions
    w_easy = w16.copy()
    h = np.zeros(d_model, dtype=np.float32)
    h[hot[:64]] = 1.0
    w_easy[1234, hot[:64]] = np.float16(8.0)
    sh2 = oracle.spec_head_build(w_easy.view(np.uint16), topk=16)
    r = sh2.try_row(h, verify=True)
    assert r["certain"] and r["token"] == 1234
