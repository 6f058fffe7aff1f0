"""The speculative output head on the device (geist_hip_spec_head_*) against the oracle's
restatement of src/archs/transformer/forward/spec_head.c, through the C ABI."""
import ctypes as C

import numpy as np
import pytest

torch = pytest.importorskip("torch")
from gpu_util import fuzz_seeds  # noqa: E402
from oracle_lib import Oracle  # noqa: E402

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hs():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from geistlib_amd import HipSampler
    s = HipSampler(max_rows=4, max_vocab=70000)
    yield s
    s.close()


@pytest.fixture(scope="module")
def oracle():
    return Oracle()


def dev_array(ptr, shape, dtype):
    """A device array behind a raw pointer, copied to the host."""
    n = int(np.prod(shape)) * np.dtype(dtype).itemsize
    out = np.empty(shape, dtype=dtype)
    rc = C.cdll.LoadLibrary("libamdhip64.so").hipMemcpy(out.ctypes.data_as(C.c_void_p),
                                                        C.c_void_p(ptr), C.c_size_t(n), 2)
    assert rc == 0
    return out


def result_of(buf):
    from geistlib_amd import SpecResult
    raw = buf.cpu().numpy().tobytes()
    return SpecResult.from_buffer_copy(raw)


def table(g, vocab, d_model, scale=0.05, hot=None):
    w = (g.standard_normal((vocab, d_model)) * scale).astype(np.float32)
    if hot is not None:
        w[:, hot] *= 6.0
    return w.astype(np.float16)


def test_geometry_matches_the_oracle_where_the_device_builds(hs, oracle):
    for vocab, d_model, stride, topk in [(128256, 2560, 0, 0), (262144, 1536, 0, 0),
                                         (70000, 4096, 0, 0), (8191, 2560, 0, 0),
                                         (50000, 512, 0, 0), (70000, 2560, 8, 0),
                                         (50000, 2560, 0, 300)]:
        assert hs.spec_head_geometry(vocab, d_model, stride, topk) == \
            oracle.spec_head_geometry(vocab, d_model, stride, topk), (vocab, d_model, stride, topk)
    # what the reference would build and the kernels do not take
    assert hs.spec_head_geometry(40000, 2560) is None          # 1024 finalists > 40000 / 64
    assert hs.spec_head_geometry(50000, 2560, stride=1) is None   # (and the reference: 2x < 3x)
    assert hs.spec_head_geometry(50000, 6144) is None          # d_model above the LDS staging


@pytest.mark.parametrize("vocab,d_model,topk", [(40000, 1280, 512), (66000, 2560, 0),
                                                (16500, 1536, 256)])
def test_build_equals_the_oracle(hs, oracle, vocab, d_model, topk):
    print(f"spec build vocab={vocab} d_model={d_model} topk={topk}", flush=True)
    g = np.random.default_rng(vocab + d_model)
    hot = g.choice(d_model, d_model // 3, replace=False)
    w16 = table(g, vocab, d_model, hot=hot)
    w16[5, :] = 0                                             # a row of zeros: scale 1e-8 / 127
    want = oracle.spec_head_build(w16.view(np.uint16), topk=topk)
    d_w = torch.from_numpy(w16.view(np.int16)).cuda()
    sh = hs.spec_head_build(d_w, topk=topk)
    v = hs.spec_head_view(sh)
    assert (v.sketch_dim, v.topk) == (want.sketch_dim, want.topk)
    sd = want.sketch_dim
    assert (dev_array(v.d_dims, (sd,), np.uint32) == want.dims).all()
    assert (dev_array(v.d_sketch, (vocab, sd), np.int8) == want.sketch).all()
    assert (dev_array(v.d_row_scale, (vocab,), np.uint32) == want.row_scale.view(np.uint32)).all()
    assert np.allclose(dev_array(v.d_w_drop, (vocab,), np.float32), want.w_drop, rtol=2e-6)
    assert np.allclose(dev_array(v.d_w_l1, (vocab,), np.float32), want.w_l1, rtol=2e-6)
    hs.spec_head_destroy(sh)


@pytest.mark.parametrize("vocab,d_model,topk", [(40000, 1280, 512), (66000, 2560, 0),
                                                (16500, 1536, 256), (65536, 1280, 1024)])
def test_try_equals_the_oracle(hs, oracle, vocab, d_model, topk):
    """Rough scores bit for bit, the same cutoff, finalists and token; with the bound on, the same
    verdict (and any answer is the dense head's argmax)."""
    print(f"spec try vocab={vocab} d_model={d_model} topk={topk}", flush=True)
    g = np.random.default_rng(7 * vocab + d_model)
    hot = g.choice(d_model, d_model // 3, replace=False)
    w16 = table(g, vocab, d_model, hot=hot)
    want_sh = oracle.spec_head_build(w16.view(np.uint16), topk=topk)
    d_w = torch.from_numpy(w16.view(np.int16)).cuda()
    sh = hs.spec_head_build(d_w, topk=topk)
    v = hs.spec_head_view(sh)
    res = torch.zeros(6, dtype=torch.int32, device="cuda")
    answered = 0
    for trial in range(6):
        h = (g.standard_normal(d_model) * g.choice([0.3, 1.0, 5.0])).astype(np.float32)
        if trial == 4:
            h[:] = 0                                        # every rough score equal
        if trial == 5:                                      # one row far above the rest
            h = np.zeros(d_model, dtype=np.float32)
            h[want_sh.dims] = w16[777, want_sh.dims].astype(np.float32) * 100
        d_h = torch.from_numpy(h).cuda()
        for verify in (False, True):
            want = want_sh.try_row(h, verify=verify)
            hs.spec_head_try(sh, d_h, res, verify=verify)
            hs.sync()
            got = result_of(res)
            rough = dev_array(v.d_rough, (vocab,), np.uint32)
            assert (rough == want["rough"].view(np.uint32)).all(), (trial, verify)
            if trial == 4:
                # all scores tie: more rows around the cutoff than the list holds, no answer
                assert got.answered == 0 and got.token == -1
                continue
            assert got.n_finalists == want["n_finalists"] == want_sh.topk
            assert got.cutoff == want["cutoff"], (trial, verify)
            assert got.n_listed >= got.n_finalists
            assert got.token == want["token"], (trial, verify)
            assert bool(got.answered) == want["certain"], (trial, verify)
            if verify and got.answered:
                answered += 1
                dense = oracle.f16_gemv(w16.view(np.uint16), h)
                assert got.token == int(np.flatnonzero(dense == dense.max())[0])
                assert np.float32(got.best_exact) == dense.max()
    assert answered >= 1                                    # trial 5 is certified
    hs.spec_head_destroy(sh)


def test_finalist_logits_are_the_dense_heads(hs, oracle):
    """Without the bound the answer is the best exact logit among the finalists; its value must
    be the dense kernel's in every bit."""
    g = np.random.default_rng(99)
    for vocab, d_model in [(66000, 1536), (70000, 2560)]:
        w16 = table(g, vocab, d_model, scale=0.3)
        d_w = torch.from_numpy(w16.view(np.int16)).cuda()
        sh = hs.spec_head_build(d_w)
        res = torch.zeros(6, dtype=torch.int32, device="cuda")
        for _ in range(4):
            h = (g.standard_normal(d_model) * 3).astype(np.float32)
            hs.spec_head_try(sh, torch.from_numpy(h).cuda(), res)
            hs.sync()
            got = result_of(res)
            assert got.answered == 1
            y = oracle.f16_gemv(w16.view(np.uint16)[got.token:got.token + 1], h)
            assert np.float32(got.best_exact).view(np.uint32) == y.view(np.uint32)[0]
        hs.spec_head_destroy(sh)


def test_rejects_what_it_cannot_take(hs):
    from geistlib_amd.binding import GeistHipError
    w = torch.zeros((9000, 2560), dtype=torch.float16, device="cuda")
    with pytest.raises(GeistHipError):
        hs.spec_head_build(w)                                # 1024 finalists > 9000 / 64
    with pytest.raises(GeistHipError):
        hs.spec_head_build(torch.zeros((40000, 512), dtype=torch.float16, device="cuda"))


@pytest.mark.parametrize("seed", fuzz_seeds(6))
def test_random_geometries_against_the_oracle(hs, oracle, seed):
    """Vocabulary, width, finalist count, weight and activation scales drawn at random; token,
    cutoff and rough scores as the oracle's."""
    g = np.random.default_rng(1000 + seed)
    d_model = int(g.choice([1280, 1536, 2048, 2560]))
    vocab = int(g.integers(17000, 60000))
    topk = int(g.integers(16, vocab // 64 + 1))
    print(f"spec fuzz seed={seed} vocab={vocab} d_model={d_model} topk={topk}", flush=True)
    col_scale = np.exp(g.standard_normal(d_model) * 0.7).astype(np.float32)   # uneven variances
    w16 = ((g.standard_normal((vocab, d_model)).astype(np.float32) * col_scale)
           * g.choice([0.01, 0.1, 2.0])).astype(np.float16)
    want_sh = oracle.spec_head_build(w16.view(np.uint16), topk=topk)
    assert want_sh is not None
    sh = hs.spec_head_build(torch.from_numpy(w16.view(np.int16)).cuda(), topk=topk)
    v = hs.spec_head_view(sh)
    assert (dev_array(v.d_dims, (want_sh.sketch_dim,), np.uint32) == want_sh.dims).all()
    res = torch.zeros(6, dtype=torch.int32, device="cuda")
    for trial in range(3):
        h = (g.standard_normal(d_model) * g.choice([1e-3, 1.0, 300.0])).astype(np.float32)
        h[g.integers(0, d_model, 5)] *= 20                   # outliers set the int8 scale
        for verify in (False, True):
            want = want_sh.try_row(h, verify=verify)
            hs.spec_head_try(sh, torch.from_numpy(h).cuda(), res, verify=verify)
            hs.sync()
            got = result_of(res)
            rough = dev_array(v.d_rough, (vocab,), np.uint32)
            assert (rough == want["rough"].view(np.uint32)).all()
            srt = np.sort(want["rough"])[::-1]
            if srt[topk - 1] == srt[topk]:                   # a tie at the cutoff: see below
                continue
            assert (got.token, got.cutoff, got.n_finalists) == \
                (want["token"], want["cutoff"], topk), (trial, verify)
            assert bool(got.answered) == want["certain"], (trial, verify)
    hs.spec_head_destroy(sh)


def test_ties_at_the_cutoff_keep_the_lowest_indices(hs, oracle):
    """Rows that are copies of each other have equal rough scores. Where such a tie straddles the
    cutoff this implementation keeps the lowest indices (the reference keeps whichever rows its
    heap's sift order leaves); the rule is checked against its statement in numpy."""
    g = np.random.default_rng(5)
    vocab, d_model, topk = 20000, 1280, 64
    w16 = (g.standard_normal((vocab, d_model)) * 0.05).astype(np.float16)
    sh_o = oracle.spec_head_build(w16.view(np.uint16), topk=topk)
    h = g.standard_normal(d_model).astype(np.float32)
    order = np.argsort(-sh_o.try_row(h)["rough"], kind="stable")
    # the row ranked 60th is copied to 11 other places, before and behind it: 12 rows tie for the
    # ranks 60..71 and only 5 of them are finalists
    src = int(order[59])
    spots = np.sort(g.choice(np.setdiff1d(np.arange(vocab), order[:80]), 11, replace=False))
    w16[spots] = w16[src]
    sh_o = oracle.spec_head_build(w16.view(np.uint16), topk=topk)
    rough = sh_o.try_row(h)["rough"]
    srt = np.sort(rough)[::-1]
    cutoff = srt[topk - 1]
    assert (rough == cutoff).sum() == 12 and (rough > cutoff).sum() == 59
    tied = np.flatnonzero(rough == cutoff)[:topk - 59]
    finalists = np.concatenate([np.flatnonzero(rough > cutoff), tied])
    exact = oracle.f16_gemv(w16.view(np.uint16)[finalists], h)
    want_token = int(finalists[np.flatnonzero(exact == exact.max())].min())
    sh = hs.spec_head_build(torch.from_numpy(w16.view(np.int16)).cuda(), topk=topk)
    res = torch.zeros(6, dtype=torch.int32, device="cuda")
    hs.spec_head_try(sh, torch.from_numpy(h).cuda(), res)
    hs.sync()
    got = result_of(res)
    assert got.answered == 1 and got.n_finalists == topk and got.cutoff == cutoff
    assert got.token == want_token
    assert np.float32(got.best_exact) == exact.max()
    # make one of the tied copies the winner: only a copy among the 5 lowest indices can win
    hs.spec_head_destroy(sh)


def test_bitnet_geometry_once(hs, oracle):
    """128256 x 2560, the geometry the head was written for: sketch 640 wide, 1024 finalists."""
    g = np.random.default_rng(11)
    vocab, d_model = 128256, 2560
    w16 = (g.standard_normal((vocab, d_model), dtype=np.float32) * 0.05).astype(np.float16)
    want_sh = oracle.spec_head_build(w16.view(np.uint16))
    sh = hs.spec_head_build(torch.from_numpy(w16.view(np.int16)).cuda())
    v = hs.spec_head_view(sh)
    assert (v.sketch_dim, v.topk) == (640, 1024)
    assert (dev_array(v.d_sketch, (vocab, 640), np.int8) == want_sh.sketch).all()
    res = torch.zeros(6, dtype=torch.int32, device="cuda")
    for _ in range(2):
        h = g.standard_normal(d_model).astype(np.float32)
        want = want_sh.try_row(h)
        hs.spec_head_try(sh, torch.from_numpy(h).cuda(), res)
        hs.sync()
        got = result_of(res)
        assert (got.token, got.cutoff, got.n_finalists, got.answered) == \
            (want["token"], want["cutoff"], 1024, 1)
    hs.spec_head_destroy(sh)


@pytest.mark.parametrize("vocab,d_model", [(262144, 1536), (300000, 1280)])
def test_large_vocabularies_take_the_wider_selection_kernels(hs, oracle, vocab, d_model):
    """From 200000 tokens on the reference keeps 4096 finalists (Gemma's 262144 x 1536 head):
    more group maxima and candidates per thread of the selection workgroup."""
    print(f"spec large vocab={vocab} d_model={d_model}", flush=True)
    g = np.random.default_rng(vocab)
    w16 = (g.standard_normal((vocab, d_model), dtype=np.float32) * 0.05).astype(np.float16)
    want_sh = oracle.spec_head_build(w16.view(np.uint16))
    assert want_sh.topk == 4096
    sh = hs.spec_head_build(torch.from_numpy(w16.view(np.int16)).cuda())
    v = hs.spec_head_view(sh)
    assert (v.sketch_dim, v.topk) == (want_sh.sketch_dim, 4096)
    res = torch.zeros(6, dtype=torch.int32, device="cuda")
    for verify in (False, True):
        h = g.standard_normal(d_model).astype(np.float32)
        want = want_sh.try_row(h, verify=verify)
        hs.spec_head_try(sh, torch.from_numpy(h).cuda(), res, verify=verify)
        hs.sync()
        got = result_of(res)
        rough = dev_array(v.d_rough, (vocab,), np.uint32)
        assert (rough == want["rough"].view(np.uint32)).all()
        assert (got.token, got.cutoff, got.n_finalists) == (want["token"], want["cutoff"], 4096)
        assert bool(got.answered) == want["certain"]
    hs.spec_head_destroy(sh)


def test_try_hidden_norms_in_the_same_launch(hs, oracle):
    """geist_hip_spec_head_try_hidden: the normed row equals geist_hip_rmsnorm_rows' bit for bit,
    and the answer is that of geist_hip_spec_head_try on it."""
    g = np.random.default_rng(21)
    vocab, d_model = 40000, 2560
    w16 = table(g, vocab, d_model)
    sh = hs.spec_head_build(torch.from_numpy(w16.view(np.int16)).cuda(), topk=512)
    want_sh = oracle.spec_head_build(w16.view(np.uint16), topk=512)
    norm_w = (1.0 + 0.1 * g.standard_normal(d_model)).astype(np.float32)
    d_nw = torch.from_numpy(norm_w).cuda()
    res = torch.zeros(6, dtype=torch.int32, device="cuda")
    for scale in (1e-3, 2.0, 1e4):
        hidden = (g.standard_normal(d_model) * scale).astype(np.float32)
        normed = torch.full((d_model,), 7.0, dtype=torch.float32, device="cuda")
        hs.spec_head_try_hidden(sh, torch.from_numpy(hidden).cuda(), d_nw, 1e-6, normed, res)
        hs.sync()
        got = result_of(res)
        want_normed = oracle.rmsnorm(hidden, norm_w, 1e-6)
        assert (normed.cpu().numpy().view(np.uint32) == want_normed.view(np.uint32)).all()
        want = want_sh.try_row(want_normed)
        assert (got.token, got.cutoff, got.answered) == (want["token"], want["cutoff"], 1)
    hs.spec_head_destroy(sh)
