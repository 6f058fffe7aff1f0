"""The output head in front of the sampler on the device -- RMS norm and the tied F16 lm_head
(src/archs/transformer/forward/head.c:94-129 of the reference) -- through the C ABI against the
oracle, which is itself pinned bit for bit to the reference's compiled kernel
(tests/test_lm_head_oracle.py). Every float must agree in every bit."""
import numpy as np
import pytest

from gpu_util import fuzz_seeds, to_dev

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hs():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from geistlib_amd import HipSampler
    s = HipSampler(max_rows=32, max_vocab=40000)
    yield s
    s.close()


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def run_gemv(hs, w16, x):
    d_w = to_dev(w16.view(np.int16), torch)
    d_x = to_dev(x, torch)
    y = torch.full((x.shape[0], w16.shape[0]), 7.0, dtype=torch.float32, device="cuda")
    hs.f16_gemv(d_w, d_x, y)
    hs.sync()
    return y.cpu().numpy()


@pytest.mark.parametrize("n_out,n_in,m", [(1000, 2560, 1), (130, 64, 1), (129, 128, 3),
                                          (4097, 1536, 2), (300, 8, 1), (300, 16, 5), (257, 24, 4),
                                          (31, 2568, 8), (640, 4096, 16), (500, 2560, 17),
                                          (50, 72, 16), (33, 40, 9), (1, 2560, 1)])
def test_f16_gemv_rows_bit_exact(hs, oracle, n_out, n_in, m):
    print(f"gemv n_out={n_out} n_in={n_in} m={m}", flush=True)
    g = np.random.default_rng(n_out * 7 + n_in + m)
    w16 = (g.standard_normal((n_out, n_in)) * g.choice([0.02, 1.0])).astype(np.float16).view(np.uint16)
    x = (g.standard_normal((m, n_in)) * g.choice([0.1, 1.0, 30.0], (m, 1))).astype(np.float32)
    got = run_gemv(hs, w16, x)
    want = oracle.f16_gemv(w16, x)
    assert (bits(got) == bits(want)).all(), np.argwhere(bits(got) != bits(want))[:5]


def test_f16_gemv_special_values(hs, oracle):
    """Subnormal and extreme binary16 weights, zeros of both signs, a row of zeros with negative
    activations (the sign of a zero result is part of the result)."""
    n_out, n_in = 64, 96
    g = np.random.default_rng(3)
    w = g.standard_normal((n_out, n_in)).astype(np.float16)
    w[0, :] = 0.0
    w[1, :] = -0.0
    w[2, :] = np.float16(6e-8)                     # smallest subnormals
    w[3, :] = np.float16(65504.0)
    w[4, ::2] = np.float16(-65504.0)
    w[5, :] = np.float16(2.0 ** -14)
    w16 = w.view(np.uint16)
    x = np.stack([g.standard_normal(n_in), -np.abs(g.standard_normal(n_in)),
                  np.full(n_in, 1e-30), np.full(n_in, 3e30)]).astype(np.float32)
    got = run_gemv(hs, w16, x)
    want = oracle.f16_gemv(w16, x)
    same = (bits(got) == bits(want)) | (np.isnan(got) & np.isnan(want))
    assert same.all(), np.argwhere(~same)[:5]


def test_f16_gemv_strides_and_errors(hs, oracle):
    from geistlib_amd.binding import GeistHipError
    g = np.random.default_rng(4)
    n_out, n_in, m = 200, 256, 3
    w16 = g.standard_normal((n_out, n_in)).astype(np.float16).view(np.uint16)
    xbuf = np.full((m, n_in + 5), 1e30, dtype=np.float32)
    xbuf[:, :n_in] = g.standard_normal((m, n_in))
    d_x = to_dev(xbuf, torch)[:, :n_in]
    ybuf = torch.full((m, n_out + 3), -1.0, dtype=torch.float32, device="cuda")
    hs.f16_gemv(to_dev(w16.view(np.int16), torch), d_x, ybuf[:, :n_out])
    hs.sync()
    got = ybuf.cpu().numpy()
    assert (bits(got[:, :n_out]) == bits(oracle.f16_gemv(w16, xbuf[:, :n_in]))).all()
    assert (got[:, n_out:] == -1.0).all()
    bad = torch.zeros((4, 20), dtype=torch.float16, device="cuda")        # n_in % 8 != 0
    with pytest.raises(GeistHipError):
        hs.f16_gemv(bad, torch.zeros((1, 20), device="cuda"), torch.zeros((1, 4), device="cuda"))


@pytest.mark.parametrize("rows,n", [(1, 2560), (5, 1536), (17, 4096), (3, 7), (2, 300)])
def test_rmsnorm_rows_bit_exact(hs, oracle, rows, n):
    g = np.random.default_rng(rows * 100 + n)
    x = (g.standard_normal((rows, n)) * g.choice([1e-3, 1.0, 50.0], (rows, 1))).astype(np.float32)
    w = (1.0 + 0.2 * g.standard_normal(n)).astype(np.float32)
    for eps in (1e-6, 1e-5):
        d_x = to_dev(x, torch)
        y = torch.empty_like(d_x)
        hs.rmsnorm(d_x, to_dev(w, torch), eps, y)
        hs.sync()
        assert (bits(y.cpu().numpy()) == bits(oracle.rmsnorm(x, w, eps))).all()
        hs.rmsnorm(d_x, to_dev(w, torch), eps, d_x)                        # in place
        hs.sync()
        assert (bits(d_x.cpu().numpy()) == bits(oracle.rmsnorm(x, w, eps))).all()


def test_head_to_token_without_leaving_the_device(hs, oracle):
    """head.c:94-188 end to end: norm -> lm_head -> sampler, logits never on the host. Equal to
    the oracle's chain on the oracle's logits, token for token."""
    from geistlib_amd import HipSampler, SampleParams
    g = np.random.default_rng(12)
    vocab, d_model, k = 32000, 2560, 6
    w16 = (g.standard_normal((vocab, d_model)) * 0.05).astype(np.float16).view(np.uint16)
    hidden = (g.standard_normal((k, d_model)) * 3).astype(np.float32)
    norm_w = (1.0 + 0.1 * g.standard_normal(d_model)).astype(np.float32)
    u = g.random(k).astype(np.float32)
    d_h = to_dev(hidden, torch)
    hs.rmsnorm(d_h, to_dev(norm_w, torch), 1e-6, d_h)
    logits = torch.empty((k, vocab), dtype=torch.float32, device="cuda")
    hs.f16_gemv(to_dev(w16.view(np.int16), torch), d_h, logits)
    out = torch.empty(k, dtype=torch.int32, device="cuda")
    prm = dict(temperature=0.8, top_k=40, top_p=0.95)
    hs.sample(HipSampler.rows(logits), SampleParams.make(**prm), to_dev(u, torch), out)
    hs.sync()
    want_logits = oracle.f16_gemv(w16, oracle.rmsnorm(hidden, norm_w, 1e-6))
    assert (bits(logits.cpu().numpy()) == bits(want_logits)).all()
    want = [oracle.chain_u(want_logits[r], float(u[r]), **prm)[0] for r in range(k)]
    assert out.cpu().tolist() == want


@pytest.mark.parametrize("rows", [1, 2, 5])
@pytest.mark.parametrize("vocab,d_model", [(32000, 2560), (20001, 136), (8192, 64), (8193, 1536)])
def test_project_sample_rows_equals_the_separate_steps(hs, oracle, rows, vocab, d_model):
    """geist_hip_project_sample_rows: for one or two rows the norm runs inside the projection and,
    on the top-k path without soft-cap, the projection's epilogue replaces the sampler's scan.
    Logits bit-identical to the oracle's, tokens those of the oracle's chain."""
    from geistlib_amd import SampleParams
    print(f"project rows={rows} vocab={vocab} d_model={d_model}", flush=True)
    g = np.random.default_rng(rows * 1000 + vocab + d_model)
    w16 = (g.standard_normal((vocab, d_model)) * 0.05).astype(np.float16).view(np.uint16)
    hidden = (g.standard_normal((rows, d_model)) * 3).astype(np.float32)
    norm_w = (1.0 + 0.1 * g.standard_normal(d_model)).astype(np.float32)
    u = g.random(rows).astype(np.float32)
    normed_want = oracle.rmsnorm(hidden, norm_w, 1e-6)
    # one row: the x86 decode kernel; more: the portable kernel that backend runs for batches
    want_logits = (oracle.f16_gemv(w16, normed_want) if rows == 1
                   else oracle.f16_linear_f64(w16, normed_want))
    d_w, d_h, d_nw, d_u = (to_dev(w16.view(np.int16), torch), to_dev(hidden, torch),
                           to_dev(norm_w, torch), to_dev(u, torch))
    normed = torch.empty((rows, d_model), dtype=torch.float32, device="cuda")
    for prm in (dict(temperature=0.8, top_k=40, top_p=0.95), dict(temperature=0.7, top_k=5),
                dict(temperature=0.0), dict(temperature=1.0), dict(temperature=0.9, top_p=0.9),
                dict(temperature=0.8, top_k=40, softcap=20.0), dict(temperature=0.8, top_k=300)):
        logits = torch.full((rows, vocab), 7.0, dtype=torch.float32, device="cuda")
        out = torch.full((rows,), -3, dtype=torch.int32, device="cuda")
        hs.project_sample(d_h, d_nw, 1e-6, d_w, logits, SampleParams.make(**prm), d_u, out,
                          normed=normed)
        hs.sync()
        assert (bits(logits.cpu().numpy()) == bits(want_logits)).all(), prm
        kw = {k: v for k, v in prm.items() if k != "softcap"}
        want = []
        for r in range(rows):
            row = want_logits[r]
            if prm.get("softcap") and prm["temperature"] > 0:
                row = oracle.softcap(row, prm["softcap"])
            want.append(oracle.argmax(row) if prm["temperature"] <= 0
                        else oracle.chain_u(row, float(u[r]), **kw)[0])
        assert out.cpu().tolist() == want, prm
    assert (d_h.cpu().numpy() == hidden).all()


def test_project_sample_rows_with_the_device_rng(hs, oracle):
    from geistlib_amd import SampleParams
    from geistlib_amd.workloads import xorshift_units
    g = np.random.default_rng(2)
    vocab, d_model, rows = 30000, 512, 2
    w16 = (g.standard_normal((vocab, d_model)) * 0.05).astype(np.float16).view(np.uint16)
    hidden = (g.standard_normal((rows, d_model)) * 3).astype(np.float32)
    norm_w = np.ones(d_model, dtype=np.float32)
    st = torch.tensor([0xABCDEF], dtype=torch.int64, device="cuda")
    logits = torch.empty((rows, vocab), dtype=torch.float32, device="cuda")
    out = torch.empty(rows, dtype=torch.int32, device="cuda")
    hs.project_sample(to_dev(hidden, torch), to_dev(norm_w, torch), 1e-5,
                      to_dev(w16.view(np.int16), torch), logits,
                      SampleParams.make(temperature=0.8, top_k=40), None, out, rng_states=st,
                      normed=torch.empty((rows, d_model), dtype=torch.float32, device="cuda"))
    hs.sync()
    u, after = xorshift_units(0xABCDEF, rows)
    want_logits = oracle.f16_linear_f64(w16, oracle.rmsnorm(hidden, norm_w, 1e-5))
    want = [oracle.top_k_u(want_logits[r], 40, 0.8, float(u[r]))[0] for r in range(rows)]
    assert out.cpu().tolist() == want
    assert int(st.cpu().numpy().view(np.uint64)[0]) == after


@pytest.mark.parametrize("n_out,n_in,m", [(1000, 2560, 1), (130, 128, 1), (129, 256, 3),
                                          (4097, 1536, 2), (300, 16, 1), (300, 32, 5), (257, 48, 4),
                                          (640, 4096, 8), (500, 2560, 11), (33, 144, 2)])
def test_q8w_quantise_and_gemv_bit_exact(hs, oracle, n_out, n_in, m):
    """geist_hip_f16_to_q8w and geist_hip_q8w_gemv_rows against the oracle's restatement of
    f16_to_q8w / q8w_gemv_m1 (kernel_f16_gemv.c:66-127): int8 values, scales and results equal in
    every bit."""
    print(f"q8w n_out={n_out} n_in={n_in} m={m}", flush=True)
    g = np.random.default_rng(n_out + 3 * n_in + m)
    w16 = (g.standard_normal((n_out, n_in)) * g.choice([0.02, 1.0])).astype(np.float16)
    w16[0, :] = 0
    x = (g.standard_normal((m, n_in)) * g.choice([0.1, 1.0, 30.0], (m, 1))).astype(np.float32)
    d_w = to_dev(w16.view(np.int16), torch)
    d_wq = torch.empty((n_out, n_in), dtype=torch.int8, device="cuda")
    d_sc = torch.empty(n_out, dtype=torch.float32, device="cuda")
    hs.f16_to_q8w(d_w, d_wq, d_sc)
    y = torch.full((m, n_out), 7.0, dtype=torch.float32, device="cuda")
    hs.q8w_gemv(d_wq, d_sc, to_dev(x, torch), y)
    hs.sync()
    wq, sc = oracle.f16_to_q8w(w16.view(np.uint16))
    assert (d_wq.cpu().numpy() == wq).all()
    assert (bits(d_sc.cpu().numpy()) == bits(sc)).all()
    want = oracle.q8w_gemv(wq, sc, x)
    got = y.cpu().numpy()
    assert (bits(got) == bits(want)).all(), np.argwhere(bits(got) != bits(want))[:5]


@pytest.mark.parametrize("rows,vocab,d_model", [(1, 40000, 256), (1, 20000, 2560), (2, 9000, 512),
                                                (3, 8200, 128), (9, 5000, 64)])
def test_project_sample_rows_q8w_equals_the_separate_steps(hs, oracle, rows, vocab, d_model):
    """geist_hip_project_sample_rows_q8w: the int8 table in the fused tail. Logits bit-identical
    to the oracle's rmsnorm + q8w_gemv_m1, tokens those of the oracle's chain on them."""
    from geistlib_amd import SampleParams
    print(f"project q8w rows={rows} vocab={vocab} d_model={d_model}", flush=True)
    g = np.random.default_rng(rows * 77 + vocab + d_model)
    w16 = (g.standard_normal((vocab, d_model)) * 0.05).astype(np.float16).view(np.uint16)
    wq, sc = oracle.f16_to_q8w(w16)
    hidden = (g.standard_normal((rows, d_model)) * 3).astype(np.float32)
    norm_w = (1.0 + 0.1 * g.standard_normal(d_model)).astype(np.float32)
    u = g.random(rows).astype(np.float32)
    want_logits = oracle.q8w_gemv(wq, sc, oracle.rmsnorm(hidden, norm_w, 1e-6))
    d_wq, d_sc, d_h, d_nw, d_u = (to_dev(wq, torch), to_dev(sc, torch), to_dev(hidden, torch),
                                  to_dev(norm_w, torch), to_dev(u, torch))
    normed = torch.empty((rows, d_model), dtype=torch.float32, device="cuda")
    for prm in (dict(temperature=0.8, top_k=40, top_p=0.95), dict(temperature=0.0),
                dict(temperature=0.9, top_p=0.9), dict(temperature=0.8, top_k=40, softcap=20.0),
                dict(temperature=0.8, top_k=300)):
        logits = torch.full((rows, vocab), 7.0, dtype=torch.float32, device="cuda")
        out = torch.full((rows,), -3, dtype=torch.int32, device="cuda")
        hs.project_sample_q8w(d_h, d_nw, 1e-6, d_wq, d_sc, logits, SampleParams.make(**prm), d_u,
                              out, normed=normed)
        hs.sync()
        assert (bits(logits.cpu().numpy()) == bits(want_logits)).all(), prm
        kw = {k: v for k, v in prm.items() if k != "softcap"}
        want = []
        for r in range(rows):
            row = want_logits[r]
            if prm.get("softcap") and prm["temperature"] > 0:
                row = oracle.softcap(row, prm["softcap"])
            want.append(oracle.argmax(row) if prm["temperature"] <= 0
                        else oracle.chain_u(row, float(u[r]), **kw)[0])
        assert out.cpu().tolist() == want, prm


def test_project_sample_rows_q8w_rejects_what_it_cannot_take(hs):
    from geistlib_amd import SampleParams
    from geistlib_amd.binding import GeistHipError
    vocab, d_model = 4096, 72                      # a multiple of 8, not of 16
    wq = torch.zeros((vocab, d_model), dtype=torch.int8, device="cuda")
    sc = torch.ones(vocab, dtype=torch.float32, device="cuda")
    h = torch.ones((1, d_model), dtype=torch.float32, device="cuda")
    nw = torch.ones(d_model, dtype=torch.float32, device="cuda")
    logits = torch.empty((1, vocab), dtype=torch.float32, device="cuda")
    out = torch.empty(1, dtype=torch.int32, device="cuda")
    with pytest.raises(GeistHipError):
        hs.project_sample_q8w(h, nw, 1e-6, wq, sc, logits, SampleParams.make(temperature=0.0),
                              None, out, normed=torch.empty_like(h))
    with pytest.raises(GeistHipError):
        hs.project_sample_q8w(h, nw, 1e-6, wq, None, logits, SampleParams.make(temperature=0.0),
                              None, out, normed=torch.empty_like(h))


@pytest.mark.parametrize("n_out,n_in,m", [(1000, 2560, 1), (130, 128, 1), (129, 256, 3),
                                          (4097, 1536, 2), (300, 8, 1), (300, 40, 5), (257, 72, 4),
                                          (640, 4096, 8), (500, 2560, 11), (20000, 2560, 8)])
def test_f16_linear_in_double_bit_exact(hs, oracle, n_out, n_in, m):
    """geist_hip_f16_linear_rows against cpu_scalar_w_quant_mN (weight_resolve.c:215-241): the
    double sum in index order, rounded once -- equal in every bit, also where the sum lies at a
    binary32 rounding boundary (integer inputs make many sums land exactly on one)."""
    print(f"f16 linear f64 n_out={n_out} n_in={n_in} m={m}", flush=True)
    g = np.random.default_rng(n_out + 5 * n_in + m)
    w16 = (g.standard_normal((n_out, n_in)) * g.choice([0.02, 1.0])).astype(np.float16)
    x = (g.standard_normal((m, n_in)) * g.choice([0.1, 1.0, 30.0], (m, 1))).astype(np.float32)
    if n_out > 256:
        # rows whose sums are exact halves of a binary32 step: every order must agree there too
        w16[:128] = g.integers(-4, 5, (128, n_in)).astype(np.float16)
        x[0] = g.integers(-3, 4, n_in).astype(np.float32)
        x[0, 0] += np.float32(2.0 ** -20)
    y = torch.full((m, n_out), 7.0, dtype=torch.float32, device="cuda")
    hs.f16_linear(to_dev(w16.view(np.int16), torch), to_dev(x, torch), y)
    hs.sync()
    want = oracle.f16_linear_f64(w16.view(np.uint16), x)
    got = y.cpu().numpy()
    assert (bits(got) == bits(want)).all(), np.argwhere(bits(got) != bits(want))[:5]


@pytest.mark.parametrize("m", [1, 3, 7])
def test_f16_linear_in_double_at_the_ends_of_the_range(hs, oracle, m):
    """Sums that overflow binary32, sums in its subnormal range, zero rows, weights that are
    binary16 subnormals and infinities: the vector kernels (m <= 4) and the matrix-core kernel
    agree with the oracle in every bit (NaN where it has NaN)."""
    g = np.random.default_rng(m)
    n_out, n_in = 700, 512
    w16 = (g.standard_normal((n_out, n_in)) * 0.05).astype(np.float16)
    w16[0] = 0
    w16[1] = np.float16(6.0e-8)                       # the smallest binary16 subnormals
    w16[2] = np.float16(65504.0)                      # the largest binary16
    w16[3, 5] = np.float16(np.inf)
    w16[4, 7] = np.float16(-np.inf)
    w16[4, 9] = np.float16(np.inf)                    # inf - inf
    x = (g.standard_normal((m, n_in)) * 3).astype(np.float32)
    x[0] = np.float32(1.0e-38)                        # subnormal results against rows of 0.05
    if m > 1:
        x[1] = np.float32(3.0e38)                     # overflows against every row of one sign
        x[1, ::2] *= -1
        x[1, :4] = np.float32(3.0e38)
    y = torch.full((m, n_out), 7.0, dtype=torch.float32, device="cuda")
    hs.f16_linear(to_dev(w16.view(np.int16), torch), to_dev(x, torch), y)
    hs.sync()
    want = oracle.f16_linear_f64(w16.view(np.uint16), x)
    got = y.cpu().numpy()
    nan = np.isnan(want)
    assert (np.isnan(got) == nan).all()
    assert (bits(got)[~nan] == bits(want)[~nan]).all(), np.argwhere(bits(got) != bits(want))[:5]
    assert np.isinf(want).any() and nan.any() and (np.abs(want[0, 5:]) < 1.2e-38).any()


@pytest.mark.parametrize("m", [2, 9, 19])
def test_f16_linear_in_double_with_row_strides(hs, oracle, m):
    """Padded rows on both sides (row strides above the row lengths), 19 rows in two passes of the
    matrix-core kernel; the padding of the output is left alone."""
    g = np.random.default_rng(40 + m)
    n_out, n_in = 3000, 1536
    w16 = (g.standard_normal((n_out, n_in)) * 0.05).astype(np.float16)
    xbuf = (g.standard_normal((m, n_in + 24)) * 2).astype(np.float32)
    d_x = to_dev(xbuf, torch)
    y = torch.full((m, n_out + 8), 7.0, dtype=torch.float32, device="cuda")
    hs.f16_linear(to_dev(w16.view(np.int16), torch), d_x[:, :n_in], y[:, :n_out])
    hs.sync()
    got = y.cpu().numpy()
    want = oracle.f16_linear_f64(w16.view(np.uint16), xbuf[:, :n_in])
    assert (bits(got[:, :n_out]) == bits(want)).all()
    assert (got[:, n_out:] == 7.0).all()


def test_project_sample_rows_in_the_portable_backends_arithmetic(hs, oracle):
    """geist_hip_sampler_set_projection(PORTABLE): one row goes through the double-accumulation
    kernel too, as on the reference's cpu_scalar backend."""
    from geistlib_amd import SampleParams
    g = np.random.default_rng(61)
    vocab, d_model = 30000, 1536
    w16 = (g.standard_normal((vocab, d_model)) * 0.05).astype(np.float16).view(np.uint16)
    hidden = (g.standard_normal((1, d_model)) * 3).astype(np.float32)
    norm_w = (1.0 + 0.1 * g.standard_normal(d_model)).astype(np.float32)
    u = g.random(1).astype(np.float32)
    normed_want = oracle.rmsnorm(hidden, norm_w, 1e-6)
    logits = torch.empty((1, vocab), dtype=torch.float32, device="cuda")
    out = torch.empty(1, dtype=torch.int32, device="cuda")
    args = (to_dev(hidden, torch), to_dev(norm_w, torch), 1e-6, to_dev(w16.view(np.int16), torch),
            logits, SampleParams.make(temperature=0.8, top_k=40), to_dev(u, torch), out)
    normed = torch.empty((1, d_model), dtype=torch.float32, device="cuda")
    try:
        hs.set_projection(True)
        hs.project_sample(*args, normed=normed)
        hs.sync()
        want = oracle.f16_linear_f64(w16, normed_want)
        assert (bits(logits.cpu().numpy()) == bits(want)).all()
        assert out.cpu().tolist() == [oracle.top_k_u(want[0], 40, 0.8, float(u[0]))[0]]
    finally:
        hs.set_projection(False)
    hs.project_sample(*args, normed=normed)
    hs.sync()
    assert (bits(logits.cpu().numpy()) == bits(oracle.f16_gemv(w16, normed_want))).all()


@pytest.mark.parametrize("seed", fuzz_seeds(4))
def test_random_projection_shapes(hs, oracle, seed):
    """Norm, F16 and int8 projections, the quantiser and the projection in double on random
    shapes, scales and row counts, each against the oracle in every bit. Integer-valued and
    cancelling data put the sums in double on rounding boundaries of binary32."""
    g = np.random.default_rng(9000 + seed)
    for case in range(5):
        n_out = int(g.integers(1, 5000))
        n_in = 16 * int(g.integers(1, 257)) + (8 if g.random() < 0.3 else 0)
        m = int(g.integers(1, 21))
        kind = int(g.integers(0, 3))
        print(f"projection seed {seed} case {case}: n_out={n_out} n_in={n_in} m={m} kind={kind}",
              flush=True)
        w = (g.standard_normal((n_out, n_in)) * g.choice([1e-3, 0.05, 1.0, 30.0])).astype(np.float16)
        x = (g.standard_normal((m, n_in)) * g.choice([1e-3, 1.0, 100.0], (m, 1))).astype(np.float32)
        if kind == 1:
            w = g.integers(-6, 7, (n_out, n_in)).astype(np.float16)
            x = g.integers(-5, 6, (m, n_in)).astype(np.float32)
            x[:, 0] += np.float32(2.0 ** -int(g.integers(10, 30)))
        if kind == 2:
            w[:, 1::2] = -w[:, ::2]
            x[:, 1::2] = x[:, ::2] * np.float32(1 + 2.0 ** -12)
        w16 = w.view(np.uint16)
        d_w, d_x = to_dev(w.view(np.int16), torch), to_dev(x, torch)
        y = torch.full((m, n_out), 7.0, dtype=torch.float32, device="cuda")
        hs.f16_gemv(d_w, d_x, y)
        hs.sync()
        assert (bits(y.cpu().numpy()) == bits(oracle.f16_gemv(w16, x))).all()
        y.fill_(7.0)
        hs.f16_linear(d_w, d_x, y)
        hs.sync()
        assert (bits(y.cpu().numpy()) == bits(oracle.f16_linear_f64(w16, x))).all()
        if n_in % 16 == 0:
            wq = torch.empty((n_out, n_in), dtype=torch.int8, device="cuda")
            sc = torch.empty(n_out, dtype=torch.float32, device="cuda")
            hs.f16_to_q8w(d_w, wq, sc)
            hs.sync()
            wq_want, sc_want = oracle.f16_to_q8w(w16)
            assert (wq.cpu().numpy() == wq_want).all()
            assert (bits(sc.cpu().numpy()) == bits(sc_want)).all()
            y.fill_(7.0)
            hs.q8w_gemv(wq, sc, d_x, y)
            hs.sync()
            assert (bits(y.cpu().numpy()) == bits(oracle.q8w_gemv(wq_want, sc_want, x))).all()
        norm_w = g.standard_normal(n_in).astype(np.float32)
        eps = float(g.choice([1e-5, 1e-6, 0.0]))
        normed = torch.empty((m, n_in), dtype=torch.float32, device="cuda")
        hs.rmsnorm(d_x, to_dev(norm_w, torch), eps, normed)
        hs.sync()
        assert (bits(normed.cpu().numpy()) == bits(oracle.rmsnorm(x, norm_w, eps))).all()


@pytest.mark.parametrize("m", [1, 2, 5, 9, 14])
def test_f16_linear_in_double_on_order_sensitive_rows(hs, oracle, m):
    """Rows whose last quarter cancels a huge first quarter: the small terms in between are added
    to a sum 2^24 times their size, so the binary32 result depends on the ORDER of the additions in
    double (numpy's own float64 product rounds some of these outputs to another value). The
    device kernels add in another order and re-add, in index order, what their bound cannot
    decide: every bit equals the oracle, which equals the reference's cpu_scalar_w_quant_mN
    compiled from its tree (tests/test_lm_head_oracle.py)."""
    g = np.random.default_rng(900 + m)
    n_out, n_in = 3000, 1024
    q = n_in // 4
    w = (g.standard_normal((n_out, n_in)) * 4).astype(np.float16)
    x = (g.standard_normal((m, n_in)) * 100).astype(np.float32)
    x[:, :q] *= np.float32(2.0 ** 24)
    w[:, 3 * q: 4 * q] = -w[:, :q]
    x[:, 3 * q: 4 * q] = x[:, :q]
    y = torch.full((m, n_out), float("nan"), dtype=torch.float32, device="cuda")
    hs.f16_linear(to_dev(w.view(np.int16), torch), to_dev(x, torch), y)
    hs.sync()
    want = np.atleast_2d(oracle.f16_linear_f64(w.view(np.uint16), x if m > 1 else x[0]))
    got = y.cpu().numpy()
    other = (x.astype(np.float64) @ w.astype(np.float64).T).astype(np.float32)
    assert (other != want).any()          # the case does hang on the order
    assert (got.view(np.uint32) == want.view(np.uint32)).all(), int((got != want).sum())
