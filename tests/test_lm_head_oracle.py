"""The oracle's lm_head steps (oracle/lm_head_oracle.c) against what pins them: the reference's
own F16 GEMV kernel compiled from its tree (bit for bit), the exact-double reference of the
reference's unit test (tests/test_q8w_gemv_unit.c:49-56), numpy's float16, closed forms of the
norm."""
import ctypes as C

import numpy as np
import pytest

from oracle_lib import load_ref_f16gemv


def weights(g, n_out, n_in, scale=1.0):
    w = (g.standard_normal((n_out, n_in)) * scale).astype(np.float16)
    return w.view(np.uint16)


def test_f16_conversions_match_numpy_on_every_pattern(oracle):
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([oracle.lib.oracle_f16_to_f32(int(b)) for b in bits], dtype=np.float32)
    same = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
    assert same.all()
    # and back: every binary16 value, the midpoints between neighbours, values just beside them
    g = np.random.default_rng(0)
    vals = np.concatenate([want[np.isfinite(want)], g.standard_normal(200000).astype(np.float32) * 3,
                           (g.standard_normal(50000) * 1e-6).astype(np.float32),
                           np.array([65504, 65519.99, 65520, 65536, 1e9, 5.96e-8, 2.98e-8, 2.9802322e-8,
                                     2.9802326e-8, 0, -0.0, np.inf, -np.inf], dtype=np.float32)])
    fin = want[np.isfinite(want)]
    mids = ((fin[:-1].astype(np.float64) + fin[1:].astype(np.float64)) / 2).astype(np.float32)
    vals = np.concatenate([vals, mids, np.nextafter(mids, np.float32(np.inf)),
                           np.nextafter(mids, np.float32(-np.inf))])
    with np.errstate(over="ignore"):
        want16 = vals.astype(np.float16).view(np.uint16)
    got16 = np.array([oracle.lib.oracle_f32_to_f16(float(v)) for v in vals], dtype=np.uint16)
    assert (got16 == want16).all()


@pytest.mark.parametrize("fast", [False, True])
def test_gemv_equals_the_compiled_reference_kernel(oracle, fast):
    """f16_gemv_m1 of the reference (src/backends/cpu_x86/kernel_f16_gemv.c), built with strict
    flags and with the reference's release flags: identical bits for every n_in a model can have
    (multiples of 8), with and without the trailing block of eight."""
    ref = load_ref_f16gemv(fast)
    if ref is None:
        pytest.skip("oracle/_ref not built (needs the reference tree: make -C oracle ref)")
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    got = np.array([ref.fp16_to_fp32(int(b)) for b in bits[::7]], dtype=np.float32)
    want = np.array([oracle.lib.oracle_f16_to_f32(int(b)) for b in bits[::7]], dtype=np.float32)
    assert ((got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))).all()
    g = np.random.default_rng(5)
    for n_out, n_in, scale in [(64, 2560, 1.0), (33, 1536, 0.02), (17, 4096, 30.0), (5, 16, 1.0),
                               (9, 8, 1.0), (7, 24, 1.0), (12, 2568, 1.0), (3, 40, 100.0)]:
        w = weights(g, n_out, n_in, scale)
        x = (g.standard_normal(n_in) * g.choice([0.01, 1.0, 50.0])).astype(np.float32)
        y = np.zeros(n_out, dtype=np.float32)
        ref.f16_gemv_m1(n_out, n_in, x.ctypes.data_as(C.POINTER(C.c_float)),
                        w.ctypes.data_as(C.POINTER(C.c_uint16)),
                        y.ctypes.data_as(C.POINTER(C.c_float)))
        mine = oracle.f16_gemv(w, x)
        assert (mine.view(np.uint32) == y.view(np.uint32)).all(), (n_out, n_in, scale)


def test_gemv_against_the_exact_sum(oracle):
    """tests/test_q8w_gemv_unit.c:49-56: the exact reference is the double-precision dot. The
    fp32 chains stay within n_in * 2^-24 * sum |w x| of it."""
    g = np.random.default_rng(6)
    for n_in in (8, 16, 24, 2560, 2573):           # 2573: the element-by-element tail
        w = weights(g, 40, n_in)
        x = g.standard_normal(n_in).astype(np.float32)
        wf = w.view(np.float16).astype(np.float64)
        exact = wf @ x.astype(np.float64)
        bound = (np.abs(wf) @ np.abs(x.astype(np.float64))) * n_in * 2.0 ** -24
        assert (np.abs(oracle.f16_gemv(w, x) - exact) <= bound).all()
    # one-hot activations pick single weights exactly; signs and zeros survive
    w = weights(g, 10, 32)
    for k in (0, 7, 8, 15, 16, 31):
        x = np.zeros(32, dtype=np.float32)
        x[k] = 2.0
        assert (oracle.f16_gemv(w, x) == 2.0 * w.view(np.float16)[:, k].astype(np.float32)).all()


def test_gemv_order_is_the_documented_one(oracle):
    """A row built so that a different association gives a different float: the chains (element
    k goes to chain k % 16, in order of k / 16), then chain j + chain j+8, lane i + lane i+4,
    (0+1) + (2+3), written out in numpy float32 with fused multiply-adds from math.fma-free
    arithmetic (products of binary16 and small integers are exact)."""
    n_in = 48
    g = np.random.default_rng(8)
    w16 = (g.integers(-8, 9, (6, n_in)) * 2.0 ** g.integers(-10, 11, (6, n_in))).astype(np.float16)
    x = (g.integers(-4, 5, n_in) * 2.0 ** g.integers(-12, 13, n_in)).astype(np.float32)
    prod = w16.astype(np.float64) * x.astype(np.float64)          # exact
    want = np.empty(6, dtype=np.float32)
    for r in range(6):
        chain = np.zeros(16, dtype=np.float32)
        for t in range(n_in // 16):
            for j in range(16):                                     # fma: one rounding of a + p
                chain[j] = np.float32(np.float64(chain[j]) + prod[r, 16 * t + j])
        v = (chain[:8] + chain[8:]).astype(np.float32)
        q = (v[:4] + v[4:]).astype(np.float32)
        want[r] = np.float32(np.float32(q[0] + q[1]) + np.float32(q[2] + q[3]))
    got = oracle.f16_gemv(w16.view(np.uint16), x)
    assert (got.view(np.uint32) == want.view(np.uint32)).all()


def test_rmsnorm_closed_forms(oracle):
    n, eps = 2560, 1e-6
    w = np.ones(n, dtype=np.float32)
    x = np.full(n, 3.0, dtype=np.float32)
    inv = np.float32(1.0 / np.sqrt(9.0 + np.float64(np.float32(eps))))
    assert (oracle.rmsnorm(x, w, eps) == np.float32(3.0) * inv).all()
    g = np.random.default_rng(9)
    xs = (g.standard_normal((5, n)) * g.choice([1e-3, 1.0, 40.0], (5, 1))).astype(np.float32)
    ws = (1.0 + 0.1 * g.standard_normal(n)).astype(np.float32)
    got = oracle.rmsnorm(xs, ws, eps)
    for r in range(5):
        sumsq = 0.0
        for v in xs[r].astype(np.float64):                         # index order, in double
            sumsq += v * v
        inv = np.float32(1.0 / np.sqrt(sumsq / n + np.float64(np.float32(eps))))
        want = (xs[r] * inv).astype(np.float32) * ws
        assert (got[r].view(np.uint32) == want.astype(np.float32).view(np.uint32)).all()
    assert oracle.rmsnorm(np.zeros(n, dtype=np.float32), w, eps).tolist() == [0.0] * n


@pytest.mark.parametrize("fast", [False, True])
def test_q8w_equals_the_compiled_reference_kernels(oracle, fast):
    """f16_to_q8w and q8w_gemv_m1 of the reference (kernel_f16_gemv.c:66-127). The quantiser is
    compared with the strict build in every bit; against the release build (-ffast-math, which
    may form max|w| / 127 through a reciprocal) the scales may differ in the last bit, the int8
    values not. The GEMV is identical under both builds."""
    ref = load_ref_f16gemv(fast)
    if ref is None:
        pytest.skip("oracle/_ref not built (needs the reference tree: make -C oracle ref)")
    g = np.random.default_rng(15)
    for n_out, n_in, scale in [(64, 2560, 0.05), (33, 1536, 1.0), (9, 16, 3.0), (20, 48, 1e-3),
                               (5, 4096, 100.0)]:
        w = weights(g, n_out, n_in, scale)
        w[0, :] = 0                                  # a row of zeros: scale 0, zeros
        wq_ref = np.empty((n_out, n_in), dtype=np.int8)
        sc_ref = np.empty(n_out, dtype=np.float32)
        ref.f16_to_q8w(n_out, n_in, w.ctypes.data_as(C.POINTER(C.c_uint16)),
                       wq_ref.ctypes.data_as(C.POINTER(C.c_int8)),
                       sc_ref.ctypes.data_as(C.POINTER(C.c_float)))
        wq, sc = oracle.f16_to_q8w(w)
        assert (wq == wq_ref).all(), (n_out, n_in)
        if fast:
            assert (np.abs(sc.view(np.int32) - sc_ref.view(np.int32)) <= 1).all()
        else:
            assert (sc.view(np.uint32) == sc_ref.view(np.uint32)).all()
        x = (g.standard_normal(n_in) * g.choice([0.01, 1.0, 50.0])).astype(np.float32)
        y = np.zeros(n_out, dtype=np.float32)
        ref.q8w_gemv_m1(n_out, n_in, x.ctypes.data_as(C.POINTER(C.c_float)),
                        wq_ref.ctypes.data_as(C.POINTER(C.c_int8)),
                        sc_ref.ctypes.data_as(C.POINTER(C.c_float)),
                        y.ctypes.data_as(C.POINTER(C.c_float)))
        mine = oracle.q8w_gemv(wq_ref, sc_ref, x)
        assert (mine.view(np.uint32) == y.view(np.uint32)).all(), (n_out, n_in)


def test_q8w_keeps_the_reference_tests_bar(oracle):
    """tests/test_q8w_gemv_unit.c: cosine similarity with the exact product >= 0.999."""
    g = np.random.default_rng(16)
    n_out, n_in = 512, 2560
    w = ((g.integers(0, 65536, (n_out, n_in)) / 65536.0 * 2 - 1)).astype(np.float16).view(np.uint16)
    x = (g.integers(0, 65536, n_in) / 65536.0 * 2 - 1).astype(np.float32)
    exact = w.view(np.float16).astype(np.float64) @ x.astype(np.float64)
    wq, sc = oracle.f16_to_q8w(w)
    y = oracle.q8w_gemv(wq, sc, x).astype(np.float64)
    cos = (y @ exact) / np.sqrt((y @ y) * (exact @ exact))
    assert cos >= 0.999
    assert np.abs(wq).max() <= 127 and (np.abs(wq).max(axis=1) == 127).all()


def test_f16_linear_f64_against_numpy(oracle):
    """cpu_scalar_w_quant_mN for F16 weights (weight_resolve.c:215-241): the double sum in index
    order, rounded once. numpy's float64 dot adds in another order; the two agree wherever the
    value is not within the sums' error of a binary32 rounding boundary, which is checked, and on
    integer-valued inputs (every partial sum exact) in every bit."""
    g = np.random.default_rng(31)
    n_out, n_in, m = 700, 2560, 3
    w = (g.standard_normal((n_out, n_in)) * 0.05).astype(np.float16)
    x = (g.standard_normal((m, n_in)) * 2).astype(np.float32)
    y = oracle.f16_linear_f64(w.view(np.uint16), x)
    exact = x.astype(np.float64) @ w.astype(np.float64).T
    bound = n_in * 2.0 ** -52 * (np.abs(x).astype(np.float64) @ np.abs(w).astype(np.float64).T)
    lo, hi = (exact - bound).astype(np.float32), (exact + bound).astype(np.float32)
    sure = lo == hi
    assert sure.mean() > 0.99
    assert (y[sure] == lo[sure]).all()
    assert ((y >= lo) & (y <= hi)).all()
    wi = g.integers(-8, 9, (50, 64)).astype(np.float16)
    xi = g.integers(-100, 101, (2, 64)).astype(np.float32)
    assert (oracle.f16_linear_f64(wi.view(np.uint16), xi) == (xi @ wi.astype(np.float32).T)).all()
    # one row, one-dimensional in and out
    assert (oracle.f16_linear_f64(w.view(np.uint16), x[1]) == y[1]).all()


def _cancelling(g, n_out, n_in, m):
    q = n_in // 4
    w = (g.standard_normal((n_out, n_in)) * 4).astype(np.float16)
    x = (g.standard_normal((m, n_in)) * 100).astype(np.float32)
    x[:, :q] *= np.float32(2.0 ** 24)       # a huge first quarter ...
    w[:, 3 * q: 4 * q] = -w[:, :q]          # ... that the last quarter takes away again:
    x[:, 3 * q: 4 * q] = x[:, :q]           # the small terms in between are added to a huge sum
    return w, x


@pytest.mark.parametrize("fast", [False, True])
def test_f16_linear_f64_equals_the_compiled_reference(oracle, fast):
    """oracle_f16_linear_f64 against the reference's own cpu_scalar_w_quant_m1 / _mN over an F16
    table (weight_resolve.c:186-241), compiled from its tree with strict and with release flags:
    every bit, for one row and for batches, on random data and on rows whose last quarter cancels a huge first quarter -- there the binary32 result depends on the ORDER of the double-precision additions,
    which is what the device kernel claims to reproduce."""
    from oracle_lib import load_ref_wquant, ref_f16_linear
    ref = load_ref_wquant(fast=fast)
    if ref is None:
        pytest.skip("oracle/_ref/libgeist_ref_wquant*.so not built (needs the reference tree)")
    g = np.random.default_rng(77 + fast)
    for n_out, n_in, m in [(40, 64, 1), (33, 2560, 1), (21, 1536, 5), (17, 320, 9)]:
        for kind in ("random", "cancelling", "integers"):
            if kind == "random":
                w = (g.standard_normal((n_out, n_in)) * 0.05).astype(np.float16)
                x = (g.standard_normal((m, n_in)) * g.choice([1e-3, 1.0, 300.0])).astype(np.float32)
            elif kind == "cancelling":
                w, x = _cancelling(g, n_out, n_in, m)
            else:
                w = g.integers(-8, 9, (n_out, n_in)).astype(np.float16)
                x = g.integers(-100, 101, (m, n_in)).astype(np.float32)
            want = ref_f16_linear(ref, w.view(np.uint16), x)
            got = np.atleast_2d(oracle.f16_linear_f64(w.view(np.uint16), x if m > 1 else x[0]))
            if fast and kind == "cancelling":
                # -ffast-math lets the compiler add in another order, and on these rows it shows:
                # the release build is pinned to a few units in the last place only. It is the
                # strict build -- the order the source states -- that oracle and device reproduce.
                assert np.allclose(got, want, rtol=1e-5, atol=1e-3)
                continue
            assert (got.view(np.uint32) == want.view(np.uint32)).all(), (n_out, n_in, m, kind, fast)
    # the cancelling rows do hang on the order: numpy's pairwise float64 dot rounds some of them
    # to another binary32 value (if it never did, the case would pin nothing)
    if not fast:
        w, x = _cancelling(np.random.default_rng(5), 400, 1024, 2)
        other = (x.astype(np.float64) @ w.astype(np.float64).T).astype(np.float32)
        assert (other != ref_f16_linear(ref, w.view(np.uint16), x)).any()


def test_f16_linear_f64_golden_vectors(oracle):
    """The same against vectors written from the compiled reference
    (tests/golden/make_f16_linear_golden.py): these travel to where the reference does not."""
    import json
    import os
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                        "f16_linear_ref_vectors.json")
    with open(path) as f:
        cases = json.load(f)["cases"]
    assert len(cases) >= 5
    for c in cases:
        w = np.frombuffer(bytes.fromhex(c["w_hex"]), dtype=np.uint16).reshape(c["n_out"], c["n_in"])
        x = np.frombuffer(bytes.fromhex(c["x_hex"]), dtype=np.float32).reshape(c["m"], c["n_in"])
        want = np.frombuffer(bytes.fromhex(c["y_hex"]), dtype=np.float32).reshape(c["m"], c["n_out"])
        got = np.atleast_2d(oracle.f16_linear_f64(w, x if c["m"] > 1 else x[0]))
        assert (got.view(np.uint32) == want.view(np.uint32)).all(), c["kind"]
