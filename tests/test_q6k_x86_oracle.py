"""The x86 backend's decode kernel over a Q6_K table (oracle_q8k_quantize, oracle_q6k_gemv_x86)
pinned three ways: bit for bit against the reference's own kernel_q6k_gemv.c where it was compiled
(oracle/_ref/libgeist_ref_q6kgemv.so, strict flags; the release flags are compared too), against
golden vectors written from that build (tests/golden/q6k_x86_ref_vectors.json, which travel), and
against what the definition fixes."""
import json
import os

import numpy as np
import pytest

from oracle_lib import (load_oracle, load_ref_q6kgemv, oracle_dequant_q6k, oracle_q6k_gemv_x86,
                        oracle_q8k_quantize, random_q6k_table, ref_q6k_gemv_m1)

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def lib():
    return load_oracle()


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


@pytest.mark.parametrize("fast", [False, True])
def test_equals_the_compiled_reference(lib, fast):
    """Random tables over every bit pattern of ql / qh, the whole int8 range of the scales,
    normal / subnormal / zero / negative d; activations from 1e-30 to 1e4, with zeros and whole
    super-blocks of zeros. Every bit of every output. The lanes' integers pass 2^24 on the
    larger scales, so their conversion to binary32 rounds: a wrong lane assignment shows."""
    ref = load_ref_q6kgemv(fast=fast)
    if ref is None:
        pytest.skip("oracle/_ref/libgeist_ref_q6kgemv*.so not built (needs the reference tree)")
    g = np.random.default_rng(123 + fast)
    worst = 0
    for n_out, n_in in [(64, 256), (33, 512), (40, 1536), (17, 2560), (9, 16384)]:
        for scale in (1e-30, 1e-3, 1.0, 300.0, 1e4):
            w = random_q6k_table(g, n_out, n_in)
            x = (g.standard_normal(n_in) * scale).astype(np.float32)
            x[g.random(n_in) < 0.1] = 0.0
            if n_in >= 512:
                x[256:512] = 0.0
            want = ref_q6k_gemv_m1(ref, w, x, n_in)
            got = oracle_q6k_gemv_x86(lib, w, x, n_in)
            if fast:
                # the release build may form amax / 127 and 127 / amax by a reciprocal: where it
                # does, an activation can round to the neighbouring int8 value
                worst = max(worst, int((bits(got) != bits(want)).sum()))
                assert np.allclose(got, want, rtol=2e-2, atol=1e-30 + 1e-2 * np.abs(want).max())
            else:
                assert (bits(got) == bits(want)).all(), (n_out, n_in, scale)
    print("outputs that differ from the release build:", worst)


def test_golden_vectors(lib):
    with open(os.path.join(HERE, "golden", "q6k_x86_ref_vectors.json")) as f:
        cases = json.load(f)["cases"]
    assert len(cases) >= 6
    for c in cases:
        w = np.frombuffer(bytes.fromhex(c["w_hex"]), dtype=np.uint8).reshape(c["n_out"], -1)
        x = np.frombuffer(bytes.fromhex(c["x_hex"]), dtype=np.float32)
        want = np.frombuffer(bytes.fromhex(c["y_hex"]), dtype=np.float32)
        got = oracle_q6k_gemv_x86(lib, np.ascontiguousarray(w), x, c["n_in"])
        assert (bits(got) == bits(want)).all(), (c["n_out"], c["n_in"])


def test_activation_quantiser_by_definition(lib):
    g = np.random.default_rng(9)
    x = (g.standard_normal(512) * 3).astype(np.float32)
    x[256:] = 0.0
    x[5] = np.float32(-7.5)                      # the largest magnitude of the first super-block
    x[:256] = np.clip(x[:256], -7.5, 7.5)
    d, qs, bs = oracle_q8k_quantize(lib, x)
    assert d[0] == np.float32(7.5) / np.float32(127.0) and d[1] == 0.0
    assert qs[5] == -127 and np.abs(qs[:256]).max() == 127 and not qs[256:].any()
    assert np.array_equal(bs, qs.astype(np.int32).reshape(-1, 16).sum(axis=1).astype(np.int16))
    idf = np.float32(127.0) / np.float32(7.5)
    assert np.array_equal(qs[:256], np.rint(x[:256] * idf).astype(np.int8))   # rint: ties to even


def test_close_to_the_exact_product(lib):
    """What the arithmetic is for: the int8 activations cost about 1 % of the row's scale."""
    g = np.random.default_rng(10)
    n_out, n_in = 50, 1536
    w = random_q6k_table(g, n_out, n_in, scale_mode="plain")
    x = g.standard_normal(n_in).astype(np.float32)
    exact = oracle_dequant_q6k(lib, w, n_in).astype(np.float64) @ x.astype(np.float64)
    got = oracle_q6k_gemv_x86(lib, w, x, n_in).astype(np.float64)
    cos = (got @ exact) / np.sqrt((got @ got) * (exact @ exact))
    assert cos > 0.9995
