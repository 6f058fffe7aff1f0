"""The x86 backend's decode kernel over a Q6_K table (oracle_q8k_quantize, oracle_q6k_gemv_x86)
pinned three ways: bit for bit against the reference's own kernel_q6k_gemv.c where it was compiled
(oracle/_ref/libgeist_ref_q6kgemv.so, strict flags; the release flags are compared too), against
golden vectors written from that build (tests/golden/q6k_x86_ref_vectors.json, which travel), and
against what the definition fixes."""
import json
import os

import numpy as np
import pytest

from oracle_lib import (load_oracle, load_ref_q6kgemv, load_ref_q6kmn, oracle_dequant_q6k,
                        oracle_q6k_gemv_x86, oracle_q6k_linear_x86, oracle_q8_sym_row_quantize,
                        oracle_q8k_quantize, random_q6k_table, ref_q6k_gemv_m1, ref_q6k_linear_mN)

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


def tie_rows(g, m, n_in, scale):
    """Rows whose scale is a power of two, with activations exactly between two int8 values."""
    x = (g.standard_normal((m, n_in)) * scale).astype(np.float32)
    x[:, ::7] = 0.0
    d = np.float32(2.0) ** np.ceil(np.log2(scale) - 3)
    x[:, 0] = np.float32(127.0) * d
    for k, h in enumerate((0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 63.5, -126.5)):
        x[:, 1 + k] = np.float32(h) * d
    return x


def test_batch_path_equals_the_compiled_reference(lib):
    """cpu_x86_linear_q6k_resolve + cpu_x86_linear_q6k_mN as the reference calls them
    (q6k_to_w8a8_row, the interleaving, w4a8_quantize_acts_row, w8a8_gemm / w8x8_gemm /
    w8x16_gemm) against oracle_q6k_linear_x86, bit for bit: on a VNNI host the lane kernels for
    tables of a multiple of 8 rows and the VNNI kernel with the scalar expression for others; on
    other hosts (or under GEIST_FORCE_ISA) the scalar kernel."""
    ref = load_ref_q6kmn()
    if ref is None:
        pytest.skip("built only where the reference tree is mounted (make -C oracle ref)")
    vnni = bool(ref.w8a8_isa_is_vnni())
    g = np.random.default_rng(66)
    differ = 0
    for n_out, n_in, m in [(64, 512, 2), (64, 512, 3), (48, 768, 8), (40, 1024, 4), (20, 512, 5),
                           (128, 2560, 16), (8, 256, 2), (12, 256, 3), (16, 16384, 2)]:
        w = random_q6k_table(g, n_out, n_in)
        for scale in (1e-3, 1.0, 100.0):
            x = tie_rows(g, m, n_in, scale)
            want, lanes = ref_q6k_linear_mN(ref, w, x, n_in)
            assert lanes == (vnni and n_out % 8 == 0)
            got = oracle_q6k_linear_x86(lib, w, x, n_in, vnni=vnni)
            assert np.array_equal(bits(got), bits(want)), (n_out, n_in, m, scale)
            if n_out % 8 == 0:       # the two hosts' arithmetics are not the same function
                other = oracle_q6k_linear_x86(lib, w, x, n_in, vnni=not vnni)
                differ += int((bits(other) != bits(got)).sum())
    assert differ > 0


def test_batch_quantiser_by_definition(lib):
    g = np.random.default_rng(9)
    x = tie_rows(g, 1, 768, 2.5)[0]
    d, q, sm = oracle_q8_sym_row_quantize(lib, x)
    assert np.float32(d) == np.float32(np.abs(x).max()) / np.float32(127.0) == np.float32(0.5)
    v = (x * (np.float32(1.0) / np.float32(d))).astype(np.float32)
    assert np.array_equal(q, np.rint(v).astype(np.int8))                 # lrintf: ties to even
    assert list(q[1:9]) == [0, 2, 2, 0, -2, -2, 64, -126]
    assert np.array_equal(sm, q.reshape(-1, 16).astype(np.int32).sum(1))
    d0, q0, _ = oracle_q8_sym_row_quantize(lib, np.zeros(256, dtype=np.float32))
    assert d0 == 1.0 and not q0.any()                                    # a row of zeros: scale 1


def test_batch_against_the_dequantised_table(lib):
    """With activations that are whole multiples of the row's scale the int8 values are exact and
    both arithmetics give the dot product with the dequantised table up to their few roundings."""
    g = np.random.default_rng(15)
    n_out, n_in = 16, 512
    w = random_q6k_table(g, n_out, n_in, scale_mode="plain")
    q = g.integers(-127, 128, (2, n_in))
    q[:, 0] = 127
    x = (q * np.float32(0.5)).astype(np.float32)
    deq = oracle_dequant_q6k(lib, w, n_in).astype(np.float64)
    want = x.astype(np.float64) @ deq.T
    mag = np.abs(x).astype(np.float64) @ np.abs(deq).T
    for vnni in (True, False):
        y = oracle_q6k_linear_x86(lib, w, x, n_in, vnni=vnni)
        assert (np.abs(y - want) <= 1e-4 * mag + 1e-30).all(), vnni


def test_golden_batches(lib):
    with open(os.path.join(HERE, "golden", "q6k_x86_ref_vectors.json")) as f:
        cases = json.load(f)["batch_cases"]
    assert len(cases) >= 5 and any(c["lanes"] for c in cases) and not all(c["lanes"] for c in cases)
    for c in cases:
        n_out, n_in, m = c["n_out"], c["n_in"], c["m"]
        w = np.frombuffer(bytes.fromhex(c["w_hex"]), dtype=np.uint8).reshape(n_out, -1).copy()
        x = np.frombuffer(bytes.fromhex(c["x_hex"]), dtype=np.float32).reshape(m, n_in).copy()
        y = np.frombuffer(bytes.fromhex(c["y_hex"]), dtype=np.float32).reshape(m, n_out)
        got = oracle_q6k_linear_x86(lib, w, x, n_in, vnni=True)       # written on a VNNI host
        assert np.array_equal(bits(got), bits(y)), (n_out, n_in, m)
