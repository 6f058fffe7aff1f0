"""The Q6_K part of the oracle (oracle_dequant_q6_K_row, oracle_q6k_linear_f64) pinned three ways:
bit for bit against the reference's own q6_K.c and weight_resolve.c where they were compiled
(oracle/_ref/libgeist_ref_wquant.so, strict and release flags), against golden vectors written
from that build (tests/golden/q6k_ref_vectors.json, which travel), and against blocks whose
values follow from the format's definition alone."""
import json
import os

import numpy as np
import pytest

from oracle_lib import (load_oracle, load_ref_wquant, oracle_dequant_q6k, oracle_q6k_linear,
                        random_q6k_table, ref_q6k_linear, _fp)
import ctypes as C

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def lib():
    return load_oracle()


def block(ql=0, qh=0, scales=1, d=1.0):
    b = np.zeros(210, dtype=np.uint8)
    b[:128] = ql
    b[128:192] = qh
    b[192:208] = np.asarray(scales, dtype=np.int8).view(np.uint8)
    b[208:210] = np.frombuffer(np.float16(d).tobytes(), dtype=np.uint8)
    return b.reshape(1, 210)


def test_blocks_whose_values_follow_from_the_definition(lib):
    # q = 32 everywhere (low nibbles 0, high bits 10b): every element is d * sc * 0
    assert not oracle_dequant_q6k(lib, block(ql=0x00, qh=0xAA, scales=7, d=0.5), 256).any()
    # q = 0 everywhere: -32 * d * sc, with the sixteen scales 1..16 over the groups of 16 elements
    # in the order (half, quarter, l / 16): element 128 h + 32 j + l has scale index 8 h + 2 j + l / 16
    y = oracle_dequant_q6k(lib, block(ql=0x00, qh=0x00, scales=np.arange(1, 17), d=2.0), 256)[0]
    want = np.repeat(-64.0 * np.arange(1, 17, dtype=np.float32), 16)
    assert np.array_equal(y, want)
    # low nibble 5, high nibble 9, high bits 0: quarters 0 and 1 take the low nibble (q = 5),
    # quarters 2 and 3 the high one (q = 9)
    y = oracle_dequant_q6k(lib, block(ql=0x95, qh=0x00, scales=1, d=1.0), 256)[0].reshape(2, 4, 32)
    assert np.all(y[:, :2] == 5 - 32) and np.all(y[:, 2:] == 9 - 32)
    # qh = 0b11100100: quarter j takes the bits 2 j, 2 j + 1, i.e. the values 0, 1, 2, 3
    y = oracle_dequant_q6k(lib, block(ql=0x00, qh=0xE4, scales=1, d=1.0), 256)[0].reshape(2, 4, 32)
    for j in range(4):
        assert np.all(y[:, j] == 16 * j - 32)
    # ql[l] and ql[l + 32] feed different quarters; qh[l] is shared by the four quarters at l
    b = block(ql=0, qh=0, scales=1, d=1.0)
    b[0, 3] = 0x21           # ql[3]:  quarter 0 gets 1, quarter 2 gets 2   (first half)
    b[0, 32 + 3] = 0x43      # ql[35]: quarter 1 gets 3, quarter 3 gets 4
    b[0, 128 + 3] = 0x1B     # qh[3] = 00 01 10 11b: quarters 0..3 get high bits 3, 2, 1, 0
    y = oracle_dequant_q6k(lib, b, 256)[0]
    assert [int(y[32 * j + 3]) + 32 for j in range(4)] == [1 + 48, 3 + 32, 2 + 16, 4 + 0]
    # a projection that is exact in binary32: integers
    w = block(ql=0x11, qh=0x00, scales=1, d=1.0)             # every element 1 - 32 = -31
    x = np.ones((1, 256), dtype=np.float32)
    assert oracle_q6k_linear(lib, w, x, 256)[0, 0] == -31.0 * 256


@pytest.mark.parametrize("fast", [False, True])
def test_dequant_and_projection_equal_the_compiled_reference(lib, fast):
    ref = load_ref_wquant(fast)
    if ref is None:
        pytest.skip("built only where the reference tree is mounted (make -C oracle ref)")
    g = np.random.default_rng(11 + fast)
    for n_out, n_in, m in [(64, 256, 1), (33, 1024, 1), (17, 1536, 4), (6, 2560, 2)]:
        w = random_q6k_table(g, n_out, n_in)
        got = oracle_dequant_q6k(lib, w, n_in)
        want = np.empty_like(got)
        for j in range(n_out):
            ref.dequant_q6_K_row(w[j].ctypes.data_as(C.c_void_p), _fp(want[j]), n_in)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (n_out, n_in)
        for scale in (1e-3, 1.0, 100.0):
            x = (g.standard_normal((m, n_in)) * scale).astype(np.float32)
            a = oracle_q6k_linear(lib, w, x, n_in)
            b = ref_q6k_linear(ref, w, x, n_in)
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), (n_out, n_in, m, scale)


def test_golden_vectors_of_the_reference(lib):
    with open(os.path.join(HERE, "golden", "q6k_ref_vectors.json")) as f:
        cases = json.load(f)["cases"]
    assert len(cases) >= 4
    for c in cases:
        n_out, n_in, m = c["n_out"], c["n_in"], c["m"]
        w = np.frombuffer(bytes.fromhex(c["w_hex"]), dtype=np.uint8).reshape(n_out, -1).copy()
        x = np.frombuffer(bytes.fromhex(c["x_hex"]), dtype=np.float32).reshape(m, n_in).copy()
        y = np.frombuffer(bytes.fromhex(c["y_hex"]), dtype=np.float32).reshape(m, n_out)
        r0 = np.frombuffer(bytes.fromhex(c["dequant_row0_hex"]), dtype=np.float32)
        assert np.array_equal(oracle_dequant_q6k(lib, w[:1], n_in)[0].view(np.uint32),
                              r0.view(np.uint32))
        got = oracle_q6k_linear(lib, w, x, n_in)
        # a NaN's sign and payload are not part of the result
        assert np.array_equal(np.isnan(got), np.isnan(y))
        assert np.array_equal(got.view(np.uint32)[~np.isnan(y)], y.view(np.uint32)[~np.isnan(y)])
    assert any(c.get("not_finite") for c in cases)
