"""The Q4_K part of the oracle (oracle_dequant_q4_K_row, oracle_q4k_linear_f64) pinned three ways:
bit for bit against the reference's own q4_K.c and weight_resolve.c where they were compiled
(oracle/_ref/libgeist_ref_wquant.so, strict and release flags), against golden vectors written
from that build (tests/golden/q4k_ref_vectors.json, which travel), and against blocks whose
values follow from the format's definition alone."""
import ctypes as C
import json
import os

import numpy as np
import pytest

from oracle_lib import (load_oracle, load_ref_wquant, oracle_dequant_q4k, oracle_q4k_linear,
                        random_q4k_table, ref_q4k_linear, _fp)

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def lib():
    return load_oracle()


def block(d=1.0, dmin=0.0, scales=None, qs=0):
    b = np.zeros(144, dtype=np.uint8)
    b[0:2] = np.frombuffer(np.float16(d).tobytes(), dtype=np.uint8)
    b[2:4] = np.frombuffer(np.float16(dmin).tobytes(), dtype=np.uint8)
    if scales is not None:
        b[4:16] = scales
    b[16:] = qs
    return b.reshape(1, 144)


def pack_scales(sc, mn):
    """The 12 bytes that hold eight 6-bit scales and eight 6-bit minima: bytes 0..3 the low six
    bits of scales 0..3 (their top two bits: bits 4, 5 of scales 4..7), bytes 4..7 the same for
    the minima, bytes 8..11 the low nibbles of scale 4 + i (low half) and minimum 4 + i (high)."""
    q = np.zeros(12, dtype=np.uint8)
    for j in range(4):
        q[j] = (sc[j] & 63) | ((sc[j + 4] >> 4) << 6)
        q[j + 4] = (mn[j] & 63) | ((mn[j + 4] >> 4) << 6)
        q[j + 8] = (sc[j + 4] & 0xF) | ((mn[j + 4] & 0xF) << 4)
    return q


def test_blocks_whose_values_follow_from_the_definition(lib):
    sc = np.array([1, 2, 3, 4, 33, 47, 63, 16])
    mn = np.array([0, 5, 6, 7, 62, 17, 32, 1])
    # every value 3: element of sub-block j is d * sc[j] * 3 - dmin * mn[j]
    y = oracle_dequant_q4k(lib, block(d=0.5, dmin=0.25, scales=pack_scales(sc, mn), qs=0x33), 256)[0]
    want = np.repeat(0.5 * sc * 3 - 0.25 * mn, 32).astype(np.float32)
    assert np.array_equal(y, want)
    # low nibble 5, high nibble 9: sub-blocks 0, 2, 4, 6 take the low nibbles of the 32 bytes
    # of their pair, sub-blocks 1, 3, 5, 7 the high ones
    y = oracle_dequant_q4k(lib, block(d=1.0, scales=pack_scales(np.ones(8, int), np.zeros(8, int)),
                                      qs=0x95), 256)[0].reshape(4, 2, 32)
    assert np.all(y[:, 0] == 5) and np.all(y[:, 1] == 9)
    # byte l of pair s feeds elements 64 s + l (low) and 64 s + 32 + l (high)
    b = block(d=1.0, scales=pack_scales(np.ones(8, int), np.zeros(8, int)), qs=0)
    b[0, 16 + 32 * 2 + 7] = 0xC4
    y = oracle_dequant_q4k(lib, b, 256)[0]
    assert y[64 * 2 + 7] == 4 and y[64 * 2 + 32 + 7] == 12 and y.sum() == 16
    # a subtraction that rounds: d * sc * q = 15 * 2^-14 * 63, dmin * m = 1000 * 63
    y = oracle_dequant_q4k(lib, block(d=2.0 ** -14, dmin=1000.0,
                                      scales=pack_scales(np.full(8, 63), np.full(8, 63)), qs=0xFF),
                           256)[0]
    assert np.all(y == np.float32(np.float32(2.0 ** -14 * 63 * 15) - np.float32(63000.0)))
    # a projection that is exact in binary32: integers
    w = block(d=1.0, dmin=1.0, scales=pack_scales(np.full(8, 2), np.full(8, 3)), qs=0x77)
    x = np.ones((1, 256), dtype=np.float32)                # every element 2 * 7 - 3 = 11
    assert oracle_q4k_linear(lib, w, x, 256)[0, 0] == 11.0 * 256


@pytest.mark.parametrize("fast", [False, True])
def test_dequant_and_projection_equal_the_compiled_reference(lib, fast):
    ref = load_ref_wquant(fast)
    if ref is None:
        pytest.skip("built only where the reference tree is mounted (make -C oracle ref)")
    g = np.random.default_rng(21 + fast)
    for n_out, n_in, m in [(64, 256, 1), (33, 1024, 1), (17, 1536, 4), (6, 2560, 2)]:
        w = random_q4k_table(g, n_out, n_in)
        got = oracle_dequant_q4k(lib, w, n_in)
        want = np.empty_like(got)
        for j in range(n_out):
            ref.dequant_q4_K_row(w[j].ctypes.data_as(C.c_void_p), _fp(want[j]), n_in)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (n_out, n_in)
        for scale in (1e-3, 1.0, 100.0):
            x = (g.standard_normal((m, n_in)) * scale).astype(np.float32)
            a = oracle_q4k_linear(lib, w, x, n_in)
            b = ref_q4k_linear(ref, w, x, n_in)
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), (n_out, n_in, m, scale)


def test_golden_vectors_of_the_reference(lib):
    with open(os.path.join(HERE, "golden", "q4k_ref_vectors.json")) as f:
        cases = json.load(f)["cases"]
    assert len(cases) >= 4
    for c in cases:
        n_out, n_in, m = c["n_out"], c["n_in"], c["m"]
        w = np.frombuffer(bytes.fromhex(c["w_hex"]), dtype=np.uint8).reshape(n_out, -1).copy()
        x = np.frombuffer(bytes.fromhex(c["x_hex"]), dtype=np.float32).reshape(m, n_in).copy()
        y = np.frombuffer(bytes.fromhex(c["y_hex"]), dtype=np.float32).reshape(m, n_out)
        r0 = np.frombuffer(bytes.fromhex(c["dequant_row0_hex"]), dtype=np.float32)
        assert np.array_equal(oracle_dequant_q4k(lib, w[:1], n_in)[0].view(np.uint32),
                              r0.view(np.uint32))
        assert np.array_equal(oracle_q4k_linear(lib, w, x, n_in).view(np.uint32), y.view(np.uint32))
