"""The oracle's restatement of the x86 backend's Q4_K decode kernel (oracle_q4k_gemv_x86) against
the reference's own q4k_to_q4kx8_matrix + q4kx8_gemv_m1, compiled from its tree
(oracle/_ref/libgeist_ref_q4kgemv.so: kernel_q4kx8_gemm_avx512.c, kernel_q4kx8_gemm_scalar.c,
q4k_to_q4kx8.c), bit for bit with strict flags; the batch path (oracle_q4k_linear_x86) against
quantize_q8_Kx4 + q4kx8_gemm_avx512 of the same build; against golden vectors written from that
build; and against what the definition fixes."""
import json
import os

import numpy as np
import pytest

from oracle_lib import (load_oracle, load_ref_q4kgemv, oracle_dequant_q4k, oracle_q4k_gemv_x86,
                        oracle_q4k_linear_x86, oracle_q8k_row_quantize, oracle_q8kx4_row_quantize,
                        random_q4k_table, ref_q4k_gemv_m1, ref_q4k_linear_mN)

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def lib():
    return load_oracle()


def activations(g, n_in, scale):
    x = (g.standard_normal(n_in) * scale).astype(np.float32)
    x[::7] = 0.0
    return x


@pytest.mark.parametrize("fast", [False, True])
def test_decode_kernel_equals_the_compiled_reference(lib, fast):
    ref = load_ref_q4kgemv(fast)
    if ref is None:
        pytest.skip("built only where the reference tree is mounted (make -C oracle ref)")
    g = np.random.default_rng(21 + fast)
    worst = 0
    for n_out, n_in in [(8, 256), (64, 512), (40, 1536), (1024, 2560), (16, 16384)]:
        w = random_q4k_table(g, n_out, n_in)
        for scale in (1e-4, 0.02, 1.0, 37.0, 3e4):
            x = activations(g, n_in, scale)
            if scale == 1.0:
                x[5] = np.float32(1e6)            # one huge activation: the others round to zero
            a = oracle_q4k_gemv_x86(lib, w, x, n_in)
            b = ref_q4k_gemv_m1(ref, w, x, n_in)
            if not fast:
                assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), (n_out, n_in, scale)
            else:
                # the release build forms amax / 127 and 1 / scale by reciprocals: an activation on
                # a rounding edge may land on the neighbouring int8
                worst += int((a.view(np.uint32) != b.view(np.uint32)).sum())
                ok = np.isclose(a, b, rtol=2e-2, atol=2e-2 * float(np.abs(b).max() + 1e-30))
                assert ok.all(), (n_out, n_in, scale)
        x0 = np.zeros(n_in, dtype=np.float32)     # a row of zeros: scale 1, every product 0
        assert not oracle_q4k_gemv_x86(lib, w, x0, n_in).any()
        assert not ref_q4k_gemv_m1(ref, w, x0, n_in).any()
    print("outputs that differ from the release build:", worst)


def test_quantiser_against_the_definition(lib):
    g = np.random.default_rng(3)
    x = activations(g, 768, 2.5)
    d, qs, bs = oracle_q8k_row_quantize(lib, x)
    amax = np.abs(x).max()
    assert np.float32(d) == np.float32(amax) / np.float32(127.0)
    v = x * (np.float32(1.0) / np.float32(d))
    want = np.where(v < 0, v - np.float32(0.5), v + np.float32(0.5)).astype(np.float32)
    want = np.clip(np.trunc(want), -128, 127).astype(np.int8)
    assert np.array_equal(qs, want)
    assert np.array_equal(bs, qs.reshape(-1, 16).astype(np.int32).sum(1).astype(np.int16))
    assert np.abs(qs).max() == 127


def test_against_the_dequantised_table(lib):
    """With activations that are whole multiples of the row's scale the int8 values are exact,
    and the kernel's result is the dot product with the dequantised table up to the rounding of
    its few binary32 steps."""
    g = np.random.default_rng(5)
    n_out, n_in = 16, 512
    w = random_q4k_table(g, n_out, n_in)
    q = g.integers(-127, 128, n_in)
    q[0] = 127
    x = (q * np.float32(0.5)).astype(np.float32)          # scale 63.5 / 127 = 0.5 exactly
    y = oracle_q4k_gemv_x86(lib, w, x, n_in)
    deq = oracle_dequant_q4k(lib, w, n_in).astype(np.float64)
    want = deq @ x.astype(np.float64)
    mag = np.abs(deq) @ np.abs(x).astype(np.float64)
    assert (np.abs(y - want) <= 1e-4 * mag + 1e-30).all()


def test_golden_vectors_of_the_reference(lib):
    with open(os.path.join(HERE, "golden", "q4k_x86_ref_vectors.json")) as f:
        cases = json.load(f)["cases"]
    assert len(cases) >= 4
    for c in cases:
        n_out, n_in = c["n_out"], c["n_in"]
        w = np.frombuffer(bytes.fromhex(c["w_hex"]), dtype=np.uint8).reshape(n_out, -1).copy()
        x = np.frombuffer(bytes.fromhex(c["x_hex"]), dtype=np.float32).copy()
        y = np.frombuffer(bytes.fromhex(c["y_hex"]), dtype=np.float32)
        assert np.array_equal(oracle_q4k_gemv_x86(lib, w, x, n_in).view(np.uint32), y.view(np.uint32))


def host_has_avx512():
    try:
        flags = open("/proc/cpuinfo").read()
    except OSError:
        return False
    return all(f in flags for f in ("avx512f", "avx512bw", "avx512dq", "avx512vl"))


def tie_rows(g, m, n_in, scale):
    """Rows with activations exactly between two int8 values, where the decode kernel's quantiser
    (half away from zero) and the batch quantiser (lrintf) part ways."""
    x = (g.standard_normal((m, n_in)) * scale).astype(np.float32)
    x[:, ::7] = 0.0
    d = np.float32(2.0) ** np.ceil(np.log2(scale) - 3)   # the row's scale: a power of two,
    x[:, 0] = np.float32(127.0) * d                      # so that the ties are exact
    for k, h in enumerate((0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 63.5, -126.5)):
        x[:, 1 + k] = np.float32(h) * d
    return x


def test_batch_kernel_equals_the_compiled_reference(lib):
    """cpu_x86_linear_q4k_mN's calls (quantize_q8_Kx4, q4kx8_gemm_avx512; the decode kernel row by
    row for row counts that are no multiple of 4) against oracle_q4k_linear_x86, bit for bit. On
    a host with AVX-512 the reference takes its 16 x 16 tiles where both counts are multiples of
    16; elsewhere, and on other hosts, the AVX2 kernel."""
    ref = load_ref_q4kgemv(False)
    if ref is None:
        pytest.skip("built only where the reference tree is mounted (make -C oracle ref)")
    if os.environ.get("GEIST_FORCE_ISA"):
        pytest.skip("GEIST_FORCE_ISA changes which of the reference's kernels runs")
    avx512 = host_has_avx512()
    g = np.random.default_rng(77)
    for n_out, n_in, m in [(64, 512, 2), (64, 512, 3), (64, 512, 4), (48, 768, 8), (64, 256, 12),
                           (64, 1024, 16), (72, 512, 16), (128, 512, 32), (64, 256, 20),
                           (32, 16384, 4)]:
        w = random_q4k_table(g, n_out, n_in)
        for scale in (1e-3, 1.0, 100.0):
            x = tie_rows(g, m, n_in, scale)
            a = oracle_q4k_linear_x86(lib, w, x, n_in, avx512=avx512)
            b = ref_q4k_linear_mN(ref, w, x, n_in)
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), (n_out, n_in, m, scale)
            if m % 16 == 0 and n_out % 16 == 0:          # the two hosts give different bits
                c = oracle_q4k_linear_x86(lib, w, x, n_in, avx512=not avx512)
                assert not np.array_equal(a.view(np.uint32), c.view(np.uint32))


def test_batch_quantiser_against_the_definition(lib):
    g = np.random.default_rng(8)
    x = tie_rows(g, 1, 768, 2.5)[0]
    d, qs, bs = oracle_q8kx4_row_quantize(lib, x)
    d1, qs1, _ = oracle_q8k_row_quantize(lib, x)
    assert np.float32(d) == np.float32(np.abs(x).max()) / np.float32(127.0) == np.float32(d1)
    assert np.float32(d) == np.float32(0.5)
    v = (x * (np.float32(1.0) / np.float32(d))).astype(np.float32)
    assert np.array_equal(qs, np.rint(v).astype(np.int8))           # ties to even
    assert np.array_equal(bs, qs.reshape(-1, 16).astype(np.int32).sum(1).astype(np.int16))
    # the ties: 0.5 -> 0 here and 1 in the decode kernel, 2.5 -> 2 and 3, 1.5 -> 2 in both
    assert list(qs[1:9]) == [0, 2, 2, 0, -2, -2, 64, -126]
    assert list(qs1[1:9]) == [1, 2, 3, -1, -2, -3, 64, -127]


def test_golden_batches_of_the_reference(lib):
    with open(os.path.join(HERE, "golden", "q4k_x86_ref_vectors.json")) as f:
        cases = json.load(f)["batch_cases"]
    assert len(cases) >= 6 and any(c["tiles"] for c in cases)
    for c in cases:
        n_out, n_in, m = c["n_out"], c["n_in"], c["m"]
        w = np.frombuffer(bytes.fromhex(c["w_hex"]), dtype=np.uint8).reshape(n_out, -1).copy()
        x = np.frombuffer(bytes.fromhex(c["x_hex"]), dtype=np.float32).reshape(m, n_in).copy()
        y = np.frombuffer(bytes.fromhex(c["y_hex"]), dtype=np.float32).reshape(m, n_out)
        got = oracle_q4k_linear_x86(lib, w, x, n_in, avx512=True)   # written on an AVX-512 host
        assert np.array_equal(got.view(np.uint32), y.view(np.uint32)), (n_out, n_in, m)


def test_shapes_the_kernel_does_not_take(lib):
    import ctypes as C
    lib.oracle_q4k_gemv_x86.restype = C.c_int
    g = np.random.default_rng(1)
    w = random_q4k_table(g, 12, 256)                      # 12 rows: not a multiple of 8
    y = np.zeros(12, dtype=np.float32)
    x = np.zeros(256, dtype=np.float32)
    rc = lib.oracle_q4k_gemv_x86(12, 256, x.ctypes.data_as(C.POINTER(C.c_float)),
                                 w.ctypes.data_as(C.c_void_p), y.ctypes.data_as(C.POINTER(C.c_float)))
    assert rc == -1
