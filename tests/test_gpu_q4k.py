"""The lm_head over a Q4_K table on the GPU against the oracle, which is pinned to the reference's
own q4_K.c and weight_resolve.c (tests/test_q4k_oracle.py): logits bit for bit, for one activation
row and for batches, and token ids through the head with a soft-cap."""
import ctypes as C

import numpy as np
import pytest

from oracle_lib import (oracle_q4k_gemv_x86, oracle_q4k_linear, oracle_q4k_linear_x86,
                        oracle_q8k_row_quantize, random_q4k_table)
from test_gpu_host_layer import SessionOpts, host, make_head  # noqa: F401 (fixture)

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def hs():
    from geistlib_amd import HipSampler
    s = HipSampler(max_rows=16, max_vocab=262144)
    yield s
    s.close()


def packed_copy(hs, w, n_in):
    d_w = torch.from_numpy(w).cuda()
    packed = torch.full((hs.q4k_packed_bytes(w.shape[0], n_in),), 0xA5, dtype=torch.uint8,
                        device="cuda")
    hs.q4k_pack(d_w, n_in, packed)
    return packed


@pytest.mark.parametrize("n_out,n_in,m", [(1, 256, 1), (64, 256, 1), (300, 512, 1), (1000, 768, 3),
                                          (5000, 1536, 1), (4097, 1536, 5), (2000, 2560, 9),
                                          (70000, 1024, 2)])
def test_q4k_linear_equals_the_portable_kernel(hs, oracle, n_out, n_in, m):
    print(f"q4k linear {n_out} x {n_in}, {m} rows", flush=True)
    g = np.random.default_rng(n_out + n_in + m)
    w = random_q4k_table(g, n_out, n_in)
    packed = packed_copy(hs, w, n_in)
    for scale in (1.0, 1e-4, 300.0):
        x = (g.standard_normal((m, n_in)) * scale).astype(np.float32)
        x[0, ::5] = 0.0
        want = oracle_q4k_linear(oracle.lib, w, x, n_in)
        d_x = torch.from_numpy(x).cuda()
        y = torch.full((m, n_out), np.nan, dtype=torch.float32, device="cuda")
        hs.q4k_packed_linear(packed, n_out, n_in, d_x, y)
        hs.sync()
        got = y.cpu().numpy()
        bad = np.argwhere(got.view(np.uint32) != want.view(np.uint32))
        assert bad.size == 0, (scale, bad[:5], got[tuple(bad[0])], want[tuple(bad[0])])


@pytest.mark.parametrize("n_out,n_in", [(8, 256), (64, 256), (304, 512), (5000, 1536),
                                        (4104, 2560), (70000, 1024), (72, 16384)])
def test_q4k_decode_equals_the_x86_kernel(hs, oracle, n_out, n_in):
    """The x86 backend's integer decode kernel (q4kx8_gemv_m1 over the table its repacker
    interleaves), to which the oracle is pinned by the compiled reference
    (tests/test_q4k_x86_oracle.py): logits bit for bit, row by row."""
    print(f"q4k x86 decode {n_out} x {n_in}", flush=True)
    g = np.random.default_rng(n_out + n_in)
    w = random_q4k_table(g, n_out, n_in)
    packed = packed_copy(hs, w, n_in)
    for scale in (1.0, 1e-4, 300.0, 0.0):
        x = (g.standard_normal((3, n_in)) * scale).astype(np.float32)
        x[0, ::5] = 0.0
        x[2, 7] = np.float32(1e30)            # one huge activation: the others round to zero
        d_x = torch.from_numpy(x).cuda()
        y = torch.full((3, n_out), np.nan, dtype=torch.float32, device="cuda")
        hs.q4k_packed_gemv_x86(packed, n_out, n_in, d_x, y)
        hs.sync()
        got = y.cpu().numpy()
        for m in range(3):
            want = oracle_q4k_gemv_x86(oracle.lib, w, x[m], n_in)
            bad = np.flatnonzero(got[m].view(np.uint32) != want.view(np.uint32))
            assert bad.size == 0, (scale, m, bad[:5], got[m][bad[:3]], want[bad[:3]])
        # the kernel's two halves: the int8 activations as the reference's quantiser leaves them
        # (per eight elements the even ones, then the odd ones), and the dot products over them
        nb = n_in // 256
        act = torch.full((hs.q8k_row_act_bytes(n_in) // 4,), -1, dtype=torch.int32, device="cuda")
        hs.q8k_row_quantize(d_x[1], act)
        y1 = torch.full((n_out,), np.nan, dtype=torch.float32, device="cuda")
        hs.q4k_packed_gemv_q8k(packed, n_out, n_in, act, y1)
        hs.sync()
        a = act.cpu().numpy()
        d, qs, bs = oracle_q8k_row_quantize(oracle.lib, x[1])
        blocks = a[:nb * 72].reshape(nb, 72)
        q = blocks[:, :64].copy().view(np.int8).reshape(nb, 32, 2, 4)    # [block, eight, parity, i]
        assert (q.transpose(0, 1, 3, 2).reshape(-1) == qs).all(), scale
        assert (blocks[:, 64:].reshape(-1) ==
                bs.astype(np.int32).reshape(-1, 2).sum(axis=1)).all(), scale
        assert a[nb * 72:].view(np.float32)[0] == np.float32(d), scale
        assert (y1.cpu().numpy().view(np.uint32) == got[1].view(np.uint32)).all(), scale


def tie_rows(g, m, n_in, scale):
    """Rows whose scale is a power of two, with activations exactly between two int8 values: there
    the decode kernel's quantiser (half away from zero) and the batch quantiser (lrintf) differ."""
    x = (g.standard_normal((m, n_in)) * scale).astype(np.float32)
    x[:, ::7] = 0.0
    d = np.float32(2.0) ** np.ceil(np.log2(scale) - 3)
    x[:, 0] = np.float32(127.0) * d
    for k, h in enumerate((0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 63.5, -126.5)):
        x[:, 1 + k] = np.float32(h) * d
    return x


@pytest.mark.parametrize("n_out,n_in,m", [(64, 512, 2), (64, 512, 3), (5000, 1536, 4), (304, 512, 5),
                                          (4104, 2560, 8), (64, 256, 12), (4112, 1024, 16),
                                          (4104, 1024, 16), (128, 512, 32), (72, 16384, 4),
                                          (70000, 1024, 7)])
def test_q4k_batch_equals_the_x86_backend(hs, oracle, n_out, n_in, m):
    """cpu_x86_linear_q4k_mN over the packed copy, to which the oracle is pinned by the compiled
    reference (tests/test_q4k_x86_oracle.py): row counts that are no multiple of 4 (the decode
    kernel row by row), multiples of 4 (the batch quantiser), multiples of 16 over 16 n table rows
    (the AVX-512 tiles' order of accumulation, and the AVX2 kernel's in projection mode
    X86_AVX2), with activations on the quantisers' ties. Logits bit for bit."""
    print(f"q4k x86 batch {n_out} x {n_in}, {m} rows", flush=True)
    g = np.random.default_rng(n_out + n_in + m)
    w = random_q4k_table(g, n_out, n_in)
    packed = packed_copy(hs, w, n_in)
    try:
        for scale in (1.0, 1e-3, 100.0):
            x = tie_rows(g, m, n_in, scale)
            d_x = torch.from_numpy(x).cuda()
            for mode, avx512 in ((0, True), (2, False)):
                hs.set_projection(mode)
                y = torch.full((m, n_out), np.nan, dtype=torch.float32, device="cuda")
                hs.q4k_packed_linear_x86(packed, n_out, n_in, d_x, y)
                hs.sync()
                got = y.cpu().numpy()
                want = oracle_q4k_linear_x86(oracle.lib, w, x, n_in, avx512=avx512)
                bad = np.argwhere(got.view(np.uint32) != want.view(np.uint32))
                assert bad.size == 0, (scale, mode, bad[:5])
            # every row as a decode call of its own, whatever the batch
            y = torch.full((m, n_out), np.nan, dtype=torch.float32, device="cuda")
            hs.q4k_packed_gemv_x86(packed, n_out, n_in, d_x, y)
            hs.sync()
            got = y.cpu().numpy()
            for i in range(m):
                want = oracle_q4k_gemv_x86(oracle.lib, w, x[i], n_in)
                assert np.array_equal(got[i].view(np.uint32), want.view(np.uint32)), (scale, i)
    finally:
        hs.set_projection(0)


def test_q4k_decode_refuses_shapes_the_x86_kernel_does_not_take(hs):
    from geistlib_amd.binding import GeistHipError
    packed = torch.zeros((hs.q4k_packed_bytes(12, 256),), dtype=torch.uint8, device="cuda")
    x = torch.zeros((1, 256), dtype=torch.float32, device="cuda")
    y = torch.zeros((1, 12), dtype=torch.float32, device="cuda")
    with pytest.raises(GeistHipError):                        # 12 rows: not a multiple of 8
        hs.q4k_packed_gemv_x86(packed, 12, 256, x, y)


def test_q4k_x86_argument_errors(hs):
    from geistlib_amd.binding import GeistHipError
    packed = torch.zeros((hs.q4k_packed_bytes(8, 256) + 16,), dtype=torch.uint8, device="cuda")
    x = torch.zeros((4, 256), dtype=torch.float32, device="cuda")
    y = torch.full((4, 8), 7.0, dtype=torch.float32, device="cuda")
    hs.q4k_packed_linear_x86(packed, 8, 256, x, y)
    hs.sync()
    assert not y.cpu().numpy().any()                          # zeros: scale 1, every product 0
    f = hs.lib.geist_hip_q4k_packed_linear_x86_rows
    with pytest.raises(GeistHipError):                        # 12 rows: not a multiple of 8
        hs._check(f(hs.h, packed.data_ptr(), 12, 256, x.data_ptr(), 256, 4, y.data_ptr(), 12))
    with pytest.raises(GeistHipError):                        # packed copy not 16-byte aligned
        hs._check(f(hs.h, packed.data_ptr() + 4, 8, 256, x.data_ptr(), 256, 4, y.data_ptr(), 8))
    with pytest.raises(GeistHipError):                        # rows closer than their length
        hs._check(f(hs.h, packed.data_ptr(), 8, 256, x.data_ptr(), 128, 4, y.data_ptr(), 8))
    with pytest.raises(GeistHipError):                        # no rows
        hs._check(f(hs.h, packed.data_ptr(), 8, 256, x.data_ptr(), 256, 0, y.data_ptr(), 8))
    act = torch.zeros((hs.q8k_row_act_bytes(256) + 64,), dtype=torch.uint8, device="cuda")
    with pytest.raises(GeistHipError):                        # activations not 64-byte aligned
        hs._check(hs.lib.geist_hip_q8k_row_quantize(hs.h, x.data_ptr(), 256, act.data_ptr() + 4))
    with pytest.raises(GeistHipError):                        # not a whole number of blocks
        hs._check(hs.lib.geist_hip_q8k_row_quantize(hs.h, x.data_ptr(), 200, act.data_ptr()))
    assert hs.q8k_row_act_bytes(200) == 0 and hs.q8k_row_act_bytes(256) == (72 + 8) * 4


def test_q4k_linear_rows_whose_sums_cancel(hs, oracle):
    """Activations that repeat with alternating sign make pairs of products cancel: sums close to
    rounding boundaries, which only the reference's order of additions gets right."""
    g = np.random.default_rng(6)
    n_out, n_in = 3000, 1536
    w = random_q4k_table(g, n_out, n_in)
    packed = packed_copy(hs, w, n_in)
    for trial in range(3):
        x = (g.standard_normal((2, n_in)) * 3).astype(np.float32)
        x[:, 1::2] = -x[:, 0::2] * np.float32(1 + 2.0 ** -(8 + 4 * trial))
        want = oracle_q4k_linear(oracle.lib, w, x, n_in)
        y = torch.empty((2, n_out), dtype=torch.float32, device="cuda")
        hs.q4k_packed_linear(packed, n_out, n_in, torch.from_numpy(x).cuda(), y)
        hs.sync()
        assert np.array_equal(y.cpu().numpy().view(np.uint32), want.view(np.uint32)), trial


def test_q4k_argument_errors(hs):
    from geistlib_amd.binding import GeistHipError
    assert hs.q4k_packed_bytes(4, 200) == 0                   # not a whole number of blocks
    assert hs.q4k_packed_bytes(4, 256) == 64 * 37 * 4         # one group of 64 rows, one block
    w = torch.zeros((4, 144), dtype=torch.uint8, device="cuda")
    packed = torch.zeros((hs.q4k_packed_bytes(4, 256) + 16,), dtype=torch.uint8, device="cuda")
    x = torch.ones((1, 256), dtype=torch.float32, device="cuda")
    y = torch.full((1, 4), 7.0, dtype=torch.float32, device="cuda")
    hs.q4k_pack(w, 256, packed)
    hs.q4k_packed_linear(packed, 4, 256, x, y)
    hs.sync()
    assert not y.cpu().numpy().any()                          # a table of zeros
    with pytest.raises(GeistHipError):                        # packed copy not 16-byte aligned
        hs._check(hs.lib.geist_hip_q4k_packed_linear_rows(hs.h, packed.data_ptr() + 4, 4, 256,
                                                          x.data_ptr(), 256, 1, y.data_ptr(), 4))
    with pytest.raises(GeistHipError):                        # table not 4-byte aligned
        hs._check(hs.lib.geist_hip_q4k_pack(hs.h, w.data_ptr() + 2, 3, 256, packed.data_ptr()))


def test_head_over_a_q4k_table_with_a_soft_cap(host, oracle):
    """262144 x 1536 Q4_K behind the head with soft-cap 30 (head.c:94-188): norm, projection,
    soft-cap, dispatch, one shared generator. Tokens equal the oracle's session on the oracle's
    logits, for decode steps and for batches (3 rows: the decode kernel row by row; 4 and 8: the
    batch quantiser), in the x86 backend's arithmetic and in the portable one; without
    geist_hip_head_q4k_load the call is refused."""
    host.geist_hip_head_project_finalize_q4k.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t,
                                                         C.c_size_t, C.c_void_p, C.c_float,
                                                         C.c_void_p, C.c_size_t,
                                                         C.POINTER(C.c_int32)]
    host.geist_hip_head_q4k_load.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
    g = np.random.default_rng(2027)
    vocab, d_model, cap = 262144, 1536, 30.0
    w = random_q4k_table(g, vocab, d_model)
    w[:, 2::144] = 0                      # dmin = 0.0 or tiny: logits stay within the cap's range
    w[:, 3::144] &= 0x03
    norm_w = (1.0 + 0.1 * g.standard_normal(d_model)).astype(np.float32)
    d_w, d_nw = torch.from_numpy(w).cuda(), torch.from_numpy(norm_w).cuda()
    host.geist_hip_head_set_projection.argtypes = [C.c_void_p, C.c_int]
    for T, p, top_k, portable in [(0.0, 1.0, 0, False), (0.8, 1.0, 40, False),
                                  (0.9, 0.95, 0, False), (0.8, 1.0, 40, True)]:
        print(f"q4k table T={T} p={p} k={top_k} portable={portable}", flush=True)
        h = make_head(host, vocab, 8, cap)
        if portable:
            assert host.geist_hip_head_set_projection(h, 1) == 0
        opts = SessionOpts(0, T, p, top_k, 4242, None, 0, 8)
        assert host.geist_hip_head_apply_opts(h, C.byref(opts)) == 0
        hidden = (g.standard_normal((1, d_model)) * 4).astype(np.float32)
        d_hid = torch.from_numpy(hidden).cuda()
        out1 = (C.c_int32 * 1)()
        assert host.geist_hip_head_project_finalize_q4k(
            h, C.c_void_p(d_hid.data_ptr()), d_model, 1, C.c_void_p(d_nw.data_ptr()), 1e-6,
            C.c_void_p(d_w.data_ptr()), d_model, out1) != 0     # not loaded yet
        assert host.geist_hip_head_q4k_load(h, C.c_void_p(d_w.data_ptr()), d_model) == 0, \
            host.geist_hip_head_errmsg(h)
        sess = oracle.session(T, p, top_k, seed=4242)
        for k in (1, 1, 3, 4, 8):
            hidden = (g.standard_normal((k, d_model)) * 4).astype(np.float32)
            d_hid = torch.from_numpy(hidden).cuda()
            out = (C.c_int32 * k)()
            rc = host.geist_hip_head_project_finalize_q4k(
                h, C.c_void_p(d_hid.data_ptr()), d_model, k, C.c_void_p(d_nw.data_ptr()), 1e-6,
                C.c_void_p(d_w.data_ptr()), d_model, out)
            assert rc == 0, host.geist_hip_head_errmsg(h)
            normed = oracle.rmsnorm(hidden, norm_w, 1e-6)
            if not portable:    # the x86 backend: its decode kernel, cpu_x86_linear_q4k_mN
                logits = oracle_q4k_linear_x86(oracle.lib, w, normed, d_model)
            else:
                logits = oracle_q4k_linear(oracle.lib, w, normed, d_model)
            want = oracle.finalize_batch(sess, logits, softcap=cap).tolist()
            assert list(out) == want, (T, p, top_k, k, portable)
        host.geist_hip_head_destroy(h)
