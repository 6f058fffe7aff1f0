"""The lm_head over a Q6_K table on the GPU against the oracle, which is pinned to the reference's
own q6_K.c and weight_resolve.c (tests/test_q6k_oracle.py): logits bit for bit, for one activation
row and for batches, and token ids through the head with the Gemma soft-cap at the size of the
Gemma vocabulary."""
import ctypes as C

import numpy as np
import pytest

from oracle_lib import (oracle_q6k_gemv_x86, oracle_q6k_linear, oracle_q6k_linear_x86,
                        oracle_q8k_quantize, random_q6k_table)
from test_gpu_host_layer import SessionOpts, host, make_head  # noqa: F401 (fixture)

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def hs():
    from geistlib_amd import HipSampler
    s = HipSampler(max_rows=16, max_vocab=262144)
    yield s
    s.close()


@pytest.mark.parametrize("n_out,n_in,m", [(1, 256, 1), (64, 256, 1), (300, 512, 1), (1000, 768, 3),
                                          (5000, 1536, 1), (4097, 1536, 5), (2000, 2560, 9),
                                          (70000, 1024, 2)])
def test_q6k_linear_equals_the_portable_kernel(hs, oracle, n_out, n_in, m):
    print(f"q6k linear {n_out} x {n_in}, {m} rows", flush=True)
    g = np.random.default_rng(n_out + n_in + m)
    w = random_q6k_table(g, n_out, n_in)
    for scale in (1.0, 1e-4, 300.0):
        x = (g.standard_normal((m, n_in)) * scale).astype(np.float32)
        x[0, ::5] = 0.0
        want = oracle_q6k_linear(oracle.lib, w, x, n_in)
        d_w, d_x = torch.from_numpy(w).cuda(), torch.from_numpy(x).cuda()
        y = torch.full((m, n_out), np.nan, dtype=torch.float32, device="cuda")
        hs.q6k_linear(d_w, n_in, d_x, y)
        hs.sync()
        got = y.cpu().numpy()
        bad = np.argwhere(got.view(np.uint32) != want.view(np.uint32))
        assert bad.size == 0, (scale, bad[:5], got[tuple(bad[0])], want[tuple(bad[0])])
        # the same over the table repacked for the device
        packed = torch.full((hs.q6k_packed_bytes(n_out, n_in),), 0xA5, dtype=torch.uint8,
                            device="cuda")
        hs.q6k_pack(d_w, n_in, packed)
        y2 = torch.full((m, n_out), np.nan, dtype=torch.float32, device="cuda")
        hs.q6k_packed_linear(packed, n_out, n_in, d_x, y2)
        hs.sync()
        got = y2.cpu().numpy()
        bad = np.argwhere(got.view(np.uint32) != want.view(np.uint32))
        assert bad.size == 0, ("packed", scale, bad[:5], got[tuple(bad[0])], want[tuple(bad[0])])


def test_q6k_linear_rows_whose_sums_cancel(hs, oracle):
    """Sums that nearly cancel lie close to rounding boundaries far more often than random ones:
    every such output has to come out of the second, sequential kernel with the reference's
    bits. Activations that repeat with alternating sign make pairs of products cancel."""
    g = np.random.default_rng(5)
    n_out, n_in = 3000, 1536
    w = random_q6k_table(g, n_out, n_in)
    for trial in range(3):
        x = (g.standard_normal((2, n_in)) * 3).astype(np.float32)
        x[:, 1::2] = -x[:, 0::2] * np.float32(1 + 2.0 ** -(8 + 4 * trial))
        want = oracle_q6k_linear(oracle.lib, w, x, n_in)
        y = torch.empty((2, n_out), dtype=torch.float32, device="cuda")
        d_w, d_x = torch.from_numpy(w).cuda(), torch.from_numpy(x).cuda()
        hs.q6k_linear(d_w, n_in, d_x, y)
        hs.sync()
        assert np.array_equal(y.cpu().numpy().view(np.uint32), want.view(np.uint32)), trial
        packed = torch.empty((hs.q6k_packed_bytes(n_out, n_in),), dtype=torch.uint8, device="cuda")
        hs.q6k_pack(d_w, n_in, packed)
        y.fill_(0)
        hs.q6k_packed_linear(packed, n_out, n_in, d_x, y)
        hs.sync()
        assert np.array_equal(y.cpu().numpy().view(np.uint32), want.view(np.uint32)), trial


@pytest.mark.parametrize("n_out,n_in", [(1, 256), (64, 256), (300, 512), (5000, 1536),
                                        (4097, 2560), (70000, 1024)])
def test_q6k_decode_equals_the_x86_kernel(hs, oracle, n_out, n_in):
    """The x86 backend's integer decode kernel (kernel_q6k_gemv.c), to which the oracle is pinned
    by the compiled reference (tests/test_q6k_x86_oracle.py): logits bit for bit, row by row."""
    print(f"q6k x86 decode {n_out} x {n_in}", flush=True)
    g = np.random.default_rng(n_out + n_in)
    w = random_q6k_table(g, n_out, n_in)
    d_w = torch.from_numpy(w).cuda()
    packed = torch.full((hs.q6k_packed_bytes(n_out, n_in),), 0xA5, dtype=torch.uint8, device="cuda")
    hs.q6k_pack(d_w, n_in, packed)
    for scale in (1.0, 1e-4, 300.0, 0.0):
        x = (g.standard_normal((3, n_in)) * scale).astype(np.float32)
        x[0, ::5] = 0.0
        x[1, :256] = 0.0                      # a super-block of zeros: its scale is zero
        x[2, 7] = np.float32(1e30)            # one huge activation: the others round to zero
        d_x = torch.from_numpy(x).cuda()
        y = torch.full((3, n_out), np.nan, dtype=torch.float32, device="cuda")
        hs.q6k_packed_gemv_x86(packed, n_out, n_in, d_x, y)
        hs.sync()
        got = y.cpu().numpy()
        for m in range(3):
            want = oracle_q6k_gemv_x86(oracle.lib, w, x[m], n_in)
            bad = np.flatnonzero(got[m].view(np.uint32) != want.view(np.uint32))
            assert bad.size == 0, (scale, m, bad[:5], got[m][bad[:3]], want[bad[:3]])
        # the same over the table as it lies in the file
        y0 = torch.full((3, n_out), np.nan, dtype=torch.float32, device="cuda")
        hs.q6k_gemv_x86(d_w, n_in, d_x, y0)
        hs.sync()
        assert np.array_equal(y0.cpu().numpy().view(np.uint32), got.view(np.uint32)), scale
        # the kernel's two halves: the int8 activations as the reference's quantiser leaves
        # them, and the dot products over them
        nb = n_in // 256
        act = torch.full((hs.q8k_act_bytes(n_in, 3) // 4,), -1, dtype=torch.int32, device="cuda")
        hs.q8k_quantize(d_x, act)
        y1 = torch.full((n_out,), np.nan, dtype=torch.float32, device="cuda")
        hs.q6k_packed_gemv_q8k(packed, n_out, n_in, act[2 * nb * 96:], y1)
        hs.sync()
        a = act.cpu().numpy().reshape(3, nb, 96)
        for m in range(3):
            d, qs, bs = oracle_q8k_quantize(oracle.lib, x[m])
            assert (a[m, :, :64].copy().view(np.int8).reshape(-1) == qs).all(), (scale, m)
            assert (a[m, :, 64:80].reshape(-1) == bs.astype(np.int32)).all(), (scale, m)
            assert (a[m, :, 80].copy().view(np.uint32) == d.view(np.uint32)).all(), (scale, m)
        assert (y1.cpu().numpy().view(np.uint32) == got[2].view(np.uint32)).all(), scale


def tie_rows(g, m, n_in, scale):
    """Rows whose scale is a power of two, with activations exactly between two int8 values."""
    x = (g.standard_normal((m, n_in)) * scale).astype(np.float32)
    x[:, ::7] = 0.0
    d = np.float32(2.0) ** np.ceil(np.log2(scale) - 3)
    x[:, 0] = np.float32(127.0) * d
    for k, h in enumerate((0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 63.5, -126.5)):
        x[:, 1 + k] = np.float32(h) * d
    return x


@pytest.mark.parametrize("n_out,n_in,m", [(64, 512, 2), (300, 512, 3), (5000, 1536, 4), (304, 512, 5),
                                          (4100, 2560, 8), (64, 256, 12), (4112, 1024, 16),
                                          (72, 16384, 2), (70000, 1024, 7), (1, 256, 2)])
def test_q6k_batch_equals_the_x86_backend(hs, oracle, n_out, n_in, m):
    """cpu_x86_linear_q6k_mN, to which the oracle is pinned by the compiled reference
    (tests/test_q6k_x86_oracle.py), over the packed copy and over the table as it lies: in
    projection mode X86 the lane kernels' arithmetic for tables of a multiple of 8 rows and the
    scalar kernel's for the others, in mode X86_AVX2 the scalar kernel's for all. Logits bit for
    bit, one row included (the decode kernel)."""
    print(f"q6k x86 batch {n_out} x {n_in}, {m} rows", flush=True)
    g = np.random.default_rng(n_out + n_in + m)
    w = random_q6k_table(g, n_out, n_in)
    d_w = torch.from_numpy(w).cuda()
    packed = torch.full((hs.q6k_packed_bytes(n_out, n_in),), 0xA5, dtype=torch.uint8, device="cuda")
    hs.q6k_pack(d_w, n_in, packed)
    try:
        for scale in (1.0, 1e-3, 100.0):
            x = tie_rows(g, m, n_in, scale)
            d_x = torch.from_numpy(x).cuda()
            for mode, vnni in ((0, True), (2, False)):
                hs.set_projection(mode)
                want = oracle_q6k_linear_x86(oracle.lib, w, x, n_in, vnni=vnni)
                for over_packed in (True, False):
                    y = torch.full((m, n_out), np.nan, dtype=torch.float32, device="cuda")
                    if over_packed:
                        hs.q6k_packed_linear_x86(packed, n_out, n_in, d_x, y)
                    else:
                        hs.q6k_linear_x86(d_w, n_in, d_x, y)
                    hs.sync()
                    got = y.cpu().numpy()
                    bad = np.argwhere(got.view(np.uint32) != want.view(np.uint32))
                    assert bad.size == 0, (scale, mode, over_packed, bad[:5])
        x1 = tie_rows(g, 1, n_in, 1.0)
        y = torch.full((1, n_out), np.nan, dtype=torch.float32, device="cuda")
        hs.q6k_packed_linear_x86(packed, n_out, n_in, torch.from_numpy(x1).cuda(), y)
        hs.sync()
        want = oracle_q6k_gemv_x86(oracle.lib, w, x1[0], n_in)
        assert np.array_equal(y.cpu().numpy()[0].view(np.uint32), want.view(np.uint32))
    finally:
        hs.set_projection(0)


def test_q6k_linear_with_activations_that_are_not_finite(hs, oracle):
    """An infinity, two of opposite sign, a NaN among the activations: the reference's sum in
    index order gives +-inf or NaN per output (golden case of tests/golden/q6k_ref_vectors.json,
    written from the compiled reference), and both device kernels give the same -- the kernel
    over the table as it lies sends every such output to its second, index-order kernel."""
    g = np.random.default_rng(404)
    n_out, n_in, m = 700, 768, 4
    w = random_q6k_table(g, n_out, n_in, scale_mode="plain")
    x = g.standard_normal((m, n_in)).astype(np.float32)
    x[0, 5] = np.inf
    x[1, 9], x[1, 300] = -np.inf, np.inf
    x[2, 17] = np.nan
    want = oracle_q6k_linear(oracle.lib, w, x, n_in)     # row 3 is finite
    assert np.isinf(want[0]).any() and np.isnan(want[1]).any() and np.isinf(want[1]).any()
    d_w, d_x = torch.from_numpy(w).cuda(), torch.from_numpy(x).cuda()
    packed = torch.zeros((hs.q6k_packed_bytes(n_out, n_in),), dtype=torch.uint8, device="cuda")
    hs.q6k_pack(d_w, n_in, packed)
    for name in ("as in the file", "packed"):
        y = torch.full((m, n_out), 7.0, dtype=torch.float32, device="cuda")
        if name == "packed":
            hs.q6k_packed_linear(packed, n_out, n_in, d_x, y)
        else:
            hs.q6k_linear(d_w, n_in, d_x, y)
        hs.sync()
        got = y.cpu().numpy()
        assert np.array_equal(np.isnan(got), np.isnan(want)), name
        ok = ~np.isnan(want)
        assert np.array_equal(got.view(np.uint32)[ok], want.view(np.uint32)[ok]), name


def test_q6k_argument_errors(hs):
    from geistlib_amd.binding import GeistHipError
    w = torch.zeros((4, 210), dtype=torch.uint8, device="cuda")
    x = torch.zeros((1, 256), dtype=torch.float32, device="cuda")
    y = torch.zeros((1, 4), dtype=torch.float32, device="cuda")
    hs.q6k_linear(w, 256, x, y)
    hs.sync()
    assert not y.cpu().numpy().any()
    with pytest.raises(GeistHipError):                       # not a whole number of blocks
        hs._check(hs.lib.geist_hip_q6k_linear_rows(hs.h, w.data_ptr(), 4, 200, x.data_ptr(), 256, 1,
                                                   y.data_ptr(), 4))
    with pytest.raises(GeistHipError):                       # table not 4-byte aligned
        hs._check(hs.lib.geist_hip_q6k_linear_rows(hs.h, w.data_ptr() + 2, 3, 256, x.data_ptr(),
                                                   256, 1, y.data_ptr(), 4))
    # the x86 backend's batch path: the same rules
    x2 = torch.zeros((2, 256), dtype=torch.float32, device="cuda")
    y2 = torch.full((2, 4), 7.0, dtype=torch.float32, device="cuda")
    hs.q6k_linear_x86(w, 256, x2, y2)
    hs.sync()
    assert not y2.cpu().numpy().any()                        # zeros: scale 1, every product 0
    packed = torch.zeros((hs.q6k_packed_bytes(4, 256) + 16,), dtype=torch.uint8, device="cuda")
    for fn, table in ((hs.lib.geist_hip_q6k_linear_x86_rows, w.data_ptr() + 2),         # alignment
                      (hs.lib.geist_hip_q6k_packed_linear_x86_rows, packed.data_ptr() + 4)):
        with pytest.raises(GeistHipError):
            hs._check(fn(hs.h, table, 4, 256, x2.data_ptr(), 256, 2, y2.data_ptr(), 4))
    with pytest.raises(GeistHipError):                       # rows closer than their length
        hs._check(hs.lib.geist_hip_q6k_packed_linear_x86_rows(hs.h, packed.data_ptr(), 4, 256,
                                                              x2.data_ptr(), 128, 2, y2.data_ptr(), 4))
    with pytest.raises(GeistHipError):                       # no rows
        hs._check(hs.lib.geist_hip_q6k_packed_linear_x86_rows(hs.h, packed.data_ptr(), 4, 256,
                                                              x2.data_ptr(), 256, 0, y2.data_ptr(), 4))
    with pytest.raises(GeistHipError):                       # an unknown projection mode
        hs.set_projection(3)


def test_head_over_the_gemma_table_with_the_soft_cap(host, oracle):
    """262144 x 1536 Q6_K (the tied table of the Gemma models) behind the head with soft-cap 30
    (head.c:94-188): norm, projection, soft-cap, dispatch, one shared generator. Tokens equal the
    oracle's session on the oracle's logits, for decode steps and for batches of 3 and 8 rows, in
    the x86 backend's arithmetic (over the packed copy and over the table as it lies) and in the
    portable one."""
    host.geist_hip_head_project_finalize_q6k.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t,
                                                         C.c_size_t, C.c_void_p, C.c_float,
                                                         C.c_void_p, C.c_size_t,
                                                         C.POINTER(C.c_int32)]
    host.geist_hip_head_reserve_projection_q6k.argtypes = [C.c_void_p, C.c_size_t]
    host.geist_hip_head_q6k_load.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
    g = np.random.default_rng(2026)
    vocab, d_model, cap = 262144, 1536, 30.0
    w = random_q6k_table(g, vocab, d_model, scale_mode="plain")
    norm_w = (1.0 + 0.1 * g.standard_normal(d_model)).astype(np.float32)
    d_w, d_nw = torch.from_numpy(w).cuda(), torch.from_numpy(norm_w).cuda()
    host.geist_hip_head_set_projection.argtypes = [C.c_void_p, C.c_int]
    for T, p, top_k, portable in [(0.0, 1.0, 0, False), (0.8, 1.0, 40, False),
                                  (0.9, 0.95, 0, False), (0.8, 1.0, 40, True)]:
        print(f"gemma table T={T} p={p} k={top_k} portable={portable}", flush=True)
        h = make_head(host, vocab, 8, cap)
        if portable:
            assert host.geist_hip_head_set_projection(h, 1) == 0
        opts = SessionOpts(0, T, p, top_k, 31337, None, 0, 8)
        assert host.geist_hip_head_apply_opts(h, C.byref(opts)) == 0
        packed = not (top_k == 0 and T == 0.0)
        if not packed:      # one configuration reads the table as it lies, the others packed
            assert host.geist_hip_head_reserve_projection_q6k(h, d_model) == 0
        else:
            assert host.geist_hip_head_q6k_load(h, C.c_void_p(d_w.data_ptr()), d_model) == 0, \
                host.geist_hip_head_errmsg(h)
        sess = oracle.session(T, p, top_k, seed=31337)
        for k in (1, 1, 3, 8):
            hidden = (g.standard_normal((k, d_model)) * 4).astype(np.float32)
            d_hid = torch.from_numpy(hidden).cuda()
            out = (C.c_int32 * k)()
            rc = host.geist_hip_head_project_finalize_q6k(
                h, C.c_void_p(d_hid.data_ptr()), d_model, k, C.c_void_p(d_nw.data_ptr()), 1e-6,
                C.c_void_p(d_w.data_ptr()), d_model, out)
            assert rc == 0, host.geist_hip_head_errmsg(h)
            normed = oracle.rmsnorm(hidden, norm_w, 1e-6)
            if not portable:    # the x86 backend (decode kernel, batch path), packed copy or not
                logits = oracle_q6k_linear_x86(oracle.lib, w, normed, d_model)
            else:
                logits = oracle_q6k_linear(oracle.lib, w, normed, d_model)
            want = oracle.finalize_batch(sess, logits, softcap=cap).tolist()
            assert list(out) == want, (T, p, top_k, k)
        host.geist_hip_head_destroy(h)
