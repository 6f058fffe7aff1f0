"""The C23 host layer on a GPU: the reference's sampler symbols served by the HIP path, and the
session/head mirror. The checks restate the reference's tests/test_sampler_unit.c (eight checks)
and the model-free part of its session sampling tests; where the reference's own unit-test binary
was built against this library (oracle/_ref/test_sampler_unit_hip) it is run as well."""
import ctypes as C
import os
import subprocess

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
c_float_p = C.POINTER(C.c_float)


class Rng(C.Structure):
    _fields_ = [("state", C.c_uint64)]


class Ws(C.Structure):
    _fields_ = [("probs", c_float_p), ("n_vocab", C.c_size_t)]


class SessionOpts(C.Structure):
    _fields_ = [("max_seq_len", C.c_size_t), ("temperature", C.c_float), ("top_p", C.c_float),
                ("top_k", C.c_int), ("random_seed", C.c_uint64), ("awq_scales_path", C.c_char_p),
                ("kv_mode", C.c_int), ("m_max", C.c_size_t)]


@pytest.fixture(scope="module")
def host():
    lib = C.CDLL(os.path.join(ROOT, "geistlib_amd", "lib", "libgeist_sampler_host.so"))
    lib.geist_rng_next_u64.restype = C.c_uint64
    lib.geist_rng_next_unit.restype = C.c_float
    lib.geist_sampler_argmax.argtypes = [C.c_size_t, c_float_p]
    lib.geist_sampler_temperature.argtypes = [C.c_size_t, c_float_p, C.c_float, C.POINTER(Rng)]
    lib.geist_sampler_workspace_init.argtypes = [C.POINTER(Ws), C.c_size_t]
    lib.geist_sampler_workspace_destroy.argtypes = [C.POINTER(Ws)]
    lib.geist_sampler_top_k_ws.argtypes = [C.POINTER(Ws), c_float_p, C.c_int, C.c_float,
                                           C.POINTER(Rng)]
    lib.geist_sampler_top_p_ws.argtypes = [C.POINTER(Ws), c_float_p, C.c_float, C.c_float,
                                           C.POINTER(Rng)]
    lib.geist_hip_head_create.argtypes = [C.c_int, C.c_size_t, C.c_size_t, C.c_float, C.c_void_p,
                                          C.POINTER(C.c_void_p)]
    lib.geist_hip_head_destroy.argtypes = [C.c_void_p]
    lib.geist_hip_head_errmsg.restype = C.c_char_p
    lib.geist_hip_head_errmsg.argtypes = [C.c_void_p]
    lib.geist_hip_head_apply_opts.argtypes = [C.c_void_p, C.POINTER(SessionOpts)]
    lib.geist_hip_head_finalize_one_row.argtypes = [C.c_void_p, C.c_void_p, C.POINTER(C.c_int32)]
    lib.geist_hip_head_finalize_batch.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t,
                                                  C.POINTER(C.c_int32)]
    lib.geist_hip_head_argmax_f32.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t,
                                              C.POINTER(C.c_int32)]
    lib.geist_hip_head_rng_state.argtypes = [C.c_void_p, C.POINTER(C.c_uint64)]
    lib.geist_hip_head_propose_drafts.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int32,
                                                  C.c_size_t, C.POINTER(C.c_int32),
                                                  C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]
    lib.geist_hip_head_project_finalize.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t,
                                                    C.c_void_p, C.c_float, C.c_void_p, C.c_size_t,
                                                    C.POINTER(C.c_int32)]
    lib.geist_hip_head_project_finalize_q8w.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t,
                                                        C.c_size_t, C.c_void_p, C.c_float,
                                                        C.c_void_p, C.c_void_p, C.c_size_t,
                                                        C.POINTER(C.c_int32)]
    lib.geist_hip_head_spec_build.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t,
                                              C.c_size_t]
    lib.geist_hip_head_project_finalize_spec.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p,
                                                         C.c_float, C.c_void_p, C.c_size_t, C.c_int,
                                                         C.POINTER(C.c_int32), C.POINTER(C.c_int)]
    lib.geist_hip_head_logits.restype = C.c_void_p
    lib.geist_hip_head_logits.argtypes = [C.c_void_p]
    lib.geist_hip_head_spec_accept.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t,
                                               C.POINTER(C.c_int32), C.c_int, C.c_size_t,
                                               C.POINTER(C.c_int32), C.POINTER(C.c_size_t)]
    return lib


def fp(a):
    return a.ctypes.data_as(c_float_p)


def f32(*v):
    return np.array(v, dtype=np.float32)


def test_reference_unit_test_binary_on_the_hip_path():
    exe = os.path.join(ROOT, "oracle", "_ref", "test_sampler_unit_hip")
    if not os.path.exists(exe):
        pytest.skip("built only where the reference tree is mounted (make -C oracle ref)")
    r = subprocess.run([exe], capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "PASS: all 8 sampler checks" in r.stdout
    # check 4 is bit-deterministic (expf(0) == 1): the counts the reference prints
    assert "[997 1055 979 999 970]" in r.stdout


def test_eight_reference_checks(host, oracle):
    # 1 (tests/test_sampler_unit.c:33-37)
    x = f32(-1, 2, .5, 3, 3, -.5)
    assert host.geist_sampler_argmax(6, fp(x)) == 3
    # 2 (40-51)
    rng = Rng()
    host.geist_rng_seed(C.byref(rng), C.c_uint64(42))
    x = f32(0, 0, 0, 10, 0)
    hits = sum(host.geist_sampler_temperature(5, fp(x), 0.1, C.byref(rng)) == 3 for _ in range(1000))
    assert hits > 990
    # 3 (54-60): greedy, and no draw consumed
    host.geist_rng_seed(C.byref(rng), C.c_uint64(1))
    x = f32(1, 2, 3, .5)
    assert host.geist_sampler_temperature(4, fp(x), 0.0, C.byref(rng)) == 2
    assert rng.state == 1
    # 4 (63-89): exact counts
    host.geist_rng_seed(C.byref(rng), C.c_uint64(7))
    x = np.zeros(5, dtype=np.float32)
    counts = [0] * 5
    for _ in range(5000):
        counts[host.geist_sampler_temperature(5, fp(x), 1.0, C.byref(rng))] += 1
    assert counts == [997, 1055, 979, 999, 970]
    # 5 (92-112)
    host.geist_rng_seed(C.byref(rng), C.c_uint64(11))
    x = f32(0, 1, 4, 2, 5, 1.5, 0, .5)
    ws = Ws()
    assert host.geist_sampler_workspace_init(C.byref(ws), 8) == 0
    seen = set(host.geist_sampler_top_k_ws(C.byref(ws), fp(x), 2, 1.0, C.byref(rng))
               for _ in range(1000))
    host.geist_sampler_workspace_destroy(C.byref(ws))
    assert seen == {2, 4}
    # 6 (115-131)
    host.geist_rng_seed(C.byref(rng), C.c_uint64(13))
    x = f32(10, 0, 0, 0, 0)
    assert host.geist_sampler_workspace_init(C.byref(ws), 5) == 0
    hits = sum(host.geist_sampler_top_p_ws(C.byref(ws), fp(x), 0.5, 1.0, C.byref(rng)) == 0
               for _ in range(1000))
    host.geist_sampler_workspace_destroy(C.byref(ws))
    assert hits > 990
    # 7 (134-148): workspace reuse, destroy is idempotent and NULL-safe
    assert host.geist_sampler_workspace_init(C.byref(ws), 8) == 0
    host.geist_rng_seed(C.byref(rng), C.c_uint64(17))
    x = f32(.1, .2, .3, 5, .1, 0, 0, 0)
    for _ in range(100):
        host.geist_sampler_top_k_ws(C.byref(ws), fp(x), 3, 1.0, C.byref(rng))
    host.geist_sampler_workspace_destroy(C.byref(ws))
    host.geist_sampler_workspace_destroy(C.byref(ws))
    host.geist_sampler_workspace_destroy(None)
    assert ws.n_vocab == 0 and not ws.probs
    # workspace_init argument errors (sampler.c:138-140): GEIST_E_INVALID_ARG == 2
    assert host.geist_sampler_workspace_init(None, 8) == 2
    assert host.geist_sampler_workspace_init(C.byref(ws), 0) == 2


def test_symbols_follow_the_oracle_draw_for_draw(host, oracle):
    g = np.random.default_rng(9)
    n = 20000
    x = (g.standard_normal(n) * 2).astype(np.float32)
    ws = Ws()
    assert host.geist_sampler_workspace_init(C.byref(ws), n) == 0
    cases = [("temperature", (0.8,)), ("top_k", (40, 0.7)), ("top_k", (1, 0.7)),
             ("top_k", (n + 5, 0.9)), ("top_k", (300, 1.1)), ("top_p", (0.9, 0.7)),
             ("top_p", (1.0, 0.7)), ("top_p", (0.0, 0.7)), ("temperature", (0.0,))]
    for mode, prm in cases:
        rng = Rng()
        host.geist_rng_seed(C.byref(rng), C.c_uint64(0xC0FFEE))
        r = oracle.rng(0xC0FFEE)
        for _ in range(6):
            if mode == "temperature":
                got = host.geist_sampler_temperature(n, fp(x), prm[0], C.byref(rng))
                want = oracle.lib.oracle_temperature(n, fp(x), prm[0], C.byref(r))
            elif mode == "top_k":
                got = host.geist_sampler_top_k_ws(C.byref(ws), fp(x), prm[0], prm[1], C.byref(rng))
                want = oracle.lib.oracle_top_k(n, fp(x), prm[0], prm[1], C.byref(r))
            else:
                got = host.geist_sampler_top_p_ws(C.byref(ws), fp(x), prm[0], prm[1], C.byref(rng))
                want = oracle.lib.oracle_top_p(n, fp(x), prm[0], prm[1], C.byref(r))
            assert got == want, (mode, prm)
        assert rng.state == int(r.state), "draw count differs from the reference"
    host.geist_sampler_workspace_destroy(C.byref(ws))


# ------------------------------------------------------------------ session / head mirror
def make_head(host, vocab, m_max=0, softcap=0.0):
    h = C.c_void_p()
    assert host.geist_hip_head_create(0, vocab, m_max, softcap, None, C.byref(h)) == 0
    return h


def test_head_dispatch_precedence_and_rng(host, oracle):
    """Model-free statement of tests/test_session_sampling_int.c: greedy is repeatable, a seeded
    stochastic run differs from greedy and repeats with the same seed; plus the dispatch table of
    head.c:172-183 and the draw count per mode."""
    g = np.random.default_rng(31)
    vocab = 32000
    x = (g.standard_normal((8, vocab)) * 2).astype(np.float32)
    d = torch.from_numpy(x).cuda()
    table = [(0.0, 1.0, 0), (0.0, 0.9, 40), (0.7, 0.9, 40), (0.7, 1.0, 40), (0.7, 0.9, 1),
             (0.7, 0.9, 0), (0.7, 1.0, 0), (0.7, 0.0, 0), (0.7, -2.0, 0), (10.0, 1.0, 200)]
    for T, p, k in table:
        h = make_head(host, vocab)
        opts = SessionOpts(0, T, p, k, 0xDEADBEEF, None, 0, 0)
        assert host.geist_hip_head_apply_opts(h, C.byref(opts)) == 0
        sess = oracle.session(T, p, k, seed=0xDEADBEEF)
        # one row at a time (decode_step cadence) ...
        for r in range(3):
            tok = C.c_int32(-1)
            assert host.geist_hip_head_finalize_one_row(h, C.c_void_p(d[r].data_ptr()),
                                                        C.byref(tok)) == 0
            assert tok.value == oracle.finalize_row(sess, x[r]), (T, p, k, r)
        # ... then a batch of rows with the shared RNG (verify_forward cadence)
        out = (C.c_int32 * 5)()
        assert host.geist_hip_head_finalize_batch(h, C.c_void_p(d[3].data_ptr()), 5, out) == 0
        assert list(out) == oracle.finalize_batch(sess, x[3:8]).tolist(), (T, p, k)
        st = C.c_uint64(0)
        assert host.geist_hip_head_rng_state(h, C.byref(st)) == 0
        assert st.value == int(sess.rng.state), "RNG consumption differs"
        host.geist_hip_head_destroy(h)


def test_head_sums_within_the_contracts_tolerance(host, oracle):
    """geist_hip_head_set_sums(h, 1): the head's temperature and top-p rows with the sums of
    exponentials from the hardware's 2^z. The tokens are the reference's on rows whose draws lie
    away from slot edges (all of these: a draw within 1e-7 of an edge is a one-in-thousands
    event), and the RNG is consumed as before."""
    g = np.random.default_rng(77)
    vocab = 50000
    x = (g.standard_normal((24, vocab)) * 2).astype(np.float32)
    d = torch.from_numpy(x).cuda()
    host.geist_hip_head_set_sums.argtypes = [C.c_void_p, C.c_int]
    for T, p, k in [(0.8, 1.0, 0), (0.9, 0.9, 0)]:
        h = make_head(host, vocab)
        opts = SessionOpts(0, T, p, k, 0xC0FFEE, None, 0, 0)
        assert host.geist_hip_head_apply_opts(h, C.byref(opts)) == 0
        assert host.geist_hip_head_set_sums(h, 7) != 0
        assert host.geist_hip_head_set_sums(h, 1) == 0
        sess = oracle.session(T, p, k, seed=0xC0FFEE)
        out = (C.c_int32 * 24)()
        assert host.geist_hip_head_finalize_batch(h, C.c_void_p(d.data_ptr()), 24, out) == 0
        assert list(out) == oracle.finalize_batch(sess, x).tolist(), (T, p, k)
        st = C.c_uint64(0)
        assert host.geist_hip_head_rng_state(h, C.byref(st)) == 0
        assert st.value == int(sess.rng.state)
        host.geist_hip_head_destroy(h)


def test_head_defaults_and_null_opts(host, oracle):
    vocab = 5000
    g = np.random.default_rng(2)
    x = (g.standard_normal((1, vocab)) * 2).astype(np.float32)
    d = torch.from_numpy(x).cuda()
    h = make_head(host, vocab)
    assert host.geist_hip_head_apply_opts(h, None) == 0          # NULL opts = greedy
    st = C.c_uint64(0)
    host.geist_hip_head_rng_state(h, C.byref(st))
    assert st.value == 0xCAFEBABE1234                              # arch_state.c:1173
    tok = C.c_int32(-1)
    assert host.geist_hip_head_finalize_one_row(h, C.c_void_p(d.data_ptr()), C.byref(tok)) == 0
    assert tok.value == oracle.argmax(x[0])
    host.geist_hip_head_rng_state(h, C.byref(st))
    assert st.value == 0xCAFEBABE1234                              # greedy draws nothing
    # random_seed == 0 keeps the default seed (step.c:393-395)
    opts = SessionOpts(0, 0.8, 1.0, 0, 0, None, 0, 0)
    host.geist_hip_head_apply_opts(h, C.byref(opts))
    host.geist_hip_head_rng_state(h, C.byref(st))
    assert st.value == 0xCAFEBABE1234
    # more rows than m_max is refused
    out = (C.c_int32 * 100)()
    assert host.geist_hip_head_finalize_batch(h, C.c_void_p(d.data_ptr()), 100, out) != 0
    assert b"m_max" in host.geist_hip_head_errmsg(h)
    host.geist_hip_head_destroy(h)


def test_head_argmax_slot(host):
    # tests/test_fused_probe_agreement_unit.c:147-157: p[i] = (i == 77 ? 100 : i % 7) -> 77
    p = np.array([100.0 if i == 77 else i % 7 for i in range(256)], dtype=np.float32)
    d = torch.from_numpy(p).cuda()
    h = make_head(host, 256)
    idx = C.c_int32(-1)
    assert host.geist_hip_head_argmax_f32(h, C.c_void_p(d.data_ptr()), 256, C.byref(idx)) == 0
    assert idx.value == 77
    assert host.geist_hip_head_argmax_f32(h, C.c_void_p(d.data_ptr()), 999, C.byref(idx)) == 7
    host.geist_hip_head_destroy(h)


def test_head_softcap_only_when_sampling(host, oracle):
    """head.c:148-159: tanhf(x / c) * c in front of the stochastic samplers, skipped when greedy.
    The device evaluates glibc's tanhf, so the ids are held to the bar of every other mode: equal
    unless the draw lies within 1e-6 of a CDF boundary."""
    g = np.random.default_rng(5)
    vocab, cap = 20000, 30.0
    x = (g.standard_normal((6, vocab)) * 12).astype(np.float32)
    d = torch.from_numpy(x).cuda()
    h = make_head(host, vocab, 0, cap)
    opts = SessionOpts(0, 0.9, 1.0, 50, 77, None, 0, 0)
    host.geist_hip_head_apply_opts(h, C.byref(opts))
    out = (C.c_int32 * 6)()
    assert host.geist_hip_head_finalize_batch(h, C.c_void_p(d.data_ptr()), 6, out) == 0
    r = oracle.rng(77)
    agree = 0
    for i in range(6):
        u = oracle.next_unit(r)
        want, info = oracle.top_k_u(oracle.softcap(x[i], cap), 50, 0.9, u)
        agree += (out[i] == want) or info.boundary_dist < 1e-6
    assert agree == 6
    host.geist_hip_head_destroy(h)


# ------------------------------------------------------------------ speculative accept step
def _accept(host, h, d, drafts, mode):
    k = len(drafts)
    dr = (C.c_int32 * k)(*drafts)
    out = (C.c_int32 * (k + 1))(*([-1] * (k + 1)))
    n_out = C.c_size_t(0)
    rc = host.geist_hip_head_spec_accept(h, C.c_void_p(d.data_ptr()), k, dr, mode, k + 1, out,
                                         C.byref(n_out))
    return rc, list(out)[:n_out.value]


@pytest.mark.parametrize("T,p,k_top", [(0.0, 1.0, 0), (0.8, 1.0, 0), (0.8, 0.9, 40), (0.7, 0.92, 0)])
def test_spec_accept_reference_loop(host, oracle, T, p, k_top):
    """src/engine/session.c:599-625 restated: sample every verify row with the session's
    sampler (shared RNG, row order), accept the longest prefix with sampled[i] == drafts[i+1],
    emit drafts[0..accepted] and the correction sampled[accepted]."""
    g = np.random.default_rng(41)
    vocab, k = 20000, 6
    x = (g.standard_normal((k, vocab)) * 3).astype(np.float32)
    x[np.arange(k), [11, 22, 33, 44, 55, 66]] += 30.0        # rows 0..5 all but surely pick these
    d = torch.from_numpy(x).cuda()
    for drafts in ([7, 11, 22, 33, 44, 55], [7, 11, 22, 99, 44, 55], [7, 5, 22, 33, 44, 55]):
        h = make_head(host, vocab)
        opts = SessionOpts(0, T, p, k_top, 1234, None, 0, 0)
        assert host.geist_hip_head_apply_opts(h, C.byref(opts)) == 0
        sess = oracle.session(T, p, k_top, seed=1234)
        sampled = oracle.finalize_batch(sess, x).tolist()
        acc = 0
        for i in range(k - 1):
            if sampled[i] != drafts[i + 1]:
                break
            acc += 1
        want = drafts[:acc + 1] + [sampled[acc]]
        rc, got = _accept(host, h, d, drafts, 0)
        assert rc == 0 and got == want, (T, drafts, got, want)
        st = C.c_uint64(0)
        host.geist_hip_head_rng_state(h, C.byref(st))
        assert st.value == int(sess.rng.state)
        host.geist_hip_head_destroy(h)


def test_spec_accept_rejection_sampling_point_mass(host, oracle):
    """Rejection sampling against the n-gram drafter's certain proposals: the oracle's verify with
    one-hot draft probabilities, fed the same k uniforms the session's RNG yields."""
    g = np.random.default_rng(43)
    vocab, k = 5000, 5
    L = k - 1
    for trial in range(12):
        x = (g.standard_normal((k, vocab)) * 2).astype(np.float32)
        drafts = [3] + [int(t) for t in g.integers(0, vocab, L)]
        for j in range(L):                                  # make acceptance likely but not sure
            x[j, drafts[j + 1]] += np.float32(g.choice([4.0, 8.0, 12.0]))
        d = torch.from_numpy(x).cuda()
        h = make_head(host, vocab)
        opts = SessionOpts(0, 0.9, 1.0, 0, 77 + trial, None, 0, 0)
        assert host.geist_hip_head_apply_opts(h, C.byref(opts)) == 0
        r = oracle.rng(77 + trial)
        u = np.array([oracle.next_unit(r) for _ in range(k)], dtype=np.float32)
        q = np.zeros((L, vocab), dtype=np.float32)
        q[np.arange(L), drafts[1:]] = 1.0
        n_acc, toks = oracle.spec_verify(x, q, np.array(drafts[1:], np.int32), u, 0.9)
        want = [drafts[0]] + toks[:n_acc + 1].tolist()
        rc, got = _accept(host, h, d, drafts, 1)
        assert rc == 0 and got == want, (trial, got, want)
        st = C.c_uint64(0)
        host.geist_hip_head_rng_state(h, C.byref(st))
        assert st.value == int(r.state), "k draws per round"
        host.geist_hip_head_destroy(h)
    # a filtered target is refused in this mode, the greedy session falls back to exact match
    h = make_head(host, vocab)
    opts = SessionOpts(0, 0.9, 0.9, 0, 1, None, 0, 0)
    host.geist_hip_head_apply_opts(h, C.byref(opts))
    rc, _ = _accept(host, h, d, drafts, 1)
    assert rc == 7
    host.geist_hip_head_destroy(h)


def test_head_propose_drafts_follows_the_reference_drafter(host, oracle):
    """session.c:564-572 with the token history on the device: seed + n-gram drafts with
    max_suffix = 4, against the restated propose_drafts_ngram."""
    g = np.random.default_rng(12)
    h = make_head(host, 1000)
    seen = set()
    for case in range(40):
        n = int(g.choice([0, 1, 5, 60, 3000]))
        alphabet = int(g.choice([2, 5, 40]))
        hist = g.integers(0, alphabet, max(n, 1)).astype(np.int32)
        d = torch.from_numpy(hist).cuda()
        seed = int(g.integers(0, alphabet))
        k_max = int(g.integers(1, 17))
        out = (C.c_int32 * 16)(*([-5] * 16))
        n_out, mlen = C.c_size_t(77), C.c_size_t(77)
        rc = host.geist_hip_head_propose_drafts(h, C.c_void_p(d.data_ptr()), n, seed, k_max, out,
                                                C.byref(n_out), C.byref(mlen))
        assert rc == 0, host.geist_hip_head_errmsg(h)
        want, wl = oracle.propose_drafts_ngram(hist[:n], seed, k_max, 4)
        assert list(out)[:n_out.value] == want and mlen.value == wl, (case, n, seed, k_max)
        seen.add(wl)
    assert seen == {0, 1, 2, 3, 4}
    out = (C.c_int32 * 16)()
    n_out = C.c_size_t(0)
    assert host.geist_hip_head_propose_drafts(h, None, 0, 3, 17, out, C.byref(n_out), None) != 0
    assert host.geist_hip_head_propose_drafts(h, None, 5, 3, 4, out, C.byref(n_out), None) != 0
    assert host.geist_hip_head_propose_drafts(h, None, 0, 3, 4, out, C.byref(n_out), None) == 0
    assert n_out.value == 1 and out[0] == 3
    host.geist_hip_head_destroy(h)


def test_head_project_finalize_keeps_the_logits_on_the_device(host, oracle):
    """head.c:94-188 / 224-304 in one call: output norm, tied F16 lm_head, soft-cap, sampler with
    the session's RNG. The tokens are those of the oracle's session on the oracle's logits."""
    g = np.random.default_rng(77)
    vocab, d_model, k, cap = 20000, 1536, 5, 30.0
    w16 = (g.standard_normal((vocab, d_model)) * 0.08).astype(np.float16)
    hidden = (g.standard_normal((k, d_model + 4)) * 2).astype(np.float32)   # padded row stride
    norm_w = (1.0 + 0.1 * g.standard_normal(d_model)).astype(np.float32)
    d_w = torch.from_numpy(w16.view(np.int16)).cuda()
    d_hid = torch.from_numpy(hidden).cuda()
    d_nw = torch.from_numpy(norm_w).cuda()
    want_logits = oracle.f16_linear_f64(w16.view(np.uint16),
                                        oracle.rmsnorm(hidden[:, :d_model], norm_w, 1e-6))
    for T, p, top_k in [(0.0, 1.0, 0), (0.8, 1.0, 40), (0.9, 0.9, 0), (1.1, 1.0, 0)]:
        h = make_head(host, vocab, 0, cap)
        opts = SessionOpts(0, T, p, top_k, 4242, None, 0, 0)
        assert host.geist_hip_head_apply_opts(h, C.byref(opts)) == 0
        out = (C.c_int32 * k)()
        rc = host.geist_hip_head_project_finalize(h, C.c_void_p(d_hid.data_ptr()), d_model + 4, k,
                                                  C.c_void_p(d_nw.data_ptr()), 1e-6,
                                                  C.c_void_p(d_w.data_ptr()), d_model, out)
        assert rc == 0, host.geist_hip_head_errmsg(h)
        sess = oracle.session(T, p, top_k, seed=4242)
        assert list(out) == oracle.finalize_batch(sess, want_logits, softcap=cap).tolist(), (T, p, top_k)
        ptr = host.geist_hip_head_logits(h)
        got = torch.empty((k, vocab), dtype=torch.float32, device="cuda")
        C.cdll.LoadLibrary("libamdhip64.so").hipMemcpy(C.c_void_p(got.data_ptr()), C.c_void_p(ptr),
                                                       C.c_size_t(k * vocab * 4), 3)
        assert (got.cpu().numpy().view(np.uint32) == want_logits.view(np.uint32)).all()
        host.geist_hip_head_destroy(h)
    assert (d_hid.cpu().numpy() == hidden).all()                             # input untouched


def test_head_project_finalize_q8w_is_the_decode_step_of_the_x86_backend(host, oracle):
    """The int8 table behind the head (src/backends/cpu_x86/backend.c:332-372 under
    head.c:114-126): tokens are those of the oracle's session on rmsnorm + q8w_gemv_m1 logits."""
    g = np.random.default_rng(78)
    vocab, d_model, cap = 20000, 1536, 30.0
    w16 = (g.standard_normal((vocab, d_model)) * 0.08).astype(np.float16)
    wq, sc = oracle.f16_to_q8w(w16.view(np.uint16))
    norm_w = (1.0 + 0.1 * g.standard_normal(d_model)).astype(np.float32)
    d_wq, d_sc, d_nw = torch.from_numpy(wq).cuda(), torch.from_numpy(sc).cuda(), torch.from_numpy(norm_w).cuda()
    for T, p, top_k in [(0.0, 1.0, 0), (0.8, 1.0, 40), (0.9, 0.9, 0)]:
        h = make_head(host, vocab, 0, cap)
        opts = SessionOpts(0, T, p, top_k, 99, None, 0, 0)
        assert host.geist_hip_head_apply_opts(h, C.byref(opts)) == 0
        sess = oracle.session(T, p, top_k, seed=99)
        for step in range(3):                                   # three decode steps, one row each
            hidden = (g.standard_normal((1, d_model)) * 2).astype(np.float32)
            d_hid = torch.from_numpy(hidden).cuda()
            out = (C.c_int32 * 1)()
            rc = host.geist_hip_head_project_finalize_q8w(
                h, C.c_void_p(d_hid.data_ptr()), d_model, 1, C.c_void_p(d_nw.data_ptr()), 1e-6,
                C.c_void_p(d_wq.data_ptr()), C.c_void_p(d_sc.data_ptr()), d_model, out)
            assert rc == 0, host.geist_hip_head_errmsg(h)
            want_logits = oracle.q8w_gemv(wq, sc, oracle.rmsnorm(hidden, norm_w, 1e-6))
            assert list(out) == oracle.finalize_batch(sess, want_logits, softcap=cap).tolist(), (T, p, top_k, step)
        assert host.geist_hip_head_project_finalize_q8w(
            h, C.c_void_p(d_hid.data_ptr()), d_model, 1, C.c_void_p(d_nw.data_ptr()), 1e-6,
            C.c_void_p(d_wq.data_ptr()), None, d_model, out) != 0
        host.geist_hip_head_destroy(h)


def test_head_project_finalize_spec_follows_head_c(host, oracle):
    """head.c:99-129 with the sketch head in front: greedy sessions take the sketch's answer
    (the oracle's token), with the bound on a declined step falls back to the dense head, and a
    session that samples never uses the sketch."""
    g = np.random.default_rng(79)
    vocab, d_model = 66000, 1280
    w16 = (g.standard_normal((vocab, d_model)) * 0.08).astype(np.float16)
    norm_w = (1.0 + 0.1 * g.standard_normal(d_model)).astype(np.float32)
    d_w, d_nw = torch.from_numpy(w16.view(np.int16)).cuda(), torch.from_numpy(norm_w).cuda()
    sh = oracle.spec_head_build(w16.view(np.uint16))
    h = make_head(host, vocab, 0, 30.0)
    assert host.geist_hip_head_spec_build(h, C.c_void_p(d_w.data_ptr()), d_model, 0, 0) == 0, \
        host.geist_hip_head_errmsg(h)
    out, used = C.c_int32(), C.c_int()
    for step in range(4):
        hidden = (g.standard_normal(d_model) * 2).astype(np.float32)
        d_hid = torch.from_numpy(hidden).cuda()
        normed = oracle.rmsnorm(hidden, norm_w, 1e-6)
        dense = oracle.f16_gemv(w16.view(np.uint16), normed)
        for verify in (0, 1):
            rc = host.geist_hip_head_project_finalize_spec(
                h, C.c_void_p(d_hid.data_ptr()), C.c_void_p(d_nw.data_ptr()), 1e-6,
                C.c_void_p(d_w.data_ptr()), d_model, verify, C.byref(out), C.byref(used))
            assert rc == 0, host.geist_hip_head_errmsg(h)
            want = sh.try_row(normed, verify=bool(verify))
            assert bool(used.value) == want["certain"]
            if used.value:
                assert out.value == want["token"]
                assert host.geist_hip_head_logits(h) is None
            else:
                assert out.value == int(np.flatnonzero(dense == dense.max())[0])
                assert host.geist_hip_head_logits(h) is not None
    # a sampling session: the sketch is not consulted (spec_head.c:645)
    opts = SessionOpts(0, 0.8, 1.0, 40, 5, None, 0, 0)
    assert host.geist_hip_head_apply_opts(h, C.byref(opts)) == 0
    rc = host.geist_hip_head_project_finalize_spec(
        h, C.c_void_p(d_hid.data_ptr()), C.c_void_p(d_nw.data_ptr()), 1e-6,
        C.c_void_p(d_w.data_ptr()), d_model, 0, C.byref(out), C.byref(used))
    assert rc == 0 and used.value == 0
    sess = oracle.session(0.8, 1.0, 40, seed=5)
    assert out.value == oracle.finalize_batch(sess, dense[None, :], softcap=30.0).tolist()[0]
    # no sketch where the reference builds none: the call reports it and the head stays dense
    h2 = make_head(host, 9000, 0, 0.0)
    d_small = torch.zeros((9000, d_model), dtype=torch.float16, device="cuda")
    assert host.geist_hip_head_spec_build(h2, C.c_void_p(d_small.data_ptr()), d_model, 0, 0) != 0
    host.geist_hip_head_destroy(h2)
    host.geist_hip_head_destroy(h)
