"""The threading contract of the reference's sampler (src/engine/sampler.h:8: every entry point is
reentrant, one thread per session, different sessions concurrent), driven the way the reference's
tests/test_multi_session_parallel_int.c:1-24 drives it: 4 host threads x 4 sessions, each with its
own sampling options and generator, all running at once. Every thread's token ids and generator
states must equal the oracle's single-threaded sessions."""
import ctypes as C
import threading

import numpy as np
import pytest

from test_gpu_host_layer import Rng, SessionOpts, Ws, fp, host, make_head  # noqa: F401 (fixture)

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")

N_THREADS, N_SESSIONS = 4, 4
VOCAB = 32000
# (temperature, top_p, top_k): the dispatch table of head.c:172-183, one line per session
OPTS = [(0.0, 1.0, 0), (0.7, 0.9, 40), (0.7, 1.0, 40), (0.7, 0.9, 0),
        (0.7, 1.0, 0), (1.3, 0.5, 0), (0.9, 1.0, 8), (0.7, 0.9, 40)]


def head_with_stream(host, vocab):
    """A head that enqueues on a stream of its own."""
    st = torch.cuda.Stream()
    h = C.c_void_p()
    assert host.geist_hip_head_create(0, vocab, 0, 0.0, C.c_void_p(st.cuda_stream), C.byref(h)) == 0
    return h, st


def decode_steps(host, h, d, i0, i1):
    """Decode-style cadence: rows one at a time, and a batch of 5 after every fourth row."""
    ids = []
    n = d.shape[0]
    for i in range(i0, i1):
        tok = C.c_int32(-1)
        rc = host.geist_hip_head_finalize_one_row(h, C.c_void_p(d[i % n].data_ptr()), C.byref(tok))
        assert rc == 0, host.geist_hip_head_errmsg(h)
        ids.append(tok.value)
        if i % 4 == 3:
            out = (C.c_int32 * 5)()
            r0 = (i * 3) % (n - 5)
            rc = host.geist_hip_head_finalize_batch(h, C.c_void_p(d[r0].data_ptr()), 5, out)
            assert rc == 0, host.geist_hip_head_errmsg(h)
            ids += list(out)
    return ids


def rng_state(host, h):
    st = C.c_uint64(0)
    assert host.geist_hip_head_rng_state(h, C.byref(st)) == 0
    return st.value


def oracle_loop(oracle, x, T, p, k, seed, steps):
    """The same cadence on one oracle session, single-threaded."""
    sess = oracle.session(T, p, k, seed=seed)
    ids = []
    n = x.shape[0]
    for i in range(steps):
        ids.append(int(oracle.finalize_row(sess, x[i % n])))
        if i % 4 == 3:
            r0 = (i * 3) % (n - 5)
            ids += oracle.finalize_batch(sess, x[r0:r0 + 5]).tolist()
    return ids, int(sess.rng.state)


def run_threads(fn, n):
    errors = [None] * n

    def guarded(t):
        try:
            fn(t)
        except BaseException as e:  # noqa: BLE001 (reported in the main thread)
            errors[t] = e

    th = [threading.Thread(target=guarded, args=(t,)) for t in range(n)]
    for t in th:
        t.start()
    for t in th:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in th), "a thread did not finish"
    for e in errors:
        if e is not None:
            raise e


def test_four_threads_times_four_sessions(host, oracle):
    g = np.random.default_rng(77)
    x = (g.standard_normal((16, VOCAB)) * 2).astype(np.float32)
    d = torch.from_numpy(x).cuda()
    torch.cuda.synchronize()
    steps = 24
    combos = {(t, s): (*OPTS[(t * N_SESSIONS + s) % len(OPTS)], 0xC0FFEE + 97 * t + s)
              for t in range(N_THREADS) for s in range(N_SESSIONS)}
    heads = {}
    for key, (T, p, k, seed) in combos.items():
        h, st = head_with_stream(host, VOCAB)
        opts = SessionOpts(0, T, p, k, seed, None, 0, 0)
        assert host.geist_hip_head_apply_opts(h, C.byref(opts)) == 0
        heads[key] = (h, st)
    got = {}
    barrier = threading.Barrier(N_THREADS)

    def worker(t):
        barrier.wait()
        # the thread's sessions advance in turn, as a server thread that owns several would
        ids = {s: [] for s in range(N_SESSIONS)}
        for i0 in range(0, steps, 4):
            for s in range(N_SESSIONS):
                ids[s] += decode_steps(host, heads[(t, s)][0], d, i0, i0 + 4)
        for s in range(N_SESSIONS):
            got[(t, s)] = (ids[s], rng_state(host, heads[(t, s)][0]))

    run_threads(worker, N_THREADS)
    assert len(got) == N_THREADS * N_SESSIONS
    for key, (T, p, k, seed) in combos.items():
        assert got[key] == oracle_loop(oracle, x, T, p, k, seed, steps), key
    for h, _ in heads.values():
        host.geist_hip_head_destroy(h)


def test_sessions_made_and_destroyed_inside_threads(host, oracle):
    """Each thread creates, uses and destroys its own heads while the others do the same."""
    g = np.random.default_rng(5)
    x = (g.standard_normal((12, 5000)) * 3).astype(np.float32)
    d = torch.from_numpy(x).cuda()
    torch.cuda.synchronize()
    results = {}

    def worker(t):
        for s in range(N_SESSIONS):
            T, p, k = OPTS[(3 * t + s) % len(OPTS)]
            h, st = head_with_stream(host, 5000)
            opts = SessionOpts(0, T, p, k, 1000 + 10 * t + s, None, 0, 0)
            assert host.geist_hip_head_apply_opts(h, C.byref(opts)) == 0
            results[(t, s)] = (decode_steps(host, h, d, 0, 8), rng_state(host, h))
            host.geist_hip_head_destroy(h)

    run_threads(worker, N_THREADS)
    for (t, s), (ids, state) in results.items():
        T, p, k = OPTS[(3 * t + s) % len(OPTS)]
        assert (ids, state) == oracle_loop(oracle, x, T, p, k, 1000 + 10 * t + s, 8), (t, s)


def dropin_sequence(host, oracle, x, seed, check):
    """All nine symbols of src/engine/sampler.h on one thread: its own generator, its own
    workspace, the thread's own hidden context behind argmax / temperature."""
    n = x.shape[1]
    rng, orng = Rng(), oracle.rng(seed)
    host.geist_rng_seed(C.byref(rng), C.c_uint64(seed))
    ws = Ws()
    assert host.geist_sampler_workspace_init(C.byref(ws), n) == 0
    for i, row in enumerate(x):
        check(host.geist_sampler_argmax(n, fp(row)), oracle.argmax(row), ("argmax", i))
        check(host.geist_rng_next_u64(C.byref(rng)), oracle.next_u64(orng), ("u64", i))
        check(host.geist_sampler_temperature(n, fp(row), 0.8, C.byref(rng)),
              oracle.temperature_u(row, 0.8, oracle.next_unit(orng))[0], ("temperature", i))
        check(host.geist_sampler_top_k_ws(C.byref(ws), fp(row), 40, 0.7, C.byref(rng)),
              oracle.top_k_u(row, 40, 0.7, oracle.next_unit(orng))[0], ("top_k", i))
        check(host.geist_sampler_top_p_ws(C.byref(ws), fp(row), 0.9, 0.7, C.byref(rng)),
              oracle.top_p_u(row, 0.9, 0.7, oracle.next_unit(orng))[0], ("top_p", i))
        check(host.geist_rng_next_unit(C.byref(rng)), oracle.next_unit(orng), ("unit", i))
    host.geist_sampler_workspace_destroy(C.byref(ws))
    check(rng.state, int(orng.state), ("state",))


def test_dropin_symbols_from_four_threads(host, oracle):
    g = np.random.default_rng(123)
    xs = [(g.standard_normal((6, 4096 + 1000 * t)) * 2).astype(np.float32)
          for t in range(N_THREADS)]
    for wave in range(2):  # the second wave's threads are new: the first wave's contexts are gone
        mism = []

        def worker(t):
            def check(got, want, where):
                if got != want:
                    mism.append((t, where, got, want))
            dropin_sequence(host, oracle, xs[t], 900 + 31 * t + wave, check)

        run_threads(worker, N_THREADS)
        assert not mism, mism[:5]
