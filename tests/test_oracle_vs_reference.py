"""Direct comparison of the oracle with the compiled reference (oracle/_ref) on seeded rows.
Runs where `make -C oracle ref` has produced the library; skipped elsewhere."""
import ctypes as C

import numpy as np
import pytest

from oracle_lib import OracleRng, RefWorkspace, _fp


def _ref_call(ref, row, mode, prm, rng):
    ws = RefWorkspace()
    assert ref.geist_sampler_workspace_init(C.byref(ws), row.size) == 0
    try:
        if mode == "temperature":
            return ref.geist_sampler_temperature(row.size, _fp(row), prm[0], C.byref(rng))
        if mode == "top_k":
            return ref.geist_sampler_top_k_ws(C.byref(ws), _fp(row), prm[0], prm[1], C.byref(rng))
        return ref.geist_sampler_top_p_ws(C.byref(ws), _fp(row), prm[0], prm[1], C.byref(rng))
    finally:
        ref.geist_sampler_workspace_destroy(C.byref(ws))


def _oracle_call(o, row, mode, prm, rng):
    if mode == "temperature":
        return o.lib.oracle_temperature(row.size, _fp(row), prm[0], C.byref(rng))
    if mode == "top_k":
        return o.lib.oracle_top_k(row.size, _fp(row), prm[0], prm[1], C.byref(rng))
    return o.lib.oracle_top_p(row.size, _fp(row), prm[0], prm[1], C.byref(rng))


@pytest.mark.parametrize("n", [1, 2, 7, 100, 1024, 1025, 5000, 8192, 8193, 40000])
def test_random_rows_all_modes(oracle, ref, n):
    g = np.random.default_rng(n)
    for trial in range(4):
        scale = [0.5, 2.0, 5.0, 1.0][trial]
        row = (g.standard_normal(n) * scale).astype(np.float32)
        if trial == 3:  # exact ties everywhere
            row = np.round(row * 2).astype(np.float32) / 2
        assert oracle.argmax(row) == ref.geist_sampler_argmax(n, _fp(row))
        cases = [("temperature", (0.7,)), ("temperature", (1.5,)), ("top_k", (5, 0.9)),
                 ("top_k", (40, 0.7)), ("top_k", (n, 1.0)), ("top_k", (9000, 1.3)),
                 ("top_p", (0.3, 1.0)), ("top_p", (0.9, 0.7)), ("top_p", (0.999, 2.0))]
        for mode, prm in cases:
            ra, rb = OracleRng(), OracleRng()
            ref.geist_rng_seed(C.byref(ra), C.c_uint64(1000 + trial))
            oracle.lib.oracle_rng_seed(C.byref(rb), C.c_uint64(1000 + trial))
            for _ in range(12):
                want = _ref_call(ref, row, mode, prm, ra)
                got = _oracle_call(oracle, row, mode, prm, rb)
                assert got == want, (n, trial, mode, prm)
            assert ra.state == rb.state


def test_u_variants_equal_rng_variants(oracle):
    g = np.random.default_rng(5)
    row = (g.standard_normal(3000) * 2).astype(np.float32)
    r1, r2 = oracle.rng(77), oracle.rng(77)
    for _ in range(20):
        u = oracle.next_unit(r1)
        assert oracle.top_k_u(row, 40, 0.7, u)[0] == oracle.lib.oracle_top_k(
            row.size, _fp(row), 40, 0.7, C.byref(r2))
    r1, r2 = oracle.rng(78), oracle.rng(78)
    for _ in range(20):
        u = oracle.next_unit(r1)
        assert oracle.top_p_u(row, 0.9, 0.7, u)[0] == oracle.lib.oracle_top_p(
            row.size, _fp(row), 0.9, 0.7, C.byref(r2))
        # the chain with a single filter set is the reference mode
        assert oracle.chain_u(row, u, temperature=0.7, top_p=0.9)[0] == oracle.top_p_u(row, 0.9, 0.7, u)[0]
        assert oracle.chain_u(row, u, temperature=0.7, top_k=40)[0] == oracle.top_k_u(row, 40, 0.7, u)[0]
        assert oracle.chain_u(row, u, temperature=0.7)[0] == oracle.temperature_u(row, 0.7, u)[0]


NONFINITE_ROWS = [("nan mid", lambda x: x.__setitem__(len(x) // 2, np.nan)),
                  ("nan first", lambda x: x.__setitem__(0, np.nan)),
                  ("nan last", lambda x: x.__setitem__(len(x) - 1, np.nan)),
                  ("+inf", lambda x: x.__setitem__(7 % len(x), np.inf)),
                  ("all -inf", lambda x: x.fill(-np.inf)),
                  ("all nan", lambda x: x.fill(np.nan))]


@pytest.mark.parametrize("n", [64, 300, 9000])
def test_rows_that_are_not_finite(oracle, ref, n):
    """A NaN or +inf in the row, or nothing finite at all: the softmax sum is NaN and the
    reference's functions fall through their loops (sampler.c:90-102, 243, 287-303). The oracle
    follows the compiled reference in the temperature and top-p modes, and with top-k where the
    row holds no NaN; with a NaN among finite values the reference's comparator is inconsistent
    (sampler.c:166-176 returns 0 against a NaN) and the pick is whatever libc's qsort makes of
    that: not pinned."""
    g = np.random.default_rng(n)
    for desc, mod in NONFINITE_ROWS:
        row = g.standard_normal(n).astype(np.float32)
        mod(row)
        for mode, prm in [("temperature", (0.9,)), ("top_p", (0.3, 1.3)), ("top_p", (0.9, 1.0)),
                          ("top_k", (40, 0.8))]:
            if mode == "top_k" and np.isnan(row).any() and not np.isnan(row).all():
                continue
            ra, rb = OracleRng(), OracleRng()
            ref.geist_rng_seed(C.byref(ra), C.c_uint64(5))
            oracle.lib.oracle_rng_seed(C.byref(rb), C.c_uint64(5))
            for _ in range(3):
                want = _ref_call(ref, row, mode, prm, ra)
                got = _oracle_call(oracle, row, mode, prm, rb)
                assert got == want, (n, desc, mode, prm)
            assert ra.state == rb.state
            if mode != "top_k":
                assert want == n - 1, (n, desc, mode)
