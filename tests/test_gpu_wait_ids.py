"""geist_hip_sampler_notify_ids / _wait_ids: a caller learns that the ids of a sampling call are
written from a word in page-locked memory instead of waiting for the stream; when the word does
not change in time the call falls back to the stream. Both ways the ids are the oracle's."""
import numpy as np
import pytest

from gpu_util import compare_ids, to_dev

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def P():
    from geistlib_amd import SampleParams
    return SampleParams.make


def units(g, rows):
    return (g.integers(0, 1 << 24, rows) / np.float32(1 << 24)).astype(np.float32)


def want_rows(oracle, x, u, hist=None, pen=None, **kw):
    res = []
    for r in range(x.shape[0]):
        row = x[r] if hist is None else oracle.penalties(x[r], hist[r], *pen)
        res.append(oracle.chain_u(row, float(u[r]), **kw))
    return [t for t, _ in res], [i for _, i in res]


@pytest.mark.parametrize("spin_us", [2000, 0])
def test_ids_reported_into_host_memory(oracle, P, spin_us):
    """spin_us = 2000: the word is watched (the one-launch top-k kernel reports from its own last
    row, every other configuration from a launch behind its kernels); 0: the fallback, the wait
    for the stream. Several calls in a row on changing rows, the ids read from page-locked memory
    right after the wait."""
    from geistlib_amd import HipSampler
    rows, n = 64, 128256
    g = np.random.default_rng(31 + spin_us)
    hs = HipSampler(rows, n)
    try:
        hs.notify_ids(True)
        hs.set_wait_spin(spin_us)
        out_host = hs.host_buffer(rows * 4)
        ids = out_host.view(np.int32)
        hist = g.integers(0, n, (rows, 512)).astype(np.int32)
        hl = np.full(rows, 512, dtype=np.int32)
        d_h, d_hl = to_dev(hist, torch), to_dev(hl, torch)
        configs = [
            (dict(temperature=0.7, top_k=40, top_p=0.9), (1.1, 0.5, 0.3)),   # one launch
            (dict(temperature=0.7, top_k=40, top_p=0.9), None),              # one launch, plain
            (dict(temperature=0.8), None),                                   # exp-sum + walk
            (dict(temperature=0.0), None),                                   # argmax
        ]
        for call in range(3):
            x = (g.standard_normal((rows, n)) * 2).astype(np.float32)
            u = units(g, rows)
            d_x, d_u = to_dev(x, torch), to_dev(u, torch)
            for kw, pen in configs:
                ids[:] = -7
                pk = {} if pen is None else dict(rep=pen[0], freq=pen[1], pres=pen[2])
                r = HipSampler.rows(d_x, d_h if pen else None, d_hl if pen else None)
                hs.sample(r, P(**kw, **pk), d_u, out_host)
                hs.wait_ids()
                got = ids.copy()          # no wait for the stream in between
                if kw["temperature"] == 0.0:
                    assert got.tolist() == [oracle.argmax(x[i]) for i in range(rows)]
                else:
                    want, infos = want_rows(oracle, x, u, hist=hist if pen else None, pen=pen, **kw)
                    compare_ids(got, want, infos, f"call {call} {kw} pen {pen} spin {spin_us}")
        hs.sync()
        out_host.close()
    finally:
        hs.close()


@pytest.mark.parametrize("rows", [1, 5])
def test_short_rows_report_after_their_ids_have_arrived(oracle, P, rows):
    """One workgroup per row and a few rows: the kernel that writes the ids tells the host within
    a microsecond of writing them, so an id that lingered in a cache on its way would be read one
    call late. Many calls in a row, every one checked right after the wait."""
    from geistlib_amd import HipSampler
    n = 32000
    g = np.random.default_rng(rows)
    hs = HipSampler(8, n)
    try:
        hs.notify_ids(True)
        out_host = hs.host_buffer(rows * 4)
        ids = out_host.view(np.int32)
        kw = dict(temperature=0.8, top_k=40, top_p=0.95)
        xs = (g.standard_normal((12, rows, n)) * 2).astype(np.float32)
        d_xs = [to_dev(x, torch) for x in xs]
        torch.cuda.synchronize()
        for call in range(48):
            x = xs[call % 12]
            u = units(g, rows)
            d_u = to_dev(u, torch)
            hs.sample(HipSampler.rows(d_xs[call % 12]), P(**kw), d_u, out_host)
            hs.wait_ids()
            got = ids.copy()
            want, infos = want_rows(oracle, x, u, **kw)
            compare_ids(got, want, infos, f"call {call}, {rows} rows")
        hs.sync()
        out_host.close()
    finally:
        hs.close()
