"""Sampling calls recorded into a HIP graph and replayed. The kernels of the modes that weigh
every element meet through slots that have to be zero when a launch starts; a recorded launch
uses an array of its own which a fill kernel recorded in front of it clears on every replay.
Every replay, with the program's own eager calls and waits in between, gives the oracle's ids."""
import numpy as np
import pytest

from gpu_util import compare_ids, to_dev

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


def units(g, rows):
    return (g.integers(0, 1 << 24, rows).astype(np.float32) / np.float32(1 << 24)).astype(np.float32)


def want_rows(oracle, x, u, **kw):
    res = [oracle.chain_u(x[r], float(u[r]), **kw) for r in range(x.shape[0])]
    return [t for t, _ in res], [i for _, i in res]


MODES = [
    (4, 128256, dict(temperature=0.8)),                       # one-kernel temperature draw
    (32, 50000, dict(temperature=0.9)),                       # exp-sum pass + index-order walk
    (64, 128256, dict(temperature=0.7, top_k=40, top_p=0.9)), # top-k in one launch
]
# the tolerance mode (a sampler object's: the entry point without one has no modes to set): the
# pass without a meeting and the launch that scales its sums
FAST = (32, 50000, dict(temperature=0.9, fast_sums=True))


@pytest.mark.parametrize("static,rows,n,kw", [(st, *m) for st in (False, True) for m in MODES]
                         + [(False, *FAST)])
def test_recorded_call_replays(oracle, static, rows, n, kw):
    from geistlib_amd import HipSampler, SampleParams, sample_rows_static
    kw = dict(kw)
    fast = kw.pop("fast_sums", False)
    g = np.random.default_rng(rows + n + static)
    prm = SampleParams.make(**kw)
    hs = HipSampler(rows, n)
    hs.set_sums(fast=fast)
    try:
        d_x = torch.zeros((rows, n), dtype=torch.float32, device="cuda")
        d_u = torch.zeros(rows, dtype=torch.float32, device="cuda")
        d_out = torch.full((rows,), -7, dtype=torch.int32, device="cuda")
        d_out2 = torch.full((rows,), -7, dtype=torch.int32, device="cuda")
        r = HipSampler.rows(d_x)

        def fresh():
            x = (g.standard_normal((rows, n)) * 2).astype(np.float32)
            u = units(g, rows)
            d_x.copy_(to_dev(x, torch))
            d_u.copy_(to_dev(u, torch))
            torch.cuda.synchronize()
            return x, u

        def eager(out):
            if static:
                sample_rows_static(r, prm, d_u, out, stream=None)
            else:
                hs.set_stream(None)
                hs.sample(r, prm, d_u, out)
            torch.cuda.synchronize()

        # eager calls first, so that the arrays of the eager launches are in use
        for _ in range(2):
            x, u = fresh()
            eager(d_out2)
            want, infos = want_rows(oracle, x, u, **kw)
            compare_ids(d_out2.cpu().numpy(), want, infos, f"eager before recording {kw}")

        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                sp = torch.cuda.current_stream().cuda_stream
                if static:
                    sample_rows_static(r, prm, d_u, d_out, stream=sp)
                else:
                    hs.set_stream(sp)
                    hs.sample(r, prm, d_u, d_out)
        torch.cuda.synchronize()
        if not static:
            hs.set_stream(None)

        for replay in range(4):
            x, u = fresh()
            d_out.fill_(-7)
            graph.replay()
            torch.cuda.synchronize()
            want, infos = want_rows(oracle, x, u, **kw)
            compare_ids(d_out.cpu().numpy(), want, infos, f"replay {replay} {kw} static={static}")
            if replay % 2 == 0:   # the program's own eager call between replays
                eager(d_out2)
                compare_ids(d_out2.cpu().numpy(), want, infos, f"eager after replay {replay} {kw}")
    finally:
        torch.cuda.synchronize()
        hs.close()
