"""The allocation-free entry point, geist_hip_sample_rows_static, through the C ABI: the oracle's
token ids, and the same ids bit for bit as geist_hip_sample_rows, on two calls in a row, the second
on a smaller batch (the workspace array keeps the first call's contents); and, in a fresh process,
before any sampler object exists (the call looks the array's device address up itself)."""
import os
import subprocess
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

from gpu_util import compare_ids, to_dev  # noqa: E402


def _oracle_ids(oracle, x, u, hist, hl, cfg):
    kw = {k: v for k, v in cfg.items() if k not in ("rep", "freq", "pres")}
    want, infos = [], []
    for r in range(x.shape[0]):
        row = x[r]
        if "rep" in cfg:
            row = oracle.penalties(row, hist[r][: hl[r]], cfg["rep"], cfg["freq"], cfg["pres"])
        if cfg["temperature"] == 0.0:
            want.append(oracle.argmax(row))
            infos.append(None)
        else:
            t, i = oracle.chain_u(row, float(u[r]), **kw)
            want.append(t)
            infos.append(i)
    return want, infos


def _batch(seed, rows, n, hist_n):
    g = np.random.default_rng(seed)
    x = (g.standard_normal((rows, n)) * 2).astype(np.float32)
    x[0, : min(n, 50)] = 1.25                      # a run of equal values
    u = (g.integers(0, 1 << 24, rows).astype(np.float32) / np.float32(1 << 24)).astype(np.float32)
    hist = g.integers(0, n, (rows, hist_n)).astype(np.int32)
    hist[:, : hist_n // 4] = np.argsort(-x, axis=1)[:, : hist_n // 4]   # leading tokens penalised
    hl = np.full(rows, hist_n, dtype=np.int32)
    return x, u, hist, hl


CONFIGS = [
    dict(temperature=0.7, top_k=40, top_p=0.9, rep=1.1, freq=0.5, pres=0.3),
    dict(temperature=0.0),
    dict(temperature=0.8),
    dict(temperature=0.6, top_k=64, top_p=0.9, min_p=0.02),
    dict(temperature=1.0, top_k=500),
]


def test_static_entry_point_matches_sample_rows(oracle):
    from geistlib_amd import HipSampler, SampleParams, sample_rows_static
    assert torch.cuda.is_available()
    hs = HipSampler(max_rows=64, max_vocab=128256)
    try:
        # two calls in a row per configuration: a full-size batch, then a smaller one
        for ci, cfg in enumerate(CONFIGS):
            for call, (rows, n, hist_n) in enumerate([(64, 128256, 512), (5, 30001, 100)]):
                print(f"static entry point: config {ci} call {call} rows={rows} n={n}", flush=True)
                x, u, hist, hl = _batch(100 * ci + call, rows, n, hist_n)
                d_x, d_u = to_dev(x, torch), to_dev(u, torch)
                d_h, d_hl = to_dev(hist, torch), to_dev(hl, torch)
                pen = "rep" in cfg
                r = HipSampler.rows(d_x, d_h if pen else None, d_hl if pen else None)
                prm = SampleParams.make(**cfg)
                want = torch.full((rows,), -7, dtype=torch.int32, device="cuda")
                got = torch.full((rows,), -9, dtype=torch.int32, device="cuda")
                hs.sample(r, prm, d_u, want)
                hs.sync()
                sample_rows_static(r, prm, d_u, got)
                torch.cuda.synchronize()
                assert got.cpu().tolist() == want.cpu().tolist(), (ci, call)
                o_want, o_infos = _oracle_ids(oracle, x, u, hist, hl, cfg)
                if cfg["temperature"] == 0.0:
                    assert got.cpu().tolist() == o_want, (ci, call)
                else:
                    compare_ids(got.cpu().numpy(), o_want, o_infos, f"static config {ci} call {call}")
    finally:
        hs.close()


def test_static_entry_point_rejects_what_it_cannot_serve():
    from geistlib_amd import HipSampler, SampleParams, sample_rows_static
    from geistlib_amd.binding import GeistHipError
    x = torch.zeros((66, 128256), dtype=torch.float32, device="cuda")
    u = torch.zeros(66, dtype=torch.float32, device="cuda")
    out = torch.zeros(66, dtype=torch.int32, device="cuda")
    with pytest.raises(GeistHipError) as e:   # 66 x 63 units > 4096
        sample_rows_static(HipSampler.rows(x), SampleParams.make(temperature=0.7, top_k=40), u, out)
    assert e.value.code == 2 and "static workspace" in str(e.value)
    with pytest.raises(GeistHipError) as e:   # top-p without top-k needs the probability rows
        sample_rows_static(HipSampler.rows(x[:4]), SampleParams.make(temperature=0.7, top_p=0.9),
                           u, out)
    assert e.value.code == 7


_FRESH = r"""
import sys
sys.path.insert(0, sys.argv[1]); sys.path.insert(0, sys.argv[1] + "/tests")
import numpy as np, torch
from geistlib_amd import HipSampler, SampleParams, sample_rows_static
from oracle_lib import Oracle
g = np.random.default_rng(5)
rows, n = 16, 128256
x = (g.standard_normal((rows, n)) * 2).astype(np.float32)
u = (g.integers(0, 1 << 24, rows).astype(np.float32) / np.float32(1 << 24)).astype(np.float32)
d_x, d_u = torch.from_numpy(x).cuda(), torch.from_numpy(u).cuda()
o = Oracle()
# no sampler object has been made in this process: the first call finds the array itself
for kw in (dict(temperature=0.7, top_k=40, top_p=0.9), dict(temperature=0.8), dict(temperature=0.7, top_k=40, top_p=0.9)):
    out = torch.full((rows,), -7, dtype=torch.int32, device="cuda")
    sample_rows_static(HipSampler.rows(d_x), SampleParams.make(**kw), d_u, out)
    torch.cuda.synchronize()
    got = out.cpu().tolist()
    for r in range(rows):
        want, info = o.chain_u(x[r], float(u[r]), **kw)
        assert got[r] == want or info.boundary_dist < 1e-6, (kw, r, got[r], want)
print("fresh process OK")
"""


def test_static_entry_point_before_any_sampler_exists():
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run([sys.executable, "-c", _FRESH, root], capture_output=True, text=True,
                       timeout=300)
    assert p.returncode == 0 and "fresh process OK" in p.stdout, (p.stdout[-2000:], p.stderr[-2000:])
