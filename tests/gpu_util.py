"""Helpers of the GPU parity tests: move a workload to the device, run it through the C ABI and
compare token ids with the oracle under the counted-exception rule."""
import os

import numpy as np


def fuzz_seeds(n):
    """The seeds of a randomised test: n by default, n * GEIST_TEST_FUZZ_SCALE for a long run
    (GEIST_TEST_FUZZ_SCALE=60 python -m pytest tests -m gpu -k random)."""
    return range(n * max(1, int(os.environ.get("GEIST_TEST_FUZZ_SCALE", "1"))))


# A draw closer than this (relative to the mass of the walk) to an edge of its CDF slot may
# legitimately land in the neighbouring slot on the device; such rows are counted, not failed.
BOUNDARY_TOL = 1e-6


def to_dev(a, torch):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def pack_allowed(allowed):
    """bool [rows, n] -> int32 mask words [rows, ceil(n / 32)], bit e % 32 of word e / 32."""
    rows, n = allowed.shape
    words = (n + 31) // 32
    bits = np.zeros((rows, words * 32), dtype=np.uint8)
    bits[:, :n] = allowed
    packed = np.packbits(bits.reshape(rows, words, 32), axis=-1, bitorder="little")
    return np.ascontiguousarray(packed).view(np.uint32).reshape(rows, words).view(np.int32)


def run_rows(sampler, torch, logits, uniforms, params, history=None, history_len=None,
             pad=0, lead=0, allowed=None):
    """pad: extra elements between rows; lead: elements before the first row (an unaligned base).
    Both gaps hold a huge logit, so a read outside a row changes the result."""
    from geistlib_amd import HipSampler
    if pad or lead:
        rows, n = logits.shape
        flat = np.full(lead + rows * (n + pad), 3e38, dtype=np.float32)
        body = flat[lead:].reshape(rows, n + pad)
        body[:, :n] = logits
        d_flat = to_dev(flat, torch)
        d_logits = d_flat[lead:].view(rows, n + pad)[:, :n]
    else:
        d_logits = to_dev(logits, torch)
    d_u = to_dev(uniforms, torch) if uniforms is not None else None
    d_h = to_dev(history, torch) if history is not None else None
    d_hl = to_dev(history_len, torch) if history_len is not None else None
    out = torch.full((logits.shape[0],), -7, dtype=torch.int32, device="cuda")
    d_a = to_dev(pack_allowed(allowed), torch) if allowed is not None else None
    rows = HipSampler.rows(d_logits, d_h, d_hl, allowed=d_a)
    sampler.sample(rows, params, d_u, out)
    sampler.sync()
    return out.cpu().numpy()


def compare_ids(got, want, infos, what=""):
    """Bit-exact ids, except rows whose draw lies within BOUNDARY_TOL of a CDF slot edge, where
    the contract allows either neighbour: those rows are not compared further, only counted, and
    the count is returned for the caller to bound (every test here has observed 0)."""
    near = 0
    bad = []
    for r, (g, w, info) in enumerate(zip(got, want, infos)):
        if g == w:
            continue
        if info is not None and info.boundary_dist < BOUNDARY_TOL:
            near += 1
            continue
        bad.append((r, int(g), int(w), None if info is None else info.boundary_dist))
    assert not bad, f"{what}: {len(bad)} rows differ away from any CDF boundary: {bad[:8]}"
    return near
