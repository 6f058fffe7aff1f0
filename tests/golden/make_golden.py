#!/usr/bin/env python3
"""Writes tests/golden/sampler_ref_vectors.json from the COMPILED REFERENCE sampler.

Run in a container that has the reference tree mounted:

    make -C oracle ref && python tests/golden/make_golden.py

The library loaded here is oracle/_ref/libgeist_ref_sampler.so, i.e. the reference's own
src/engine/sampler.c + src/base/heap.c built without fast-math. The JSON holds inputs and the
reference's outputs only (data, no code): RNG streams, token-id sequences for the four sampling
modes on small rows stored in full, and on vocabulary-sized rows regenerated from a numpy seed
(a SHA-256 of the row guards against a numpy that generates different bits).
"""
import ctypes as C
import hashlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
from oracle_lib import OracleRng, RefWorkspace, load_ref, _fp  # noqa: E402

SEEDS = [0, 1, 7, 11, 13, 17, 42, 99, 0xDEADBEEF, 0xC0FFEE, 0xCAFEBABE1234]
N_DRAWS = 24


def hexrow(a):
    return np.ascontiguousarray(a, dtype=np.float32).tobytes().hex()


def small_rows():
    rng = np.random.default_rng(20240607)
    rows = {}
    # the reference's own unit-test rows (tests/test_sampler_unit.c:34,43,57,66,96,120,141)
    rows["unit_argmax"] = np.array([-1, 2, .5, 3, 3, -.5], dtype=np.float32)
    rows["unit_peaked"] = np.array([0, 0, 0, 10, 0], dtype=np.float32)
    rows["unit_t0"] = np.array([1, 2, 3, .5], dtype=np.float32)
    rows["unit_uniform"] = np.zeros(5, dtype=np.float32)
    rows["unit_topk"] = np.array([0, 1, 4, 2, 5, 1.5, 0, .5], dtype=np.float32)
    rows["unit_topp"] = np.array([10, 0, 0, 0, 0], dtype=np.float32)
    rows["unit_ws"] = np.array([.1, .2, .3, 5, .1, 0, 0, 0], dtype=np.float32)
    rows["gauss64"] = (rng.standard_normal(64) * 2).astype(np.float32)
    rows["gauss1000"] = (rng.standard_normal(1000) * 2).astype(np.float32)
    # > 1024 entries takes the reference's heap path; quantised values force many exact ties
    rows["ties1500"] = (np.round(rng.standard_normal(1500) * 4) / 4).astype(np.float32)
    rows["gauss3000"] = (rng.standard_normal(3000) * 3).astype(np.float32)
    # > 8192 takes the heap path of the temperature sampler too
    rows["ties9000"] = (np.round(rng.standard_normal(9000) * 8) / 8).astype(np.float32)
    rows["allequal300"] = np.full(300, 1.25, dtype=np.float32)
    return rows


def big_rows():
    out = {}
    g = np.random.default_rng(1234)
    out["v128256_s2"] = (g.standard_normal(128256) * 2).astype(np.float32)
    g = np.random.default_rng(4321)
    r = (g.standard_normal(128256) * 2).astype(np.float32)
    r[g.integers(0, 128256, 5)] += 10
    out["v128256_boost"] = r
    g = np.random.default_rng(99)
    out["v151936_q"] = (np.round(g.standard_normal(151936) * 2 * 64) / 64).astype(np.float32)
    return out


MODES = [
    ("argmax", {}),
    ("temperature", {"t": 0.8}), ("temperature", {"t": 0.1}), ("temperature", {"t": 0.0}),
    ("top_k", {"k": 2, "t": 1.0}), ("top_k", {"k": 3, "t": 1.0}), ("top_k", {"k": 40, "t": 0.7}),
    ("top_k", {"k": 1, "t": 1.0}), ("top_k", {"k": 100000000, "t": 0.9}),
    ("top_k", {"k": 200, "t": 10.0}),
    ("top_p", {"p": 0.5, "t": 1.0}), ("top_p", {"p": 0.9, "t": 0.7}), ("top_p", {"p": 0.95, "t": 1.0}),
    ("top_p", {"p": 1.0, "t": 0.7}), ("top_p", {"p": 0.0, "t": 0.7}), ("top_p", {"p": 0.05, "t": 2.0}),
]


def run_mode(lib, row, mode, prm, seed, n_draws):
    rng = OracleRng()
    lib.geist_rng_seed(C.byref(rng), C.c_uint64(seed))
    ws = RefWorkspace()
    assert lib.geist_sampler_workspace_init(C.byref(ws), row.size) == 0
    toks = []
    for _ in range(n_draws):
        if mode == "argmax":
            t = lib.geist_sampler_argmax(row.size, _fp(row))
        elif mode == "temperature":
            t = lib.geist_sampler_temperature(row.size, _fp(row), prm["t"], C.byref(rng))
        elif mode == "top_k":
            t = lib.geist_sampler_top_k_ws(C.byref(ws), _fp(row), prm["k"], prm["t"], C.byref(rng))
        else:
            t = lib.geist_sampler_top_p_ws(C.byref(ws), _fp(row), prm["p"], prm["t"], C.byref(rng))
        toks.append(int(t))
    lib.geist_sampler_workspace_destroy(C.byref(ws))
    return toks, int(rng.state)


def main():
    lib = load_ref()
    if lib is None:
        sys.exit("build the reference first: make -C oracle ref")
    doc = {"source": "reference src/engine/sampler.c + src/base/heap.c, clang -std=c23 -O2 "
                     "-ffp-contract=off, glibc 2.35", "rng": [], "small": [], "big": []}
    for s in SEEDS:
        r = OracleRng()
        lib.geist_rng_seed(C.byref(r), C.c_uint64(s))
        st0 = int(r.state)
        u64 = [int(lib.geist_rng_next_u64(C.byref(r))) for _ in range(8)]
        units = [float(lib.geist_rng_next_unit(C.byref(r))).hex() for _ in range(4)]
        doc["rng"].append({"seed": s, "state0": st0, "u64": u64, "unit_after": units})
    for name, row in small_rows().items():
        cases = []
        for mode, prm in MODES:
            for seed in (7, 0xC0FFEE):
                toks, st = run_mode(lib, row, mode, prm, seed, N_DRAWS)
                cases.append({"mode": mode, "prm": prm, "seed": seed, "tokens": toks,
                              "state_after": st})
        doc["small"].append({"name": name, "n": int(row.size), "row_hex": hexrow(row),
                             "cases": cases})
    for name, row in big_rows().items():
        cases = []
        for mode, prm in MODES:
            if mode == "top_k" and prm["k"] == 100000000:
                continue  # same as the temperature case at this size
            toks, st = run_mode(lib, row, mode, prm, 0xDEADBEEF, 6)
            cases.append({"mode": mode, "prm": prm, "seed": 0xDEADBEEF, "tokens": toks,
                          "state_after": st})
        doc["big"].append({"name": name, "n": int(row.size),
                           "sha256": hashlib.sha256(row.tobytes()).hexdigest(), "cases": cases})
    # the reference unit test's check 4: exact bucket counts for 5000 draws (seed 7, T = 1)
    row = np.zeros(5, dtype=np.float32)
    toks, _ = run_mode(lib, row, "temperature", {"t": 1.0}, 7, 5000)
    doc["unit_check4_counts"] = [toks.count(i) for i in range(5)]
    with open(os.path.join(HERE, "sampler_ref_vectors.json"), "w") as f:
        json.dump(doc, f, separators=(",", ":"))
    print("wrote", os.path.join(HERE, "sampler_ref_vectors.json"))


if __name__ == "__main__":
    main()
