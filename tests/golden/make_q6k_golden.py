#!/usr/bin/env python3
"""Writes tests/golden/q6k_ref_vectors.json from the COMPILED REFERENCE kernels.

Run in a container that has the reference tree mounted:

    make -C oracle ref && python tests/golden/make_q6k_golden.py

The library loaded here is oracle/_ref/libgeist_ref_wquant.so: the reference's own
src/backends/cpu_scalar/weight_resolve.c and src/formats/gguf/q6_K.c, built without fast-math.
The JSON holds inputs and the reference's outputs only (data, no code): Q6_K tables as hex, the
activation rows as hex, the dequantised first rows and the projections the reference computed.
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
from oracle_lib import load_ref_wquant, random_q6k_table, ref_q6k_linear, _fp  # noqa: E402
import ctypes as C  # noqa: E402


def main():
    ref = load_ref_wquant()
    if ref is None:
        sys.exit("oracle/_ref/libgeist_ref_wquant.so is not built (make -C oracle ref)")
    g = np.random.default_rng(60606)
    cases = []
    for n_out, n_in, m in [(5, 256, 1), (9, 512, 1), (7, 768, 3), (4, 1536, 2)]:
        w = random_q6k_table(g, n_out, n_in)
        x = (g.standard_normal((m, n_in)) * g.choice([0.01, 1.0, 30.0])).astype(np.float32)
        x[0, ::7] = 0.0
        y = ref_q6k_linear(ref, w, x, n_in)
        row0 = np.empty(n_in, dtype=np.float32)
        ref.dequant_q6_K_row(w[0].ctypes.data_as(C.c_void_p), _fp(row0), n_in)
        cases.append({"n_out": n_out, "n_in": n_in, "m": m, "w_hex": w.tobytes().hex(),
                      "x_hex": x.tobytes().hex(), "y_hex": y.tobytes().hex(),
                      "dequant_row0_hex": row0.tobytes().hex()})
    # activations that are not finite: an infinity, two of opposite sign in one row (their
    # products meet as inf - inf wherever the weights' signs agree), a NaN
    n_out, n_in, m = 12, 512, 3
    w = random_q6k_table(g, n_out, n_in, scale_mode="plain")
    x = g.standard_normal((m, n_in)).astype(np.float32)
    x[0, 5] = np.inf
    x[1, 9], x[1, 300] = -np.inf, np.inf
    x[2, 17] = np.nan
    y = ref_q6k_linear(ref, w, x, n_in)
    row0 = np.empty(n_in, dtype=np.float32)
    ref.dequant_q6_K_row(w[0].ctypes.data_as(C.c_void_p), _fp(row0), n_in)
    cases.append({"n_out": n_out, "n_in": n_in, "m": m, "w_hex": w.tobytes().hex(),
                  "x_hex": x.tobytes().hex(), "y_hex": y.tobytes().hex(),
                  "dequant_row0_hex": row0.tobytes().hex(), "not_finite": True})
    out = os.path.join(HERE, "q6k_ref_vectors.json")
    with open(out, "w") as f:
        json.dump({"source": "oracle/_ref/libgeist_ref_wquant.so (reference weight_resolve.c + q6_K.c)",
                   "cases": cases}, f)
    print("wrote", out, os.path.getsize(out), "bytes")


if __name__ == "__main__":
    main()
