#!/usr/bin/env python3
"""Writes tests/golden/q6k_x86_ref_vectors.json from the COMPILED REFERENCE kernel.

Run in a container that has the reference tree mounted:

    make -C oracle ref && python tests/golden/make_q6k_x86_golden.py

The library loaded here is oracle/_ref/libgeist_ref_q6kgemv.so: the reference's own
src/backends/cpu_x86/kernel_q6k_gemv.c (q6k_gemv_m1: int8 activations per super-block, integer
dot products, AVX2), built without fast-math. The JSON holds inputs and the reference's outputs
only (data, no code): Q6_K tables and activation rows as hex and the outputs the reference computed.
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
from oracle_lib import load_ref_q6kgemv, random_q6k_table, ref_q6k_gemv_m1  # noqa: E402


def main():
    ref = load_ref_q6kgemv()
    if ref is None:
        sys.exit("oracle/_ref/libgeist_ref_q6kgemv.so is not built (make -C oracle ref)")
    g = np.random.default_rng(70707)
    cases = []
    for n_out, n_in, scale in [(7, 256, 1.0), (9, 512, 0.01), (5, 1536, 30.0), (4, 2560, 1.0),
                               (6, 768, 1e-20), (3, 256, 0.0)]:
        w = random_q6k_table(g, n_out, n_in)
        x = (g.standard_normal(n_in) * scale).astype(np.float32)
        x[::7] = 0.0
        if n_in >= 512:
            x[256:512] = 0.0          # a super-block of zeros: d = 0, id = 0
        y = ref_q6k_gemv_m1(ref, w, x, n_in)
        cases.append({"n_out": n_out, "n_in": n_in, "w_hex": w.tobytes().hex(),
                      "x_hex": x.tobytes().hex(), "y_hex": y.tobytes().hex()})
    out = os.path.join(HERE, "q6k_x86_ref_vectors.json")
    with open(out, "w") as f:
        json.dump({"source": "oracle/_ref/libgeist_ref_q6kgemv.so (reference kernel_q6k_gemv.c)",
                   "cases": cases}, f)
    print("wrote", out, os.path.getsize(out), "bytes")


if __name__ == "__main__":
    main()
