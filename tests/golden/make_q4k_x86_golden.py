#!/usr/bin/env python3
"""Writes tests/golden/q4k_x86_ref_vectors.json from the COMPILED REFERENCE kernel.

Run in a container that has the reference tree mounted:

    make -C oracle ref && python tests/golden/make_q4k_x86_golden.py

The library loaded here is oracle/_ref/libgeist_ref_q4kgemv.so: the reference's own
src/backends/cpu_x86/kernel_q4kx8_gemm_avx512.c (q4kx8_gemv_m1), kernel_q4kx8_gemm_scalar.c and
q4k_to_q4kx8.c, built without fast-math. The JSON holds inputs and the reference's outputs only
(data, no code): Q4_K tables and activation rows as hex, and the logits the reference computed
over the table it interleaved itself."""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
from oracle_lib import load_ref_q4kgemv, random_q4k_table, ref_q4k_gemv_m1  # noqa: E402


def main():
    ref = load_ref_q4kgemv()
    if ref is None:
        sys.exit("oracle/_ref/libgeist_ref_q4kgemv.so is not built (make -C oracle ref)")
    g = np.random.default_rng(40404)
    cases = []
    for n_out, n_in, scale in [(8, 256, 1.0), (16, 512, 0.01), (8, 768, 30.0), (24, 1536, 1.0),
                               (8, 2560, 1e-3)]:
        w = random_q4k_table(g, n_out, n_in)
        x = (g.standard_normal(n_in) * scale).astype(np.float32)
        x[::7] = 0.0
        y = ref_q4k_gemv_m1(ref, w, x, n_in)
        cases.append({"n_out": n_out, "n_in": n_in, "w_hex": w.tobytes().hex(),
                      "x_hex": x.tobytes().hex(), "y_hex": y.tobytes().hex()})
    out = os.path.join(HERE, "q4k_x86_ref_vectors.json")
    with open(out, "w") as f:
        json.dump({"source": "oracle/_ref/libgeist_ref_q4kgemv.so (reference "
                             "kernel_q4kx8_gemm_avx512.c + q4k_to_q4kx8.c)", "cases": cases}, f)
    print("wrote", out, os.path.getsize(out), "bytes")


if __name__ == "__main__":
    main()
