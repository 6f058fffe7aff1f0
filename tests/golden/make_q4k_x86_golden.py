#!/usr/bin/env python3
"""Writes tests/golden/q4k_x86_ref_vectors.json from the COMPILED REFERENCE kernel.

Run in a container that has the reference tree mounted:

    make -C oracle ref && python tests/golden/make_q4k_x86_golden.py

The library loaded here is oracle/_ref/libgeist_ref_q4kgemv.so: the reference's own
src/backends/cpu_x86/kernel_q4kx8_gemm_avx512.c (q4kx8_gemv_m1), kernel_q4kx8_gemm_scalar.c,
q4k_to_q4kx8.c and, for batches, q8_kx4.c and kernel_q4kx8_gemm_avx512_full.c, built without
fast-math. The JSON holds inputs and the reference's outputs only
(data, no code): Q4_K tables and activation rows as hex, and the logits the reference computed
over the table it interleaved itself."""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
from oracle_lib import (load_ref_q4kgemv, random_q4k_table, ref_q4k_gemv_m1,  # noqa: E402
                        ref_q4k_linear_mN)


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
    # batches, through the reference's calls in the order of cpu_x86_linear_q4k_mN: row counts
    # that are no multiple of 4 (the decode kernel row by row), multiples of 4 (quantize_q8_Kx4 +
    # the AVX2 kernel) and multiples of 16 over 16 n table rows (the 16 x 16 tiles; this script
    # must run on a host with AVX-512 for those). Every row holds activations that fall exactly
    # between two int8 values, where the two quantisers round differently.
    if not all(f in open("/proc/cpuinfo").read() for f in ("avx512f", "avx512bw", "avx512dq",
                                                           "avx512vl")):
        sys.exit("the batch cases with 16 x 16 tiles need a host with AVX-512")
    if os.environ.get("GEIST_FORCE_ISA"):
        sys.exit("unset GEIST_FORCE_ISA")
    batch_cases = []
    for n_out, n_in, m, scale in [(8, 256, 3, 1.0), (16, 512, 4, 0.01), (8, 768, 8, 30.0),
                                  (16, 512, 16, 1.0), (24, 256, 16, 1.0), (32, 256, 32, 5.0)]:
        w = random_q4k_table(g, n_out, n_in)
        x = (g.standard_normal((m, n_in)) * scale).astype(np.float32)
        x[:, ::7] = 0.0
        d = np.float32(2.0) ** np.ceil(np.log2(scale) - 3)   # the row's scale: a power of two,
        x[:, 0] = np.float32(127.0) * d                      # so that the ties are exact
        for k, h in enumerate((0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 63.5, -126.5)):
            x[:, 1 + k] = np.float32(h) * d
        y = ref_q4k_linear_mN(ref, w, x, n_in)
        batch_cases.append({"n_out": n_out, "n_in": n_in, "m": m,
                            "tiles": bool(m % 16 == 0 and n_out % 16 == 0),
                            "w_hex": w.tobytes().hex(), "x_hex": x.tobytes().hex(),
                            "y_hex": y.tobytes().hex()})
    out = os.path.join(HERE, "q4k_x86_ref_vectors.json")
    with open(out, "w") as f:
        json.dump({"source": "oracle/_ref/libgeist_ref_q4kgemv.so (reference "
                             "kernel_q4kx8_gemm_avx512.c + q4k_to_q4kx8.c; batches: q8_kx4.c + "
                             "kernel_q4kx8_gemm_avx512_full.c on an AVX-512 host)",
                   "cases": cases, "batch_cases": batch_cases}, f)
    print("wrote", out, os.path.getsize(out), "bytes")


if __name__ == "__main__":
    main()
