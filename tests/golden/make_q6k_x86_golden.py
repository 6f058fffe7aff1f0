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
from oracle_lib import (load_ref_q6kgemv, load_ref_q6kmn, random_q6k_table,  # noqa: E402
                        ref_q6k_gemv_m1, ref_q6k_linear_mN)


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
    # batches, through the reference's calls in the order of cpu_x86_linear_q6k_resolve and
    # cpu_x86_linear_q6k_mN (oracle/_ref/libgeist_ref_q6kmn.so). On a host with AVX-512 VNNI a
    # table of a multiple of 8 (16) rows goes through w8x8_gemm (w8x16_gemm), other tables through
    # the VNNI kernel with the scalar kernel's expression; this script must run on such a host.
    mn = load_ref_q6kmn()
    if mn is None:
        sys.exit("oracle/_ref/libgeist_ref_q6kmn.so is not built (make -C oracle ref)")
    if os.environ.get("GEIST_FORCE_ISA") or not mn.w8a8_isa_is_vnni():
        sys.exit("the batch cases need a host with AVX-512 VNNI and no GEIST_FORCE_ISA")
    batch_cases = []
    for n_out, n_in, m, scale in [(8, 256, 2, 1.0), (16, 512, 3, 0.01), (24, 768, 8, 30.0),
                                  (12, 256, 4, 1.0), (7, 512, 5, 3.0)]:
        w = random_q6k_table(g, n_out, n_in)
        x = (g.standard_normal((m, n_in)) * scale).astype(np.float32)
        x[:, ::7] = 0.0
        d = np.float32(2.0) ** np.ceil(np.log2(scale) - 3)   # the row's scale: a power of two,
        x[:, 0] = np.float32(127.0) * d                      # so that the ties below are exact
        for k, h in enumerate((0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 63.5, -126.5)):
            x[:, 1 + k] = np.float32(h) * d
        y, lanes = ref_q6k_linear_mN(mn, w, x, n_in)
        batch_cases.append({"n_out": n_out, "n_in": n_in, "m": m, "lanes": bool(lanes),
                            "w_hex": w.tobytes().hex(), "x_hex": x.tobytes().hex(),
                            "y_hex": y.tobytes().hex()})
    out = os.path.join(HERE, "q6k_x86_ref_vectors.json")
    with open(out, "w") as f:
        json.dump({"source": "oracle/_ref/libgeist_ref_q6kgemv.so (reference kernel_q6k_gemv.c); "
                             "batches: oracle/_ref/libgeist_ref_q6kmn.so (q6k_to_w8a8.c, "
                             "kernel_w8a8*.c, kernel_w4a8.c on a VNNI host)",
                   "cases": cases, "batch_cases": batch_cases}, f)
    print("wrote", out, os.path.getsize(out), "bytes")


if __name__ == "__main__":
    main()
