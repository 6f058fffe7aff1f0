#!/usr/bin/env python3
"""Writes tests/golden/f16_linear_ref_vectors.json from the COMPILED REFERENCE kernels.

Run in a container that has the reference tree mounted:

    make -C oracle ref && python tests/golden/make_f16_linear_golden.py

The library loaded here is oracle/_ref/libgeist_ref_wquant.so: the reference's own
src/backends/cpu_scalar/weight_resolve.c (cpu_scalar_w_quant_m1 / _mN over an F16 table), built
without fast-math. The JSON holds inputs and the reference's outputs only (data, no code): the F16
tables and the activation rows as hex, and the projections the reference computed -- among them
rows whose last quarter cancels a huge first quarter, where the binary32 result hangs on the order of the
double-precision additions.
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
from oracle_lib import load_ref_wquant, ref_f16_linear  # noqa: E402


def cancelling(g, n_out, n_in, m):
    """Tables and activations whose products nearly cancel: large terms of opposite sign around
    a small remainder."""
    q = n_in // 4
    w = (g.standard_normal((n_out, n_in)) * 4).astype(np.float16)
    x = (g.standard_normal((m, n_in)) * 100).astype(np.float32)
    x[:, :q] *= np.float32(2.0 ** 24)       # a huge first quarter ...
    w[:, 3 * q: 4 * q] = -w[:, :q]          # ... that the last quarter takes away again:
    x[:, 3 * q: 4 * q] = x[:, :q]           # the small terms in between are added to a huge sum
    return w, x


def main():
    ref = load_ref_wquant()
    if ref is None:
        sys.exit("oracle/_ref/libgeist_ref_wquant.so is not built (make -C oracle ref)")
    g = np.random.default_rng(161616)
    cases = []
    for n_out, n_in, m, kind in [(6, 64, 1, "random"), (5, 320, 3, "random"), (4, 2560, 2, "random"),
                                 (6, 256, 1, "cancelling"), (5, 1024, 4, "cancelling")]:
        if kind == "random":
            w = (g.standard_normal((n_out, n_in)) * g.choice([0.02, 1.0])).astype(np.float16)
            x = (g.standard_normal((m, n_in)) * g.choice([0.01, 1.0, 300.0])).astype(np.float32)
        else:
            w, x = cancelling(g, n_out, n_in, m)
        y = ref_f16_linear(ref, w.view(np.uint16), x)
        cases.append({"n_out": n_out, "n_in": n_in, "m": m, "kind": kind,
                      "w_hex": w.tobytes().hex(), "x_hex": x.tobytes().hex(),
                      "y_hex": y.tobytes().hex()})
    out = os.path.join(HERE, "f16_linear_ref_vectors.json")
    with open(out, "w") as f:
        json.dump({"source": "oracle/_ref/libgeist_ref_wquant.so (reference weight_resolve.c, "
                             "GEIST_DTYPE_F16)", "cases": cases}, f)
    print("wrote", out, os.path.getsize(out), "bytes")


if __name__ == "__main__":
    main()
