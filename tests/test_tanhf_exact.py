"""The device tanhf (geistlib_amd/csrc/glibc_tanhf.h, compiled here for the host) against libm
tanhf, bit for bit, for every binary32 value: the reference's soft-cap is tanhf(x / cap) * cap
(src/archs/transformer/forward/head.c:148-159)."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def checker(tmp_path_factory):
    exe = str(tmp_path_factory.mktemp("tanhf") / "tanhf_check")
    src = os.path.join(HERE, "native", "tanhf_check.cpp")
    # -ffp-contract=off and no -mfma: every operation of the header rounds on its own
    subprocess.run(["g++", "-O2", "-fopenmp", "-ffp-contract=off", "-o", exe, src], check=True)
    return exe


def run(exe, lo, hi):
    out = subprocess.run([exe, hex(lo), hex(hi)], capture_output=True, text=True, check=True)
    bad, total, first = map(int, out.stdout.split())
    return bad, total, first


def test_every_non_negative_float(checker):
    bad, total, first = run(checker, 0x00000000, 0x7F800000)      # +0 .. +inf
    assert total == 0x7F800000 + 1 and bad == 0, hex(first)


def test_every_negative_float(checker):
    bad, total, first = run(checker, 0x80000000, 0xFF800000)      # -0 .. -inf
    assert total == 0x7F800000 + 1 and bad == 0, hex(first)


def test_nans_stay_nans(checker):
    bad, _, _ = run(checker, 0x7F800001, 0x7F800100)
    assert bad == 0
    bad, _, _ = run(checker, 0xFF800001, 0xFF800100)
    assert bad == 0


def test_monotone_over_every_float(checker):
    """tanhf(next float) >= tanhf(float) for every non-negative float (the function is odd by
    construction): the soft-cap tanhf(x / cap) * cap then keeps the order of the logits, which is
    what lets the top-k path select on raw logits and cap only the candidates."""
    out = subprocess.run([checker, hex(0), hex(0x7F800000), "mono"], capture_output=True,
                         text=True, check=True)
    bad, total, first = map(int, out.stdout.split())
    assert total == 0x7F800000 and bad == 0, hex(first)
