"""The device expf (geistlib_amd/csrc/glibc_expf.h, compiled here for the host) against libm
expf, bit for bit: every float in [-104, 0] -- the whole domain the sampler feeds it, since
(l - max) * inv_t <= 0 -- plus the positive range and the special values."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def checker(tmp_path_factory):
    exe = str(tmp_path_factory.mktemp("expf") / "expf_check")
    src = os.path.join(HERE, "native", "expf_check.cpp")
    # -ffp-contract=off: the only fused operations are the explicit fma() calls of the header
    subprocess.run(["g++", "-O2", "-fopenmp", "-mfma", "-ffp-contract=off", "-o", exe, src],
                   check=True)
    return exe


def run(exe, lo, hi):
    out = subprocess.run([exe, hex(lo), hex(hi)], capture_output=True, text=True, check=True)
    bad, total = map(int, out.stdout.split())
    return bad, total


def test_every_float_from_minus_104_to_zero(checker):
    bad, total = run(checker, 0x80000000, 0xC2D00000)
    assert total == 0xC2D00000 - 0x80000000 + 1 == 1_120_927_745
    assert bad == 0


def test_below_minus_104_underflows_to_zero_like_libm(checker):
    bad, total = run(checker, 0xC2D00001, 0xC2D00001 + 5_000_000)
    assert bad == 0 and total > 0
    bad, _ = run(checker, 0xFF7F0000, 0xFF800000)      # down to -FLT_MAX and -inf
    assert bad == 0


def test_positive_range_and_specials(checker):
    bad, total = run(checker, 0x00000000, 0x42B20000)  # +0 .. 89: includes the overflow edge
    assert bad == 0 and total > 1_000_000_000
    bad, _ = run(checker, 0x7F7FFFF0, 0x7F800010)      # FLT_MAX, +inf, NaNs
    assert bad == 0
    bad, _ = run(checker, 0xFF800000, 0xFF800010)      # -inf, -NaNs
    assert bad == 0
