"""geist_quotient_f32 (geistlib_amd/csrc/exact_quotient.h, compiled here for the host) against
the division it replaces, (float) ((double) p / sum) of src/engine/sampler.c:246-253, bit for
bit on random inputs and on inputs built to fall beside the middle between two binary32
values."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def checker(tmp_path_factory):
    exe = str(tmp_path_factory.mktemp("quotient") / "quotient_check")
    src = os.path.join(HERE, "native", "quotient_check.cpp")
    # -ffp-contract=off: the only fused operations are the two written in the header
    subprocess.run(["g++", "-O2", "-fopenmp", "-mfma", "-ffp-contract=off", "-o", exe, src],
                   check=True)
    return exe


def test_quotient_equals_the_division(checker):
    out = subprocess.run([checker, "200000000", "16"], capture_output=True, text=True, check=True)
    bad, total, beside, tiny = map(int, out.stdout.split())
    assert total == 200_000_000 and bad == 0
    # the hard cases are there: millions of quotients beside a middle, millions of tiny ones,
    # and most cases are neither (they take the short way)
    assert beside > 1_000_000 and tiny > 1_000_000 and beside + tiny < total * 2 // 3
