"""The C-ABI libraries load without a GPU and export every function the headers under include/
declare. No compute call is made here."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIBDIR = os.path.join(ROOT, "geistlib_amd", "lib")

HEADERS = {
    "geist_sampler_hip.h": "libgeist_sampler_hip.so",
    "geist_lm_head_hip.h": "libgeist_sampler_hip.so",
    "geist_sampler_dropin.h": "libgeist_sampler_host.so",
    "geist_head_hip.h": "libgeist_sampler_host.so",
}


def declared_functions(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"struct\s+\w+\s*\{.*?\};", "", text, flags=re.S)
    text = re.sub(r"enum\s+\w+\s*\{.*?\};", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(geist_\w+)\s*\(", text)))


@pytest.mark.parametrize("header,lib", sorted(HEADERS.items()))
def test_library_exports_every_declared_symbol(header, lib):
    path = os.path.join(LIBDIR, lib)
    assert os.path.exists(path), f"{path} missing: run __graft_entry__.build()"
    handle = C.CDLL(path)
    names = declared_functions(header)
    assert len(names) >= 8
    missing = [n for n in names if not hasattr(handle, n)]
    assert not missing, f"{lib} lacks {missing}"


def test_no_measurement_code_in_the_product_abi():
    """Timing helpers live in libgeist_bench_hip.so (geistlib_amd/bench/), outside include/."""
    import subprocess
    for header in os.listdir(os.path.join(ROOT, "include")):
        assert not [n for n in declared_functions(header) if "_time_" in n or "bench" in n], header
    for lib in ("libgeist_sampler_hip.so", "libgeist_sampler_host.so"):
        out = subprocess.run(["nm", "-D", "--defined-only", os.path.join(LIBDIR, lib)],
                             capture_output=True, text=True, check=True).stdout
        bad = [l for l in out.splitlines() if "_time_" in l or "plain_read" in l]
        assert not bad, (lib, bad)
    assert os.path.exists(os.path.join(LIBDIR, "libgeist_bench_hip.so"))


def test_reference_symbol_set_is_complete():
    """The nine symbols of the reference's src/engine/sampler.h:34-73."""
    want = {"geist_rng_seed", "geist_rng_next_u64", "geist_rng_next_unit", "geist_sampler_argmax",
            "geist_sampler_temperature", "geist_sampler_workspace_init",
            "geist_sampler_workspace_destroy", "geist_sampler_top_k_ws", "geist_sampler_top_p_ws"}
    assert want <= set(declared_functions("geist_sampler_dropin.h"))


def test_host_rng_needs_no_device(oracle):
    """geist_rng_* are exact integer code on the host: check them against the oracle here."""
    lib = C.CDLL(os.path.join(LIBDIR, "libgeist_sampler_host.so"))
    lib.geist_rng_next_u64.restype = C.c_uint64
    lib.geist_rng_next_unit.restype = C.c_float
    for seed in (0, 1, 42, 0xDEADBEEF, 0xCAFEBABE1234):
        st = C.c_uint64(0)
        lib.geist_rng_seed(C.byref(st), C.c_uint64(seed))
        r = oracle.rng(seed)
        assert st.value == int(r.state)
        for _ in range(50):
            assert lib.geist_rng_next_u64(C.byref(st)) == oracle.next_u64(r)
        for _ in range(50):
            assert lib.geist_rng_next_unit(C.byref(st)) == oracle.next_unit(r)
