"""The drop-in sampler symbols when the device fails. The reference's samplers cannot fail; the
HIP-backed ones report to a handler that the application may replace (default: message and
abort). Runs where there is no GPU, which is the simplest device failure there is; on a machine
with a GPU these tests are skipped."""
import ctypes as C
import os
import subprocess
import sys
import threading

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "geistlib_amd", "lib", "libgeist_sampler_host.so")
HANDLER = C.CFUNCTYPE(None, C.c_char_p, C.c_char_p, C.c_void_p)


def no_gpu():
    torch = pytest.importorskip("torch")
    return torch.cuda.device_count() == 0


@pytest.fixture()
def host():
    if not os.path.exists(LIB):
        pytest.skip("host library not built")
    if not no_gpu():
        pytest.skip("needs a machine without a GPU")
    lib = C.CDLL(LIB)
    lib.geist_sampler_argmax.argtypes = [C.c_size_t, C.POINTER(C.c_float)]
    lib.geist_sampler_argmax.restype = C.c_int32
    lib.geist_sampler_dropin_on_failure.argtypes = [HANDLER, C.c_void_p]
    yield lib
    lib.geist_sampler_dropin_on_failure(HANDLER(0), None)


def test_installed_handler_is_called_and_the_call_returns(host):
    seen = []

    @HANDLER
    def on_failure(what, detail, user):
        seen.append((what.decode(), detail.decode(), user))

    host.geist_sampler_dropin_on_failure(on_failure, C.c_void_p(0x1234))
    x = np.array([1, 5, 2], dtype=np.float32)
    tok = host.geist_sampler_argmax(3, x.ctypes.data_as(C.POINTER(C.c_float)))
    assert tok == -1  # GEIST_SAMPLER_DROPIN_FAILED_TOKEN
    assert len(seen) == 1 and "device workspace" in seen[0][0] and seen[0][2] == 0x1234


def test_handler_runs_on_the_failing_thread_and_threads_end_cleanly(host):
    """Eight short-lived threads fail, report and exit: the thread-specific context that each
    made is released by its destructor (nothing to observe but a clean exit)."""
    seen = []

    @HANDLER
    def on_failure(what, detail, user):
        seen.append(threading.get_ident())

    host.geist_sampler_dropin_on_failure(on_failure, None)
    x = np.zeros(16, dtype=np.float32)
    idents, toks = [], []

    def work():
        idents.append(threading.get_ident())
        for _ in range(2):
            toks.append(host.geist_sampler_argmax(16, x.ctypes.data_as(C.POINTER(C.c_float))))

    for _ in range(8):
        t = threading.Thread(target=work)
        t.start()
        t.join()
    assert toks == [-1] * 16
    assert len(seen) == 16 and set(seen) == set(idents)


def test_default_handler_aborts_with_a_message():
    if not os.path.exists(LIB):
        pytest.skip("host library not built")
    if not no_gpu():
        pytest.skip("needs a machine without a GPU")
    code = (
        "import ctypes as C\n"
        f"lib = C.CDLL({LIB!r})\n"
        "lib.geist_sampler_argmax.argtypes = [C.c_size_t, C.POINTER(C.c_float)]\n"
        "x = (C.c_float * 4)(0, 1, 2, 3)\n"
        "lib.geist_sampler_argmax(4, x)\n")
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120)
    assert r.returncode == -6, (r.returncode, r.stderr)
    assert "geist sampler (HIP)" in r.stderr
