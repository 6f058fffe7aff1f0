"""ctypes binding of geistlib_amd/bench/geist_bench_hip.h: timing helpers for bench.py. They live
in their own library (libgeist_bench_hip.so); the product libraries hold no measurement code."""
import ctypes as C

from .binding import GeistHipError, Rows, SampleParams, library_path, load_library, _ptr

_LIB = None


def _lib():
    global _LIB
    if _LIB is None:
        load_library()   # the product library first: the bench library links against it
        lib = C.CDLL(library_path("libgeist_bench_hip.so"))
        vp, sz, i32 = C.c_void_p, C.c_size_t, C.c_int
        lib.geist_bench_timer_begin.argtypes = [vp, C.POINTER(vp)]
        lib.geist_bench_timer_end.argtypes = [vp, C.POINTER(C.c_double)]
        lib.geist_bench_time_stream_kernel.argtypes = [vp, vp, C.POINTER(Rows), sz,
                                                       C.POINTER(SampleParams), vp, vp, i32,
                                                       C.POINTER(C.c_double), C.c_char_p, sz]
        lib.geist_bench_time_plain_read.argtypes = [vp, C.POINTER(Rows), sz, i32, i32,
                                                    C.POINTER(C.c_double)]
        lib.geist_bench_step_latency.argtypes = [vp, C.POINTER(Rows), sz, C.POINTER(SampleParams),
                                                 vp, vp, i32, i32, C.POINTER(C.c_double)]
        _LIB = lib
    return _LIB


class Timer:
    """HIP events on `stream` (None = the default stream) around whatever is enqueued inside the
    `with` block; .ms afterwards."""

    def __init__(self, stream=None):
        self.stream, self.h, self.ms = stream, C.c_void_p(), None

    def __enter__(self):
        rc = _lib().geist_bench_timer_begin(self.stream, C.byref(self.h))
        if rc:
            raise GeistHipError(rc, "geist_bench_timer_begin")
        return self

    def __exit__(self, *exc):
        ms = C.c_double()
        rc = _lib().geist_bench_timer_end(self.h, C.byref(ms))
        if rc and exc[0] is None:
            raise GeistHipError(rc, "geist_bench_timer_end")
        self.ms = ms.value
        return False


def time_stream_kernel(sampler, rows_list, params, uniforms, out, launches, stream=None):
    """(mean microseconds, kernel name) of the logit-streaming kernel of the configuration alone,
    launch i reading rows_list[i % len(rows_list)]."""
    arr = (Rows * len(rows_list))(*rows_list)
    ms = C.c_double()
    name = C.create_string_buffer(64)
    rc = _lib().geist_bench_time_stream_kernel(sampler.h, stream, arr, len(rows_list),
                                               C.byref(params), _ptr(uniforms), _ptr(out),
                                               int(launches), C.byref(ms), name, len(name))
    if rc:
        raise GeistHipError(rc, sampler.lib.geist_hip_sampler_last_error(sampler.h).decode())
    return ms.value * 1e3 / launches, name.value.decode()


def step_latency(sampler, rows_list, params, uniforms, out, samples, wait_ids):
    """Microseconds of `samples` single steps, each from before geist_hip_sample_rows to after
    geist_hip_sampler_wait_ids (wait_ids=True) or geist_hip_sampler_sync, timed in C."""
    arr = (Rows * len(rows_list))(*rows_list)
    us = (C.c_double * samples)()
    rc = _lib().geist_bench_step_latency(sampler.h, arr, len(rows_list), C.byref(params),
                                         _ptr(uniforms), _ptr(out), int(bool(wait_ids)),
                                         int(samples), us)
    if rc:
        raise GeistHipError(rc, sampler.lib.geist_hip_sampler_last_error(sampler.h).decode())
    return list(us)


def time_plain_read(rows_list, launches, streamed, stream=None):
    """Mean microseconds of a kernel that only reads the rows (calibration)."""
    arr = (Rows * len(rows_list))(*rows_list)
    ms = C.c_double()
    rc = _lib().geist_bench_time_plain_read(stream, arr, len(rows_list), int(bool(streamed)),
                                            int(launches), C.byref(ms))
    if rc:
        raise GeistHipError(rc, "geist_bench_time_plain_read")
    return ms.value * 1e3 / launches
