"""geistlib_amd -- MI355X-native token-sampling path behind geistlib's sampler API.

The product is the pair of shared libraries under geistlib_amd/lib (HIP kernels behind a C ABI,
plus a C23 host layer with the reference's own sampler symbols). This Python package only binds
them with ctypes for tests and benchmarks; it contains no sampling arithmetic and no fallback.
"""
from .binding import (HipSampler, SampleParams, SpecResult, load_library,  # noqa: F401
                      library_path, sample_rows_static)
