"""MI355X-native FFT library behind the rocfft.h C interface.

The product is ``rocfft_amd/lib/librocfft_amd.so`` (C++ planner + hand-written
gfx950 kernels, built by ``__graft_entry__.build()``).  This package is a thin
ctypes mirror of that C interface, used by the tests and the benchmark; it adds
no computation of its own and raises if the shared library is missing.
"""
from .binding import (  # noqa: F401
    Library,
    Plan,
    PlanDescription,
    ExecutionInfo,
    RocfftError,
    library,
    library_path,
    STATUS,
    COMPLEX_FORWARD,
    COMPLEX_INVERSE,
    REAL_FORWARD,
    REAL_INVERSE,
    SINGLE,
    DOUBLE,
    HALF,
    INPLACE,
    NOTINPLACE,
    COMPLEX_INTERLEAVED,
    COMPLEX_PLANAR,
    REAL,
    HERMITIAN_INTERLEAVED,
    HERMITIAN_PLANAR,
    UNSET,
)
