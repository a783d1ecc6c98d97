"""MI355X (gfx950) backend for riftco-transformer's packed NF4 linear path.

The product is `lib/librthip.so` (hand-written HIP kernels behind the C ABI of
`include/rthip.h`) and the C++ `hip` backend adapter under `backend/`.  The
Python modules here are thin plumbing over that ABI for tests and measurement.
"""
from .binding import (  # noqa: F401
    ALGORITHM_AUTO,
    ALGORITHM_GEMV,
    ALGORITHM_GENERIC,
    ALGORITHM_MFMA,
    ALGORITHM_NAMES,
    ALGORITHM_RESIDENT,
    ALGORITHM_SKINNY,
    EXPORTED_SYMBOLS,
    FORWARD,
    INPUT_BACKWARD,
    LIBRARY_PATH,
    SCALE_DOUBLE_QUANTIZED_UINT8,
    SCALE_FLOAT32,
    DeviceWeight,
    InvalidArgument,
    Library,
    Overflow,
    RthipError,
    Unavailable,
    Unsupported,
    load_library,
)
