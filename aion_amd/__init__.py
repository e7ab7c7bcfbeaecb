"""aion_amd: MI355X (gfx950) execution backend for aion's quantized-inference hot path.

The product is the C-ABI library built from aion_amd/csrc (declared in include/aion_hip.h).
This package is the thin Python harness over it used by the tests and the roofline bench:
`aion_amd.hip` binds the library with ctypes, `aion_amd.backend` mirrors aion's
backend / device-memory / step vocabulary on top of it.
"""
from .hip import LIB_PATH, AionHipError, load_library  # noqa: F401
