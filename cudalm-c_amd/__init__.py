"""cudalm-c_amd: MI355X-native implementation of cudalm's QLM 4-bit weight path.

The product is libqlmx.so -- hand-written HIP kernels for gfx950 behind the plain-C ABI declared in
include/qlmx.h -- plus the C++ host mirror of the reference's call surface under host/. This Python
module is a thin ctypes loader used by the tests, bench.py and __graft_entry__.py; it adds no
arithmetic of its own and has no fallback: if the library is missing or no gfx950 device is bound,
every call raises.
"""
from .binding import (Qlmx, QlmxError, GemmProb, SPAN_DTYPE, ACT_F32, ACT_BF16, MATH_F32, MATH_MFMA, MATH_MFMA_F16,  # noqa: F401
                      load, lib_path)
