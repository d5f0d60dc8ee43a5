"""MI355X-native quantized GEMM path (GEMMLowp + offset contribution + fixed-point output stage + conv lowering).

The product is the C-ABI shared library built from csrc/ (see include/mi355_gemmlowp.h) and the C++ host layer that
mirrors the arm_compute function classes. This Python package only loads that library for the tests and the
benchmark harness; it contains no arithmetic and no fallback: without the built library every call raises.
"""
from . import capi  # noqa: F401
