"""MI355X (gfx950) device driver for CaffeConTroll's lowering-based convolution training path.

The product is the C-ABI shared library ``libcct_hip.so`` (declared in ``include/cct_hip.h``)
plus the C++ host layer in ``csrc/`` that mirrors the reference's DeviceDriver / Bridge classes.
This package is the thin Python view used by the tests and the benchmark harness.
"""
from ._lib import CctHipError, load  # noqa: F401
from .driver import HIPDriver  # noqa: F401
