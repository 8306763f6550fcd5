"""MI355X-native reduction engine with oneCCL's operator surface (ccl::datatype x ccl::reduction).

The product is the shared library ``libmi_ccl_comp.so`` (hand-written HIP kernels for gfx950 behind the C ABI
declared in ``include/mi_ccl_comp.h``) and the C++ operator surface in ``oneccl_amd/csrc/ccl_comp.hpp``.
This Python package is only a thin ctypes binding used by the tests and the benchmark; PyTorch provides
device memory and streams, nothing else.
"""
from . import comp  # noqa: F401
from .comp import *  # noqa: F401,F403
