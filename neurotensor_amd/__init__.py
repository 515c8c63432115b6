"""neurotensor_amd -- MI355X (gfx950) backend for NeuroTensor's dense matmult path.

The product is `lib/libntgemm.so` (HIP kernels behind the C ABI of include/ntgemm.h) and
the C++ facade in `nt_compat/`.  This Python package is only the ctypes face of that ABI,
used by the tests and the benchmark: `functional` mirrors nt::functional::{matmult, linear,
conv2d, unfold2d} on torch tensors that live in HBM.
"""
from . import _lib  # noqa: F401
from ._lib import NtgError, load  # noqa: F401
