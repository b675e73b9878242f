"""MI355X-native static autodiff: host-side access to the GPU hot path.

The product is the header-only C++20/HIP library under include/xyz_autodiff/ and
the kernels built on it (csrc/), exposed through the C ABI of libxad_hip.so
(include/xad_capi.h).  This package is the thin Python host layer used by the
tests and the benchmark; PyTorch only provides device memory and streams.
"""
from . import _lib  # noqa: F401
from ._lib import XadError, load  # noqa: F401
