"""MI355X-native approximate-multiplier simulator behind ApproxTrain's op surface.

The compute path is the HIP library ``libamsim.so`` (C ABI: ``include/amsim.h``).
This package is the Python host side: LUT-file loading, the functor-level calls,
and the op / gradient wiring of the reference's Python wrappers, with PyTorch
used only for device memory and streams.
"""
from ._lib import AmsimError, lib_path, load_library  # noqa: F401
from .lut import ApproxMulLut  # noqa: F401
