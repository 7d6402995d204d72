"""MI355X (gfx950) implementation of Otter's int8 convolution path.

The product is the C-ABI shared library ``tensor_amd/lib/libotter_hip_int8.so`` (see
``include/otter_hip_int8.h``) and the C++ host layer in ``tensor_amd/host`` that mirrors the Otter
Layer / ConvolutionLayer / Net interface on top of it. ``tensor_amd.capi`` is a thin ctypes binding used by
the tests and the benchmark; device memory and streams come from PyTorch (plumbing only).
"""
from . import capi  # noqa: F401
