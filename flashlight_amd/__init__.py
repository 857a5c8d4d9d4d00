"""flashlight_amd — MI355X (gfx950) kernels behind Flashlight's AutogradExtension.

The product is the C ABI in include/flhip.h (flashlight_amd/lib/libflhip.so) and
the C++ host class in flashlight_amd/host/.  This Python package is a thin
ctypes binding of the same C ABI over torch device tensors; it has no CPU path
and raises when the compiled library is missing.
"""
from . import capi  # noqa: F401
from .ops import (  # noqa: F401
    PoolingMode,
    batchnorm,
    batchnorm_backward,
    conv2d,
    conv2d_backward_data,
    conv2d_backward_filter_bias,
    conv2d_backward_filter_bias_static,
    derive_padding,
    pool2d,
    pool2d_backward,
)
