"""MI355X-native depthwise oriented 1D convolution (gfx950 HIP kernels behind a C ABI).

``DepthwiseOrientedConv1d`` mirrors the operator module of the reference
(models/dwoconv1d/dwoconv1d.py:92-198); everything it computes runs in
``libdwoconv1d_hip.so``.  There is no CPU path: importing works anywhere, calling the
operator requires the built library and a GPU.
"""
from .dwoconv1d import (  # noqa: F401
    DepthwiseOrientedConv1d,
    _DepthwiseOrientedConv1d,
    oriented_dwconv1d_get_module_from_params,
)

__all__ = ["DepthwiseOrientedConv1d"]
