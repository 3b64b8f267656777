"""Top-level alias so `from dwoconv1d import DepthwiseOrientedConv1d` (models/convnext.py:20
of the reference) resolves to the MI355X implementation when this directory is on sys.path."""
from oriented1d_amd.dwoconv1d import (  # noqa: F401
    DepthwiseOrientedConv1d,
    _DepthwiseOrientedConv1d,
    oriented_dwconv1d_get_module_from_params,
)

__all__ = ["DepthwiseOrientedConv1d"]
