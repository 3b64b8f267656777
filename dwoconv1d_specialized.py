"""Top-level alias so `from dwoconv1d_specialized import DepthwiseOrientedConv1d`
(models/convnext.py:22-23 of the reference, selected there by SPECIALIZED=1) resolves to the same
MI355X implementation: its kernels are already specialised per plane extent when the library is
built, so the general and the specialised module of the reference are one here."""
from oriented1d_amd.dwoconv1d import (  # noqa: F401
    DepthwiseOrientedConv1d,
    _DepthwiseOrientedConv1d,
    oriented_dwconv1d_get_module_from_params,
)

__all__ = ["DepthwiseOrientedConv1d"]
