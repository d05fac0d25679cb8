"""The MXFP4 value layout of the gfx950 kernels (no counterpart in the reference, which keeps value layouts of its
own for Hopper and Blackwell in this directory); the classes live in tensor_details/layout.py."""
from ..layout import CDNA4MXValueLayout, CDNA4MXValueLayoutTransformation

__all__ = ["CDNA4MXValueLayout", "CDNA4MXValueLayoutTransformation"]
