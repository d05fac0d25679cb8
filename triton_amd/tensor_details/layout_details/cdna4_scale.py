"""Module path of the reference (tensor_details/layout_details/cdna4_scale.py); the classes live in
tensor_details/layout.py."""
from ..layout import CDNA4MXScaleLayout, CDNA4MXScaleLayoutTransformation

__all__ = ["CDNA4MXScaleLayout", "CDNA4MXScaleLayoutTransformation"]
