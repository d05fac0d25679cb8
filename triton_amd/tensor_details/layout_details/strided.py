"""Module path of the reference (tensor_details/layout_details/strided.py); the class lives in tensor_details/layout.py."""
from ..layout import StridedLayout

__all__ = ["StridedLayout"]
