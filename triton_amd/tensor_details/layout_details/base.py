"""Module path of the reference (tensor_details/layout_details/base.py); the classes live in tensor_details/layout.py."""
from ..layout import Layout

__all__ = ["Layout"]
