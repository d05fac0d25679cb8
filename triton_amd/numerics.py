"""Per-tensor ("flex") scale carriers (numerics.py of the reference)."""
from dataclasses import dataclass
from typing import Optional

import torch

MAX_FINITE_FLOAT8E5 = 57344.0
MAX_FINITE_FLOAT8E4NV = 448.0
MAX_FINITE_FLOAT8E4B8 = 240.0


@dataclass(frozen=True)
class BaseFlexData:
    dtype: Optional[torch.dtype] = None

    def view(self, x: torch.Tensor):
        return x if self.dtype is None else x.view(self.dtype)

    def reinterpret(self, x):
        if self.dtype is None or x.dtype.itemsize > 1:
            return x
        return x.view(self.dtype)


@dataclass(frozen=True)
class InFlexData(BaseFlexData):
    scale: Optional[torch.Tensor] = None

    @property
    def is_per_batch(self):
        return False if self.scale is None else len(self.scale) > 1


@dataclass(frozen=True)
class OutFlexData(BaseFlexData):
    expected_scale: Optional[torch.Tensor] = None
    actual_scale: Optional[torch.Tensor] = None
    checksum_scale: Optional[torch.Tensor] = None

    @property
    def is_per_batch(self):
        return False if self.expected_scale is None else len(self.expected_scale) > 1

    def __iter__(self):
        yield self.expected_scale
        yield self.actual_scale
        yield self.checksum_scale
