"""Storage layouts.  Only the strided layout (which axis is contiguous / packed)
is needed on gfx950 for values; see tensor_details/layout_details/strided.py of
the reference for the ordering rule reproduced by `StridedLayout.order`."""
from dataclasses import dataclass


@dataclass(frozen=True)
class Layout:
    @property
    def name(self):
        raise NotImplementedError


@dataclass(frozen=True)
class StridedLayout(Layout):
    """`major_dim` is the contiguous (and, for FP4, packed) axis; the remaining
    axes keep row-major order with the last axis taking the place of major_dim."""
    major_dim: int = -1

    @property
    def name(self):
        return "STRIDED"

    def order(self, rank: int):
        """Axes from fastest to slowest varying."""
        if rank <= 0:
            return []
        if not -rank <= self.major_dim < rank:
            raise ValueError(f"major_dim {self.major_dim} out of range for rank {rank}")
        major = self.major_dim % rank
        dims = list(range(rank - 1, -1, -1))
        at = dims.index(major)
        dims[0], dims[at] = dims[at], dims[0]
        return dims

    def storage_shape(self, shape, is_fp4: bool):
        shape = list(shape)
        if is_fp4 and shape:
            d = self.order(len(shape))[0]
            if shape[d] % 2:
                raise ValueError(f"FP4 packing axis {d} must have even size, got {shape[d]}")
            shape[d] //= 2
        return shape

    def strides(self, storage_shape):
        strides = [0] * len(storage_shape)
        run = 1
        for d in self.order(len(storage_shape)):
            strides[d] = run
            run *= storage_shape[d]
        return strides


def make_default_matmul_mxfp4_w_layout(mx_axis: int, **_):
    return StridedLayout(-2)


def make_default_matmul_mxfp4_w_scale_layout(mx_axis: int, num_warps: int = 8):
    return StridedLayout(-2)
