"""Storage layouts.  Values use the strided layout (which axis is contiguous / packed; see
tensor_details/layout_details/strided.py of the reference for the ordering rule reproduced by
`StridedLayout.order`).  Weight scales may also come pre-shuffled for CDNA4
(`CDNA4MXScaleLayout`, reference tensor_details/layout_details/cdna4_scale.py:11-77), which is what
`make_default_matmul_mxfp4_w_scale_layout` selects on this target (reference tensor_details/layout.py:43-54)."""
import math
from dataclasses import dataclass

import torch


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
    """What the reference returns on AMD hardware (tensor_details/layout.py:27-40): codes contiguous along K.  The
    kernels read that layout as it is; `CDNA4MXValueLayout` below is the layout they read fastest."""
    return StridedLayout(-2)


@dataclass(frozen=True)
class CDNA4MXValueLayoutTransformation:
    """MXFP4 weight codes `[..., K, N]` (two codes per byte along K) in the order the gfx950 matmul kernels copy them:
    the counterpart, for this target, of the value layouts the reference keeps for Hopper and Blackwell
    (tensor_details/layout.py:26-41, layout_details/blackwell_value_shuffled.py).

    N is cut into strips of 64 columns and K into stages of 128; a (strip, stage) block is 4 KB, the blocks of a
    strip follow each other along K, the strips of a matrix follow each other along N, K and N are padded with zero
    codes.  Inside a block the column `n = 2 c + f` of the strip (c < 32: a gate / linear column pair shares c) is
    position `p = 32 f + c`, 64 bytes each; the position's four 16-byte parts (32 codes each, K ascending) sit in
    slots `part ^ ((c >> 2) & 3) ^ 2 f`.  A block is the image one wave of the tiled kernels holds in LDS for a K
    stage -- rotated so that its operand reads meet no bank conflicts -- so a wave copies it with four 1 KB requests of
    whole, aligned lines; the 16 consecutive columns a unit of the decode kernel streams are two runs of 512 bytes per
    stage.  (With K contiguous per column, the layout `downcast_to_mxfp` produces, a stage of a column is 64 bytes
    and a request touches 16 half lines: measured on MI355X such requests move 3.2 TB/s from HBM where whole-line runs
    move over 8.)"""
    shape: tuple
    is_fp4: bool = True

    def __post_init__(self):
        assert self.is_fp4, "the value layout holds packed e2m1 codes"
        *leading, k, n = self.shape
        assert k % 2 == 0, "two codes per byte along K"
        object.__setattr__(self, "leading_shape", list(leading))
        object.__setattr__(self, "B", math.prod(leading))
        object.__setattr__(self, "K", k)
        object.__setattr__(self, "N", n)
        object.__setattr__(self, "KS", -(-k // 128))
        object.__setattr__(self, "NS", -(-n // 64))

    @property
    def storage_shape(self):
        return [self.B, self.NS, self.KS * 4096]

    @staticmethod
    def _part_of_slot(device):
        f = torch.arange(2, device=device)[:, None, None]
        c = torch.arange(32, device=device)[None, :, None]
        s = torch.arange(4, device=device)[None, None, :]
        return f, c, s ^ ((c >> 2) & 3) ^ (2 * f)   # an involution: the same table maps slots to parts and back

    def swizzle_data(self, data):
        """`data`: uint8 `[..., K/2, N]` (low nibble = even k), any strides."""
        B, KS, NS = self.B, self.KS, self.NS
        x = data.reshape(B, self.K // 2, self.N)
        x = torch.nn.functional.pad(x, (0, NS * 64 - self.N, 0, KS * 64 - self.K // 2))
        x = x.reshape(B, KS, 4, 16, NS, 32, 2)                       # b, ks, part, byte, strip, c, f
        x = x.permute(0, 4, 1, 6, 5, 2, 3)                            # b, strip, ks, f, c, part, byte
        f, c, part = self._part_of_slot(x.device)
        out = x[:, :, :, f, c, part, :].reshape(B, NS, KS * 4096).contiguous()
        assert list(out.shape) == self.storage_shape
        return out

    def unswizzle_data(self, data):
        """Back to uint8 `[..., K/2, N]` with unit stride along K."""
        B, KS, NS = self.B, self.KS, self.NS
        x = data.reshape(B, NS, KS, 2, 32, 4, 16)                    # b, strip, ks, f, c, slot, byte
        f, c, slot = self._part_of_slot(x.device)
        x = x[:, :, :, f, c, slot, :]                                # ... f, c, part, byte
        x = x.permute(0, 1, 4, 3, 2, 5, 6).reshape(B, NS * 64, KS * 64)[:, :self.N, :self.K // 2]
        return x.contiguous().transpose(-1, -2).reshape(*self.leading_shape, self.K // 2, self.N)


@dataclass(frozen=True)
class CDNA4MXValueLayout(Layout):
    """Selects `CDNA4MXValueLayoutTransformation`: `convert_layout(w, CDNA4MXValueLayout())` for FP4 weights."""

    @property
    def name(self):
        return "CDNA4_VALUE"

    def make_transformation(self, shape, is_fp4: bool = True):
        return CDNA4MXValueLayoutTransformation(tuple(shape), is_fp4)

    def storage_shape(self, shape, is_fp4: bool = True):
        return self.make_transformation(shape, is_fp4).storage_shape


def make_native_matmul_mxfp4_w_layout(mx_axis: int = 1, **_):
    """The value layout the gfx950 kernels read fastest (no counterpart in the reference, whose AMD path keeps the
    strided layout)."""
    return CDNA4MXValueLayout()


@dataclass(frozen=True)
class CDNA4MXScaleLayoutTransformation:
    """Pre-shuffle of e8m0 scales `[..., K/32, N]` for CDNA4 (reference cdna4_scale.py:32-77).

    K/32 is padded to a multiple of 8 and N to a multiple of 32 (with zeros).  Columns are cut into blocks of 32;
    a block's scales are one contiguous run of `K_SCALE_pad * 32` bytes in which the scale of group
    `k = 8*k8 + 4*k2 + k4` of column `n = 32*nb + 16*n2 + n16` sits at byte

        256*k8 + 64*k4 + 4*n16 + 2*k2 + n2

    so that one dword holds, for one column pair (n16, n16 + 16), the groups k4 and k4 + 4: the four scale bytes a
    lane of a 16-wide scaled MFMA selects from with op_sel.  Storage is `[B, K_SCALE_pad * 32, N_pad / 32]` with unit
    stride along the middle axis, i.e. block after block in memory."""
    shape: tuple
    is_fp4: bool = False

    def __post_init__(self):
        assert not self.is_fp4, "scales are bytes"
        *leading, k_scale, n = self.shape
        object.__setattr__(self, "leading_shape", list(leading))
        object.__setattr__(self, "B", math.prod(leading))
        object.__setattr__(self, "K_SCALE", k_scale)
        object.__setattr__(self, "N", n)
        object.__setattr__(self, "K_SCALE_pad", -(-k_scale // 8) * 8)
        object.__setattr__(self, "N_pad", -(-n // 32) * 32)

    @property
    def storage_shape(self):
        return [self.B, self.K_SCALE_pad * 32, self.N_pad // 32]

    def swizzle_data(self, data):
        """`data`: `[..., K_SCALE, N]`, any strides."""
        B, kp, npad = self.B, self.K_SCALE_pad, self.N_pad
        x = data.reshape(B, self.K_SCALE, self.N)
        x = torch.nn.functional.pad(x, (0, npad - self.N, 0, kp - self.K_SCALE))
        x = x.reshape(B, kp // 8, 2, 4, npad // 32, 2, 16)  # b, k8, k2, k4, nb, n2, n16
        x = x.permute(0, 4, 1, 3, 6, 2, 5).contiguous()      # b, nb, k8, k4, n16, k2, n2
        out = x.reshape(B, npad // 32, kp * 32).transpose(-1, -2)
        assert list(out.shape) == self.storage_shape
        return out

    def unswizzle_data(self, data):
        """Back to a contiguous `[..., K_SCALE, N]`."""
        B, kp, npad = self.B, self.K_SCALE_pad, self.N_pad
        x = data.transpose(-1, -2).reshape(B, npad // 32, kp // 8, 4, 16, 2, 2)  # b, nb, k8, k4, n16, k2, n2
        x = x.permute(0, 2, 5, 3, 1, 6, 4)                                        # b, k8, k2, k4, nb, n2, n16
        x = x.reshape(B, kp, npad)[:, :self.K_SCALE, :self.N]
        return x.reshape(*self.leading_shape, self.K_SCALE, self.N).contiguous()


@dataclass(frozen=True)
class CDNA4MXScaleLayout(Layout):

    @property
    def name(self):
        return "CDNA4_SCALE"

    def make_transformation(self, shape, is_fp4: bool = False):
        return CDNA4MXScaleLayoutTransformation(tuple(shape), is_fp4)

    def storage_shape(self, shape, is_fp4: bool = False):
        return self.make_transformation(shape, is_fp4).storage_shape

    def swizzle_block_shape(self, block_shape):
        scale_k, n = block_shape[-2], block_shape[-1]
        return list(block_shape[:-2]) + [n // 32, scale_k * 32]


def make_default_matmul_mxfp4_w_scale_layout(mx_axis: int, num_warps: int = 8):
    return CDNA4MXScaleLayout()
