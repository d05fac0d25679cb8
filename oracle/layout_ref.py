"""CPU oracle: the CDNA4 pre-shuffle of MXFP4 weight scales, and the block layout of MXFP4 weight codes that the
gfx950 kernels read (cdna4_value_*: this build's own wire format, no counterpart in the reference; pinned by its
definition worked by hand and by the round trip).  Test infrastructure, never shipped.

Restates, with numpy index arithmetic (no reshape / permute chains, so that it shares no code shape with the
product's torch implementation):
  cdna4_storage_shape       tensor_details/layout_details/cdna4_scale.py:36-54 (padding and storage shape)
  cdna4_swizzle_ref         cdna4_scale.py:56-68  (host-side swizzle_data)
  cdna4_unswizzle_ref       cdna4_scale.py:70-78  (host-side unswizzle_data)
  cdna4_block_unswizzle_ref cdna4_scale.py:81-87  (what the reference's kernel applies to a loaded block)

Pinned by: the storage shapes the reference's tests spell out (tests/test_tensor.py:52-53: (3,254,60) -> [3,8192,2],
(0,64) -> [1,0,2]); the round trip on the shapes of tests/test_tensor_details/test_layout_cdna4.py:23-38; and the fact
that the kernel-side block unswizzle, restated separately from the host-side swizzle, must undo it.
"""
import numpy as np


def cdna4_storage_shape(shape):
    *leading, k_scale, n = shape
    b = int(np.prod(leading)) if leading else 1
    return [b, -(-k_scale // 8) * 8 * 32, -(-n // 32)]


def _offsets(k_scale, n):
    """Byte offset, inside one batch entry's storage, of the scale of (group k, column n)."""
    kp = -(-k_scale // 8) * 8
    k = np.arange(k_scale)[:, None]
    c = np.arange(n)[None, :]
    k8, k2, k4 = k // 8, (k % 8) // 4, k % 4
    nb, n2, n16 = c // 32, (c % 32) // 16, c % 16
    return nb * (kp * 32) + k8 * 256 + k4 * 64 + n16 * 4 + k2 * 2 + n2


def cdna4_swizzle_ref(x: np.ndarray) -> np.ndarray:
    """x: uint8 [..., K_SCALE, N] -> flat storage uint8 [B, N_pad/32 * K_SCALE_pad*32] (block after block); padding
    bytes are zero.  The reference returns the same bytes viewed as [B, K_SCALE_pad*32, N_pad/32] with unit stride
    along the middle axis."""
    *leading, k_scale, n = x.shape
    b, rows, blocks = cdna4_storage_shape(x.shape)
    out = np.zeros((b, rows * blocks), dtype=x.dtype)
    if x.size:
        out[:, _offsets(k_scale, n).ravel()] = x.reshape(b, k_scale * n)
    return out


def cdna4_unswizzle_ref(flat: np.ndarray, shape) -> np.ndarray:
    *leading, k_scale, n = shape
    b = flat.shape[0]
    if k_scale * n == 0:
        return np.zeros(tuple(shape), dtype=flat.dtype)
    return flat[:, _offsets(k_scale, n).ravel()].reshape(*leading, k_scale, n)


def cdna4_block_unswizzle_ref(block: np.ndarray, block_n: int, block_k_scale: int) -> np.ndarray:
    """The kernel-side view (cdna4_scale.py:81-87): a loaded block of `block_n/32 x block_k_scale*32` bytes becomes
    `[block_n, block_k_scale]`.  Written out as loops over the seven factors of the reshape."""
    flat = block.reshape(-1)
    out = np.zeros((block_n, block_k_scale), dtype=block.dtype)
    i = 0
    for nb in range(block_n // 32):
        for k8 in range(block_k_scale // 8):
            for k4 in range(4):
                for n16 in range(16):
                    for k2 in range(2):
                        for n2 in range(2):
                            # permute (0, 5, 3, 1, 4, 2, 6): output order nb, n2, n16, k8, k2, k4
                            out[nb * 32 + n2 * 16 + n16, k8 * 8 + k2 * 4 + k4] = flat[i]
                            i += 1
    return out


# ---------------------------------------------------------------------------------------------------------------------
# MXFP4 value layout of the gfx950 kernels: blocks of (64 columns x 128 K) = 4 KB, [strip][K stage][position][slot]
# ---------------------------------------------------------------------------------------------------------------------
def cdna4_value_storage_shape(shape):
    """Logical [..., K, N] (FP4) -> [B, ceil(N/64), ceil(K/128) * 4096] bytes."""
    *leading, k, n = shape
    b = int(np.prod(leading)) if leading else 1
    return [b, -(-n // 64), -(-k // 128) * 4096]


def cdna4_value_offset(kb: int, n: int, ks_count: int) -> int:
    """Byte offset, inside one matrix's storage, of packed byte `kb` (codes 2 kb and 2 kb + 1) of column `n`."""
    strip, cn = divmod(n, 64)
    c, f = divmod(cn, 2)            # the column pair (2c, 2c + 1) shares c: positions c and 32 + c
    ks, within = divmod(kb, 64)     # K stage of 128 codes = 64 bytes
    part, byte = divmod(within, 16)
    slot = part ^ ((c >> 2) & 3) ^ (2 * f)
    return (strip * ks_count + ks) * 4096 + (32 * f + c) * 64 + slot * 16 + byte


def cdna4_value_swizzle_ref(x: np.ndarray) -> np.ndarray:
    """x: uint8 [..., K/2, N] packed codes -> [B, ceil(N/64), ceil(K/128) * 4096]; padding bytes are zero.  Plain
    loops over every byte (small inputs only)."""
    *leading, kb_count, n_count = x.shape
    b, ns, row = cdna4_value_storage_shape([*leading, kb_count * 2, n_count])
    ks_count = row // 4096
    out = np.zeros((b, ns * row), dtype=np.uint8)
    xb = x.reshape(b, kb_count, n_count)
    for kb in range(kb_count):
        for n in range(n_count):
            out[:, cdna4_value_offset(kb, n, ks_count)] = xb[:, kb, n]
    return out.reshape(b, ns, row)


def cdna4_value_unswizzle_ref(stored: np.ndarray, shape) -> np.ndarray:
    *leading, k, n_count = shape
    b = stored.shape[0]
    ks_count = stored.shape[-1] // 4096
    flat = stored.reshape(b, -1)
    out = np.zeros((b, k // 2, n_count), dtype=np.uint8)
    for kb in range(k // 2):
        for n in range(n_count):
            out[:, kb, n] = flat[:, cdna4_value_offset(kb, n, ks_count)]
    return out.reshape(*leading, k // 2, n_count)
