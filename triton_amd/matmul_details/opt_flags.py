"""Tile selection for the grouped matmul and the constraint API of the reference
(matmul_details/opt_flags.py:405-455): constraints live in ContextVars, i.e. per
thread / task, and are read at every matmul call."""
from contextlib import contextmanager
from contextvars import ContextVar
from dataclasses import dataclass
from typing import Optional

_opt_flags_constraints: ContextVar = ContextVar("opt_flags_constraints", default=None)
_opt_flags: ContextVar = ContextVar("opt_flags", default=None)

BLOCK_M_CHOICES = (16, 32, 64, 128)


class InapplicableConstraint(Exception):
    pass


@dataclass
class OptFlags:
    block_m: int
    block_n: int = 256
    block_k: int = 128
    split_k: int = 1
    num_warps: int = 4
    xcd_swizzle: int = 8
    is_persistent: bool = False


def _constraints() -> dict:
    c = _opt_flags_constraints.get()
    return {} if c is None else c


def update_opt_flags_constraints(constraints: dict):
    merged = dict(_constraints())
    merged.update(constraints)
    _opt_flags_constraints.set(merged)


def reset_opt_flags_constraints():
    _opt_flags_constraints.set(None)


@contextmanager
def scoped_opt_flags_constraints(constraints):
    merged = dict(_constraints())
    merged.update(constraints)
    token = _opt_flags_constraints.set(merged)
    try:
        yield
    finally:
        _opt_flags_constraints.reset(token)


def reset_opt_flags():
    _opt_flags.set(None)


def set_opt_flags(opt_flags: OptFlags):
    assert not _constraints(), "setting constraints is incompatible with manual flags override"
    assert _opt_flags.get() is None, "opt_flags already set; please reset to None first"
    _opt_flags.set(opt_flags)


@contextmanager
def scoped_opt_flags(opt_flags: OptFlags):
    token = _opt_flags.set(opt_flags)
    try:
        yield
    finally:
        _opt_flags.reset(token)


# keys the reference accepts on this target (matmul_details/opt_flags.py:71-73); any other key is a caller's mistake
CONSTRAINTS_SUPPORTED = frozenset({"block_m", "block_n", "block_k", "split_k", "is_persistent", "epilogue_subtile",
                                   "idle_sms", "max_allowable_mn", "num_warps", "disable_mx4_block_swap"})


def max_allowable_mn(max_mn: int, m: int, n: int, split_k: int) -> int:
    """split_k only while the output is small (matmul_details/opt_flags.py:37-43)."""
    return 1 if m * n >= max_mn else split_k


def make_opt_flags(m: int, n: int, k: int, n_slices: int, ragged: bool,
                   expected_slice_size: Optional[int] = None, fp8_rows: bool = False) -> OptFlags:
    """Picks BLOCK_M from the expected rows per slice (no device read): the smallest tile, capped at 128, that covers
    the mean and two standard deviations of a slice's size (the sizes of routed slices scatter about like a Poisson
    count), so that nearly every slice is ONE row block: a second block streams the slice's weights a second time,
    which at 16 to 64 rows per slice costs 10 to 40 % (measured on the layer of the reference's bench_mlp).  Row
    blocks of 16 run the weight-streaming kernel, which expands fp8 rows to 16 bits; fp8 rows are faster through the
    tiled kernel's scaled MFMA, whose smallest useful block is 32 (`fp8_rows`).

    Constraints are validated as the reference validates them (opt_flags.py:71-73, 46-50): an unknown key is
    an AssertionError; a known key has to hold for the flags that come out, and since the tile's width, depth
    and wave count are fixed in the kernels (256 columns, 128 K, 4 waves, no persistent kernel, no epilogue
    sub-tiling, no idle CUs) any other value for them raises InapplicableConstraint instead of being dropped."""
    forced = _opt_flags.get()
    if forced is not None:
        return forced
    c = _constraints()
    unsupported = set(c) - CONSTRAINTS_SUPPORTED
    assert not unsupported, f"Given unsupported constraint: {unsupported}"
    if c.get("is_persistent"):
        raise InapplicableConstraint("there is no persistent kernel on gfx950")
    fixed = OptFlags(block_m=0)
    for key, have in (("block_n", fixed.block_n), ("block_k", fixed.block_k), ("num_warps", fixed.num_warps),
                      ("epilogue_subtile", 1), ("idle_sms", 0)):
        want = c.get(key)
        if want is not None and int(want) != have:
            raise InapplicableConstraint(f"{key} is fixed at {have} in the gfx950 kernels (asked for {want})")
    split_k = c.get("split_k")
    split_k = 1 if split_k is None else int(split_k)
    if split_k < 1:
        raise InapplicableConstraint("split_k must be positive")
    if (c.get("max_allowable_mn") or 0) > 0 and c.get("split_k") is not None:
        split_k = max_allowable_mn(int(c["max_allowable_mn"]), m, n, split_k)
    rows = m
    if ragged:
        rows = expected_slice_size if expected_slice_size is not None else max(1, m // max(1, n_slices))
    cover = rows + 2.0 * rows ** 0.5 if ragged else rows
    block_m = next((b for b in BLOCK_M_CHOICES if cover <= b), BLOCK_M_CHOICES[-1])
    if ragged and fp8_rows and block_m == 16:
        block_m = 32
    if c.get("block_m") is not None:
        block_m = int(c["block_m"])
        if block_m not in BLOCK_M_CHOICES:
            raise InapplicableConstraint(f"block_m must be one of {BLOCK_M_CHOICES}")
    return OptFlags(block_m=block_m, split_k=split_k)
