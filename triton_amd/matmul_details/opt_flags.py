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


def make_opt_flags(m: int, n: int, k: int, n_slices: int, ragged: bool,
                   expected_slice_size: Optional[int] = None) -> OptFlags:
    """Picks BLOCK_M from the expected rows per slice (no device read): the smallest
    tile that covers them, capped at 128, so that ragged slices waste at most one
    partly filled 16-row fragment per block."""
    forced = _opt_flags.get()
    if forced is not None:
        return forced
    c = _constraints()
    for key in ("is_persistent", ):
        if c.get(key):
            raise InapplicableConstraint("there is no persistent kernel on gfx950")
    split_k = c.get("split_k")
    split_k = 1 if split_k is None else int(split_k)
    if split_k < 1:
        raise InapplicableConstraint("split_k must be positive")
    rows = m
    if ragged:
        rows = expected_slice_size if expected_slice_size is not None else max(1, m // max(1, n_slices))
    block_m = next((b for b in BLOCK_M_CHOICES if rows <= b), BLOCK_M_CHOICES[-1])
    if c.get("block_m") is not None:
        block_m = int(c["block_m"])
        if block_m not in BLOCK_M_CHOICES:
            raise InapplicableConstraint(f"block_m must be one of {BLOCK_M_CHOICES}")
    return OptFlags(block_m=block_m, split_k=split_k)
