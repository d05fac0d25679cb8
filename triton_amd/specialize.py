"""Descriptor of a function fused into a kernel (specialize.py:68-79 of the
reference).  The reference splices Triton source; here `name` selects a compiled
epilogue variant and `fn` is unused."""
from dataclasses import dataclass
from typing import Any, Optional


@dataclass(frozen=True)
class FnSpecs:
    name: str
    fn: Optional[Any]
    fn_arg_names: tuple = tuple()
    fn_arg_do_not_specialize: tuple = tuple()
    reduction_n: int = 1

    @staticmethod
    def default():
        return FnSpecs("dflt", None, tuple())
