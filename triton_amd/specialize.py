"""`FnSpecs` names a function fused into a kernel (mirrors `triton_kernels/specialize.py:68-79`).

The reference injects Triton source into its kernels; here the fused functions are compiled into the
HIP kernels and `FnSpecs.name` selects among them ("swiglu" is the one available)."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional


@dataclass(frozen=True)
class FnSpecs:
    name: str
    fn: Optional[object]
    fn_arg_names: tuple = tuple()
    fn_arg_do_not_specialize: tuple = tuple()
    reduction_n: int = 1

    @staticmethod
    def default():
        return FnSpecs("dflt", None, tuple())
