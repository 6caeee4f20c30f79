"""Element-type descriptors (mirrors `triton_kernels/tensor_details/dtype.py:1-39`)."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Union


@dataclass(frozen=True)
class IntegerType:
    bitwidth: int
    is_signed: bool


@dataclass(frozen=True)
class FloatType:
    bitwidth_exponent: int
    bitwidth_mantissa: int
    is_signed: bool
    unsigned_zero: bool = False

    @property
    def bitwidth(self) -> int:
        return self.bitwidth_exponent + self.bitwidth_mantissa + (1 if self.is_signed else 0)


DataType = Union[IntegerType, FloatType]

BIT = IntegerType(1, False)
UINT8 = IntegerType(8, False)
INT16 = IntegerType(16, True)
INT32 = IntegerType(32, True)
INT64 = IntegerType(64, True)
FP4 = FloatType(2, 1, True)
FP8_E4M3FN = FloatType(4, 3, True)
FP8_E4M3FNUZ = FloatType(4, 3, True, unsigned_zero=True)
FP8_E5M2 = FloatType(5, 2, True)
FP16 = FloatType(5, 10, True)
BF16 = FloatType(8, 7, True)
FP32 = FloatType(8, 23, True)
FP64 = FloatType(11, 52, True)
