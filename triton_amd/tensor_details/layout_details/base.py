"""Layout interface (mirrors `triton_kernels/tensor_details/layout_details/base.py:1-46`)."""
from __future__ import annotations

from abc import ABC, abstractmethod
from dataclasses import dataclass


@dataclass(frozen=True)
class LayoutTransformation(ABC):
    """Converts between the canonical form (last dim contiguous, fp4 packed along it) and a layout."""
    shape: list
    is_fp4: bool

    @property
    def storage_shape(self) -> list:
        raise NotImplementedError

    @abstractmethod
    def swizzle_data(self, data):
        ...

    @abstractmethod
    def unswizzle_data(self, data):
        ...


@dataclass(frozen=True)
class Layout(ABC):

    def can_preserve_storage_as(self, other: "Layout", rank: int) -> bool:
        return self == other

    def storage_shape(self, shape, is_fp4: bool):
        return self.make_transformation(list(shape), is_fp4).storage_shape

    @abstractmethod
    def make_transformation(self, shape, is_fp4: bool) -> LayoutTransformation:
        ...

    @abstractmethod
    def swizzle_block_shape(self, block_shape):
        ...
