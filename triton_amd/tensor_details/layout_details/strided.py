"""Plain strided layout: only the unit-stride ("major") dimension is recorded.

Mirrors `triton_kernels/tensor_details/layout_details/strided.py:8-98` and the nibble `repack` of
`layout_details/torch_utils.py:44-91`.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from .base import Layout, LayoutTransformation


def repack(data: torch.Tensor, old_dim: int, new_dim: int, is_fp4: bool, out: torch.Tensor | None = None):
    """Moves the fp4 packing (two nibbles per byte, even index low) from `old_dim` to `new_dim`."""
    old_dim %= data.ndim
    new_dim %= data.ndim
    if not is_fp4 or old_dim == new_dim:
        if out is None:
            return data
        out.copy_(data)
        return out
    if data.dtype.is_floating_point:
        raise TypeError(f"Expected integer dtype for bitwise ops, got {data.dtype}")
    shape = list(data.shape)
    shape[old_dim] *= 2
    shape[new_dim] //= 2
    if out is None:
        out = torch.empty(shape, dtype=data.dtype, device=data.device)

    def sel(ndim, dim, start):
        idx = [slice(None)] * ndim
        idx[dim] = slice(start, None, 2)
        return tuple(idx)

    # a/b: source bytes at even/odd positions of the new packing dim; each holds two nibbles that
    # belong to positions 2i (low) and 2i+1 (high) of the old packing dim.
    a = data[sel(data.ndim, new_dim, 0)]
    b = data[sel(data.ndim, new_dim, 1)]
    out[sel(out.ndim, old_dim, 0)] = (a & 0x0F) | ((b & 0x0F) << 4)
    out[sel(out.ndim, old_dim, 1)] = (a >> 4) | (b & 0xF0)
    return out


@dataclass(frozen=True)
class StridedLayout(Layout):
    major_dim: int = -1

    def __post_init__(self):
        if not isinstance(self.major_dim, int):
            raise TypeError(f"StridedLayout(major_dim=...) must be an int, got {type(self.major_dim)}")

    @property
    def name(self):
        return "STRIDED"

    def order(self, rank: int) -> list:
        """Dimension order from fastest to slowest varying: reversed range with `major_dim` swapped to the front."""
        if rank <= 0:
            return []
        if not (-rank <= self.major_dim < rank):
            raise ValueError(f"Invalid StridedLayout.major_dim={self.major_dim} for rank={rank}")
        major = self.major_dim % rank
        order = list(range(rank - 1, -1, -1))
        pos = order.index(major)
        order[0], order[pos] = order[pos], order[0]
        return order

    def can_preserve_storage_as(self, other: Layout, rank: int) -> bool:
        return isinstance(other, StridedLayout) and self.order(rank) == other.order(rank)

    def make_transformation(self, shape, is_fp4: bool) -> LayoutTransformation:
        return StridedLayoutTransformation(list(shape), is_fp4, self.order(len(shape)))

    def swizzle_block_shape(self, block_shape):
        return block_shape


@dataclass(frozen=True)
class StridedLayoutTransformation(LayoutTransformation):
    order: list

    @property
    def storage_shape(self) -> list:
        shape = list(self.shape)
        if self.is_fp4:
            pd = self.order[0]
            if shape[pd] % 2:
                raise ValueError(f"FP4 packing dimension {pd} must have an even size, got {shape[pd]}")
            shape[pd] //= 2
        return shape

    def _dense_strides(self, storage_shape):
        strides, run = [0] * len(storage_shape), 1
        for d in self.order:
            strides[d] = run
            run *= storage_shape[d]
        return strides

    def swizzle_data(self, data):
        assert data.numel() == 0 or data.stride(-1) == 1
        out_shape = self.storage_shape
        if not out_shape:
            return data
        out = torch.empty_strided(out_shape, self._dense_strides(out_shape), dtype=data.dtype, device=data.device)
        repack(data, -1, self.order[0], self.is_fp4, out=out)
        return out

    def unswizzle_data(self, data):
        assert data.stride(self.order[0]) == 1
        shape = list(self.shape)
        if self.is_fp4:
            shape[-1] //= 2
        out = torch.empty(shape, dtype=data.dtype, device=data.device)
        repack(data, self.order[0], -1, self.is_fp4, out=out)
        return out
