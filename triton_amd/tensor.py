"""Tensor wrappers and routing data classes (mirrors `triton_kernels/tensor.py`).

`Tensor` = torch storage + a logical dtype/shape (sub-byte types such as FP4 have a logical shape twice
the storage shape along the unit-stride dimension) + a layout.  TMA helpers of the reference
(tensor.py:101-157) have no counterpart on gfx950 and are absent.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from .tensor_details.dtype import (BF16, BIT, FP4, FP8_E4M3FN, FP8_E4M3FNUZ, FP8_E5M2, FP16, FP32, FP64, INT16, INT32,
                                   INT64, UINT8, DataType, FloatType, IntegerType)
from .tensor_details.layout import Layout, StridedLayout


@dataclass
class Storage:
    data: torch.Tensor
    layout: Layout

    @property
    def device(self):
        return self.data.device


@dataclass
class Tensor:
    storage: Storage
    dtype: IntegerType | FloatType
    shape: list | None = None
    shape_max: list | None = None

    def __post_init__(self):
        assert isinstance(self.storage, Storage)
        if self.shape is None:
            if self.dtype.bitwidth < 8:
                raise ValueError("shape must be provided for sub-byte types")
            self.shape = list(self.storage.data.shape)
        self.shape = list(self.shape)
        for s in self.shape:
            assert isinstance(s, int) or (hasattr(s, "numel") and s.numel() == 1), "shape entries must be int or 1-element tensors"
        if self.shape_max is None:
            self.shape_max = [None] * len(self.shape)
        self.shape_max = list(self.shape_max)
        for i, (s, smax) in enumerate(zip(self.shape, self.shape_max)):
            if smax is None:
                self.shape_max[i] = s
            elif not isinstance(smax, int):
                raise ValueError(f"shape_max[{i}] must be `int` or `None`; got {type(smax)}")
        assert all(isinstance(s, int) for s in self.shape_max)

    # torch-like accessors
    @property
    def ndim(self):
        return len(self.shape)

    def dim(self):
        return self.ndim

    @property
    def device(self):
        return self.storage.device

    @property
    def data(self):
        return self.storage.data

    def stride(self, i=None):
        return self.storage.data.stride() if i is None else self.storage.data.stride(i)

    def data_ptr(self):
        return self.storage.data.data_ptr()

    def numel(self):
        return self.storage.data.numel()

    def element_size(self):
        return self.dtype.bitwidth // 8

    def size(self, i=None):
        return self.shape if i is None else self.shape[i]


_TO_TORCH = {
    FP4: torch.uint8,
    UINT8: torch.uint8,
    FP8_E4M3FN: torch.float8_e4m3fn,
    FP8_E4M3FNUZ: torch.float8_e4m3fnuz,
    FP8_E5M2: torch.float8_e5m2,
    BF16: torch.bfloat16,
    FP16: torch.float16,
    FP32: torch.float32,
    FP64: torch.float64,
    INT16: torch.int16,
    INT32: torch.int32,
    INT64: torch.int64,
}

_FROM_TORCH = {
    torch.uint8: UINT8,
    torch.float8_e4m3fn: FP8_E4M3FN,
    torch.float8_e4m3fnuz: FP8_E4M3FNUZ,
    torch.float8_e5m2: FP8_E5M2,
    torch.float16: FP16,
    torch.bfloat16: BF16,
    torch.float32: FP32,
    torch.float64: FP64,
    torch.int16: INT16,
    torch.int32: INT32,
    torch.int64: INT64,
}


def dtype_to_torch_dtype(dtype):
    if isinstance(dtype, (IntegerType, FloatType)):
        return _TO_TORCH[dtype]
    return dtype


def torch_dtype_to_dtype(dtype):
    if isinstance(dtype, (IntegerType, FloatType)):
        return dtype
    if dtype in _FROM_TORCH:
        return _FROM_TORCH[dtype]
    if "float8" in str(dtype):
        return FP8_E4M3FN
    raise AssertionError(f"Unknown dtype: {dtype}")


def wrap_torch_tensor(torch_tensor, dtype=None, shape=None, shape_max=None, layout=None):
    """Wraps a torch tensor; for FP4 the logical shape doubles along the unit-stride dim (tensor.py:216-233)."""
    dtype = torch_dtype_to_dtype(torch_tensor.dtype if dtype is None else dtype)
    strides = torch_tensor.stride()
    if shape is None:
        shape = list(torch_tensor.shape)
        if dtype == FP4:
            shape[strides.index(1)] *= (8 * torch_tensor.dtype.itemsize) // dtype.bitwidth
    if shape_max is None:
        shape_max = list(shape)
    if layout is None:
        major = strides.index(1) if 1 in strides else -1
        layout = StridedLayout(major_dim=major - torch_tensor.ndim)
    return Tensor(Storage(torch_tensor, layout), dtype=dtype, shape=shape, shape_max=shape_max)


def convert_layout(tensor: Tensor, layout: Layout, **layout_transformation_kwargs):
    """Re-encodes `tensor`'s storage for `layout`; a no-op when the storage is already valid for it."""
    shape = list(tensor.shape)
    if not layout_transformation_kwargs and tensor.storage.layout.can_preserve_storage_as(layout, len(shape)):
        return tensor
    is_fp4 = tensor.dtype == FP4
    canonical = tensor.storage.layout.make_transformation(shape, is_fp4).unswizzle_data(tensor.storage.data)
    new_data = layout.make_transformation(shape, is_fp4, **layout_transformation_kwargs).swizzle_data(canonical)
    return Tensor(Storage(new_data, layout), dtype=tensor.dtype, shape=shape)


def empty(shape, dtype: DataType, device, layout=None, allow_implicit_conversion: bool = False):
    """Uninitialised `Tensor` whose storage is dense in `layout`'s dimension order (tensor.py:293-313)."""
    storage_dtype = torch.uint8 if dtype == FP4 else dtype_to_torch_dtype(dtype)
    base = layout if isinstance(layout, StridedLayout) else StridedLayout()
    storage_shape = base.storage_shape(list(shape), dtype == FP4)
    strides, run = [0] * len(storage_shape), 1
    for d in base.order(len(shape)):
        strides[d] = run
        run *= storage_shape[d]
    data = torch.empty_strided(storage_shape, strides, device=device, dtype=storage_dtype)
    ret = wrap_torch_tensor(data, dtype=dtype, shape=list(shape), layout=base)
    if allow_implicit_conversion:
        ret = convert_layout(ret, layout)
    return ret


# ---------------------------------------------------------------------------------------------------
# routing data classes (tensor.py:159-209 of the reference)
# ---------------------------------------------------------------------------------------------------
from .tensor_details import bitmatrix as bitmatrix_details  # noqa: E402
from .tensor_details import ragged_tensor as ragged_tensor_details  # noqa: E402
from .tensor_details.bitmatrix import BitmatrixMetadata  # noqa: E402,F401
from .tensor_details.ragged_tensor import RaggedTensorMetadata  # noqa: E402,F401

make_bitmatrix_metadata = bitmatrix_details.make_bitmatrix_metadata
make_ragged_tensor_metadata = ragged_tensor_details.make_ragged_tensor_metadata
remap_ragged_tensor_metadata = ragged_tensor_details.remap_ragged_tensor_metadata


@dataclass
class RaggedTensor:
    """A stack of 2-D slices with a common column count, stored as one (possibly padded) 2-D tensor."""
    slice_sizes: torch.Tensor
    data: torch.Tensor
    metadata: RaggedTensorMetadata


@dataclass
class SparseMatrix:
    """Top-k result: `vals`/`indx` [T, k] plus the bit mask of selected columns.  `mask_metadata`
    (histogram and permutations) is computed on construction unless the producer already has it."""
    indx: torch.Tensor
    vals: torch.Tensor
    mask: Tensor
    mask_metadata: BitmatrixMetadata | None = None

    def __post_init__(self):
        if self.mask_metadata is None:
            self.mask_metadata = make_bitmatrix_metadata(self.indx, self.mask)
