"""Ragged-tensor metadata (mirrors `triton_kernels/tensor_details/ragged_tensor.py:12-210`).

A ragged tensor is a stack of 2-D slices (one per expert) sharing the column count.  The metadata
holds, for every row-block size a GEMM may use (16..256), where each slice's blocks start and the
flat schedule of (block, slice) pairs.  `remap_ragged_tensor_metadata` restricts the metadata to a subset
of the slices (the local experts of an expert-parallel rank).
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from .. import _native as nt


@dataclass
class RaggedTensorMetadata:
    slice_sizes: torch.Tensor  # [n_slices] int32 rows per slice
    slice_offs: torch.Tensor  # [n_slices + 1] int32 = [0] + cumsum(slice_sizes)
    block_offs_data: torch.Tensor  # [n_block_sizes, n_slices + 1] int32
    block_schedule_data: torch.Tensor  # [n_block_sizes, max_n_blocks] int32, (block << 16) | slice, -1 padded
    expected_slice_size: int | None = None
    slice_sizes_divisibility: int = None

    def __post_init__(self):
        n = len(RaggedTensorMetadata.block_sizes())
        assert self.block_offs_data.shape[0] == n
        assert self.block_schedule_data.shape[0] == n
        assert self.block_offs_data.dtype == torch.int32
        assert self.block_schedule_data.dtype == torch.int32
        if self.slice_sizes is not None:
            assert self.slice_sizes.dtype == torch.int32
        if self.slice_offs is not None:
            assert self.slice_offs.dtype == torch.int32

    @property
    def n_slices(self):
        return self.slice_sizes.shape[0]

    def block_offs(self, block_size):
        return self.block_offs_data[RaggedTensorMetadata.block_sizes().index(block_size)]

    def block_schedule(self, block_size):
        return self.block_schedule_data[RaggedTensorMetadata.block_sizes().index(block_size)]

    @staticmethod
    def n_blocks(n_slices, n_total_rows, block_size):
        """Upper bound on the number of row blocks without knowing the slice sizes."""
        if n_total_rows <= n_slices:
            return n_total_rows
        return n_slices - 1 - ((n_slices - n_total_rows - 1) // block_size)

    @staticmethod
    def max_n_blocks(n_slices, n_total_rows):
        return RaggedTensorMetadata.n_blocks(n_slices, n_total_rows, min(RaggedTensorMetadata.block_sizes()))

    @staticmethod
    def block_sizes_log2():
        return range(4, 9)

    @staticmethod
    def block_sizes():
        return [2**x for x in RaggedTensorMetadata.block_sizes_log2()]


def ragged_metadata_fields(metadata, block_size):
    return (metadata.slice_sizes, metadata.slice_offs, metadata.block_offs(block_size),
            metadata.block_schedule(block_size), metadata.expected_slice_size, metadata.slice_sizes_divisibility or 1)


def _alloc(n_slices, n_total_rows, device):
    """(slice_offs, block_offs_data, block_schedule_data) as rows of two int32 buffers."""
    n_bs = len(RaggedTensorMetadata.block_sizes())
    width = RaggedTensorMetadata.max_n_blocks(n_slices, n_total_rows)
    offs = torch.empty((n_bs + 1, n_slices + 1), dtype=torch.int32, device=device)
    sched = torch.empty((n_bs, max(width, 0)), dtype=torch.int32, device=device)
    return offs[0], offs[1:], sched, width


def make_ragged_tensor_metadata(slice_sizes, n_total_rows):
    assert slice_sizes.ndim == 1
    assert slice_sizes.dtype == torch.int32
    nt.require_gpu(slice_sizes, "slice_sizes")
    n_slices = slice_sizes.shape[0]
    slice_sizes = slice_sizes.contiguous()
    slice_offs, block_offs, sched, width = _alloc(n_slices, n_total_rows, slice_sizes.device)
    with nt.on_device(slice_sizes.device):
        nt.check(
            nt.lib().tk_ragged_metadata(nt.ptr(slice_sizes), n_slices, slice_offs.data_ptr(), block_offs.data_ptr(),
                                        block_offs.stride(0), nt.ptr(sched) if width > 0 else None,
                                        sched.stride(0) if width > 0 else 0, width, nt.stream_ptr(slice_sizes.device)))
    return RaggedTensorMetadata(slice_sizes, slice_offs, block_offs, sched)


def remap_ragged_tensor_metadata(src_ragged_tensor_metadata: RaggedTensorMetadata, slice_map: torch.Tensor) -> RaggedTensorMetadata:
    """Metadata of the ragged tensor made of the slices with `slice_map[slice_id] != -1` (ragged_tensor.py:348-381 of the
    reference; the expert-parallel step uses it to keep a rank's own experts).  Kept sizes / offsets keep their values
    and move to the front, schedule entries get `slice_map[slice_id]` as their slice id."""
    md = src_ragged_tensor_metadata
    assert slice_map.ndim == 1
    assert slice_map.shape[0] == md.slice_sizes.shape[0]
    assert slice_map.dtype == torch.int32
    nt.require_gpu(slice_map, "slice_map")
    n_slices = md.slice_sizes.shape[0]
    dev = md.slice_sizes.device
    n_bs, width = md.block_offs_data.shape[0], md.block_schedule_data.shape[-1]
    slice_sizes = torch.empty((n_slices, ), dtype=torch.int32, device=dev)
    offs = torch.empty((n_bs + 1, n_slices + 1), dtype=torch.int32, device=dev)
    sched = torch.empty((n_bs, width), dtype=torch.int32, device=dev)
    src_sizes, src_offs, smap = md.slice_sizes.contiguous(), md.slice_offs.contiguous(), slice_map.contiguous()
    bo, bs = md.block_offs_data, md.block_schedule_data
    assert bo.stride(-1) == 1 and (width == 0 or bs.stride(-1) == 1)
    with nt.on_device(dev):
        nt.check(
            nt.lib().tk_ragged_remap(nt.ptr(src_sizes), nt.ptr(src_offs), nt.ptr(bo), bo.stride(0), nt.ptr(bs) if width > 0 else None,
                                     bs.stride(0) if width > 0 else 0, nt.ptr(smap), n_slices, n_bs, width, nt.ptr(slice_sizes),
                                     offs[0].data_ptr(), offs[1:].data_ptr(), offs.stride(0), nt.ptr(sched) if width > 0 else None,
                                     sched.stride(0) if width > 0 else 0, nt.stream_ptr(dev)))
    out = RaggedTensorMetadata(slice_sizes, offs[0], offs[1:], sched)
    out.remapped_from = n_slices  # tells `matmul` that block offsets are those of the source tensor, not a running sum
    return out


def __getattr__(name):
    # the reference's torch twin of this module, resolved on first use (it needs the fully imported `tensor` module)
    if name == "make_ragged_tensor_metadata_torch":
        from .. import torch_twins
        return getattr(torch_twins, name)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
