"""Expert histogram and gather/scatter permutations of a routing bitmatrix
(mirrors `triton_kernels/tensor_details/bitmatrix.py:8-150`)."""
from __future__ import annotations

from dataclasses import dataclass

import torch

from .. import _native as nt


@dataclass
class BitmatrixMetadata:
    """
    For the bitmatrix   [0 0 1 0 1 1 0
                         0 1 0 0 0 1 0
                         1 1 1 0 0 0 1
                         0 0 1 0 1 0 0]
    col_sum         = [1 2 3 0 2 2 1]
    col_sorted_indx = [5 | 3 6 | 0 7 9 | | 1 10 | 2 4 | 8]   nonzeros numbered row-major, grouped by column
    row_sorted_indx = [3 6 8 | 1 9 | 0 2 4 10 | 5 7]          its inverse permutation
    """
    col_sum: torch.Tensor
    col_sorted_indx: torch.Tensor
    row_sorted_indx: torch.Tensor


def _route(logits, indx16, n_rows, n_experts, k, *, apply_softmax, use_provided_indx, vals, bitmatrix_data, want_meta,
           want_extras=False, ragged=None, static_scratch=False):
    """Fills and submits a tk_route_desc.  Returns a dict of the tensors it allocated.  With `static_scratch` the
    kernels' workspace is the library's own device array (`tk_route_static`) instead of a part of the allocation
    made here."""
    dev = indx16.device
    T = indx16.shape[0]
    R = T * k
    out = {}
    d = nt.RouteDesc()
    d.logits = nt.ptr(logits)
    d.logits_dtype = nt.TORCH_TO_TK[logits.dtype] if logits is not None else nt.TK_F32
    d.logits_stride_m = logits.stride(0) if logits is not None else 0
    d.n_tokens = T
    if isinstance(n_rows, torch.Tensor):
        d.n_rows = -1
        d.n_rows_ptr = n_rows.data_ptr()
        assert n_rows.dtype == torch.int32 and n_rows.is_cuda
    else:
        d.n_rows = -1 if n_rows is None else int(n_rows)
        d.n_rows_ptr = None
    d.n_experts = n_experts
    d.k = k
    d.apply_softmax = int(bool(apply_softmax))
    d.use_provided_indx = int(bool(use_provided_indx))
    d.vals = nt.ptr(vals)
    d.indx = indx16.data_ptr()
    d.indx_dtype = nt.TK_I16
    if bitmatrix_data is not None:
        d.bitmatrix = bitmatrix_data.data_ptr()
        d.bitmatrix_stride_w = bitmatrix_data.stride(1)
    if want_meta:
        # one int32 allocation carved into the histogram, both permutations (adjacent, as the reference carves them
        # from one [2R] buffer, bitmatrix.py:119-121), the gather index and the kernels' workspace
        e_pad = (n_experts + 3) & ~3
        ws_words = 0 if static_scratch else (max(1, nt.lib().tk_route_workspace_bytes(T, n_experts)) + 3) // 4
        r_pad = (R + 3) & ~3
        n_gather = r_pad if want_extras else 0
        buf = torch.empty((e_pad + 2 * r_pad + n_gather + ws_words, ), dtype=torch.int32, device=dev)
        col_sum = buf[:n_experts]
        combined = buf[e_pad:e_pad + 2 * R]
        ws = buf[e_pad + 2 * r_pad + n_gather:]
        out.update(col_sum=col_sum, col_sorted_indx=combined[:R], row_sorted_indx=combined[R:], _ws=ws)
        d.col_sum = col_sum.data_ptr()
        d.col_sorted_indx = combined.data_ptr()
        d.row_sorted_indx = combined.data_ptr() + 4 * R
        d.workspace = None if static_scratch else ws.data_ptr()
        if want_extras:
            gather = buf[e_pad + 2 * r_pad:e_pad + 2 * r_pad + R]
            d.gather_indx = gather.data_ptr()
            out["gather_indx"] = gather
            if vals is not None:
                gam = torch.empty((R, ), dtype=vals.dtype, device=dev)
                d.gammas = gam.data_ptr()
                out["gammas"] = gam
        if ragged is not None:
            slice_offs, block_offs, sched, width = ragged
            d.slice_offs = slice_offs.data_ptr()
            d.block_offs = block_offs.data_ptr()
            d.block_offs_stride = block_offs.stride(0)
            d.block_schedule = sched.data_ptr() if width > 0 else None
            d.block_schedule_stride = sched.stride(0) if width > 0 else 0
            d.max_n_blocks = width
    if T > 0:
        with nt.on_device(dev):
            entry = nt.lib().tk_route_static if static_scratch else nt.lib().tk_route
            nt.check(entry(d, nt.stream_ptr(dev)))
    elif want_meta:
        out["col_sum"].zero_()
    return out


def make_bitmatrix_metadata(nonzero_indx, bitmatrix):
    """`nonzero_indx [T, k]` expert ids (-1 = dropped); `bitmatrix` gives the column count and row bound."""
    assert nonzero_indx.ndim == 2
    nt.require_gpu(nonzero_indx, "nonzero_indx")
    n_cols = bitmatrix.shape[1]
    n_rows = bitmatrix.shape[0]
    indx16 = nonzero_indx if nonzero_indx.dtype == torch.int16 else nonzero_indx.to(torch.int16)
    indx16 = indx16.contiguous()
    r = _route(None, indx16, n_rows, n_cols, nonzero_indx.shape[1], apply_softmax=False, use_provided_indx=True,
               vals=None, bitmatrix_data=None, want_meta=True)
    return BitmatrixMetadata(col_sum=r["col_sum"], col_sorted_indx=r["col_sorted_indx"],
                             row_sorted_indx=r["row_sorted_indx"])


def __getattr__(name):
    # the reference's torch twin of this module, resolved on first use (it needs the fully imported `tensor` module)
    if name == "make_bitmatrix_metadata_torch":
        from .. import torch_twins
        return getattr(torch_twins, name)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
