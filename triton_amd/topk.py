"""Top-k (+softmax) router (mirrors `triton_kernels/topk.py:25-141`).

`topk` launches the fused routing pass: selection, gate softmax, bitmatrix, expert histogram and both
permutations come out of one `tk_route` call, so the returned `SparseMatrix` already carries its
`mask_metadata`.  The backward pass, `all_gather` and symmetric-memory outputs of the reference are
training / multi-GPU features and are not part of this build.
"""
from __future__ import annotations

from typing import Optional, Union

import torch

from . import _native as nt
from .tensor import SparseMatrix, Tensor, wrap_torch_tensor
from .tensor_details.bitmatrix import BitmatrixMetadata, _route
from .tensor_details.dtype import BIT


def _cdiv(a, b):
    return (a + b - 1) // b


def _topk_route(x, k, apply_softmax, y_indx, n_rows, *, want_meta, want_extras=False, ragged=None):
    if isinstance(x, Tensor):
        n_rows = x.shape[0] if n_rows is None else n_rows
        x = x.storage.data
    assert x.ndim == 2
    nt.require_gpu(x, "x")
    T, E = x.shape
    assert E < 32768
    if x.stride(1) != 1:
        x = x.contiguous()
    if k & (k - 1) or k > 32:
        raise ValueError(f"k must be a power of two <= 32 (got {k})")
    dev = x.device
    y_vals = torch.empty((T, k), dtype=x.dtype, device=dev)
    provided = y_indx is not None
    if provided:
        indx16 = (y_indx if y_indx.dtype == torch.int16 else y_indx.to(torch.int16)).contiguous()
    else:
        indx16 = torch.empty((T, k), dtype=torch.int16, device=dev)
    words = _cdiv(E, 32)
    bm = torch.empty((words, _cdiv(T, 32) * 32), dtype=torch.uint32, device=dev)
    bm_t = torch.transpose(bm, 0, 1)[:T]
    n_rows_arg = None if (n_rows is None or (isinstance(n_rows, int) and n_rows == T)) else n_rows
    r = _route(x, indx16, n_rows_arg, E, k, apply_softmax=apply_softmax, use_provided_indx=provided, vals=y_vals,
               bitmatrix_data=bm_t, want_meta=want_meta, want_extras=want_extras, ragged=ragged)
    shape0 = T if n_rows is None else n_rows
    mask = wrap_torch_tensor(bm_t, dtype=BIT, shape=[shape0, E], shape_max=[T, None])
    return y_vals, (y_indx if provided else indx16), mask, r


def topk_forward(x, k, apply_softmax=True, dim=1, y_indx=None, n_rows=None, all_gather=False, symm_mem_pool=None):
    assert dim == 1
    if all_gather or symm_mem_pool is not None:
        raise NotImplementedError("all_gather / symmetric-memory outputs are multi-GPU features")
    y_vals, y_indx, mask, _ = _topk_route(x, k, apply_softmax, y_indx, n_rows, want_meta=False)
    return y_vals, y_indx, mask


def topk(x: Union[Tensor, torch.Tensor], k: int, apply_softmax: bool = True, dim: int = 1,
         y_indx: Optional[torch.Tensor] = None, n_rows: Optional[int] = None, all_gather: bool = False,
         symm_mem_pool=None):
    """Top-k of each row of `x [n_tokens, n_expts]`.

    Returns a `SparseMatrix` with `vals` (softmax over the k kept logits when `apply_softmax`), `indx`
    (int16, value-descending, ties to the lower index) and the bit `mask`; rows `>= n_rows` are not routed.
    """
    assert dim == 1
    if all_gather or symm_mem_pool is not None:
        raise NotImplementedError("all_gather / symmetric-memory outputs are multi-GPU features")
    if x.requires_grad if isinstance(x, torch.Tensor) else False:
        raise NotImplementedError("topk backward is not part of this build (inference only)")
    y_vals, y_indx, mask, r = _topk_route(x, k, apply_softmax, y_indx, n_rows, want_meta=True)
    meta = BitmatrixMetadata(col_sum=r["col_sum"], col_sorted_indx=r["col_sorted_indx"],
                             row_sorted_indx=r["row_sorted_indx"])
    return SparseMatrix(vals=y_vals, indx=y_indx, mask=mask, mask_metadata=meta)
