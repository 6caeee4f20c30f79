"""Top-k (+softmax) router (mirrors `triton_kernels/topk.py:25-141`).

`topk` launches the fused routing pass: selection, gate softmax, bitmatrix, expert histogram and both
permutations come out of one `tk_route` call, so the returned `SparseMatrix` already carries its
`mask_metadata`.  The backward pass (`topk_backward`, used through autograd when the logits require a gradient)
is a kernel of its own; `all_gather` and symmetric-memory outputs of the reference are multi-GPU features and are
not part of this build.
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


def topk_backward(x, y_indx, dy_vals, k, n_rows, apply_softmax):
    """dx [n_tokens, n_expts] for the gradient `dy_vals [n_tokens, k]` of the kept values (topk.py:76-85)."""
    assert dy_vals.shape[-1] == k and x.ndim == 2
    nt.require_gpu(x, "x")
    if x.stride(1) != 1:
        x = x.contiguous()
    dy = dy_vals.to(x.dtype)
    if dy.stride(1) != 1:
        dy = dy.contiguous()
    indx16 = (y_indx if y_indx.dtype == torch.int16 else y_indx.to(torch.int16)).contiguous()
    dx = torch.empty_like(x, memory_format=torch.contiguous_format)
    T, E = x.shape
    rows_imm, rows_ptr = -1, None
    if isinstance(n_rows, torch.Tensor):
        assert n_rows.dtype == torch.int32 and n_rows.is_cuda
        rows_ptr = n_rows.data_ptr()
    elif n_rows is not None:
        rows_imm = int(n_rows)
    with nt.on_device(x.device):
        nt.check(
            nt.lib().tk_topk_backward(x.data_ptr(), nt.TORCH_TO_TK[x.dtype], x.stride(0), indx16.data_ptr(), indx16.stride(0),
                                      dy.data_ptr(), dy.stride(0), dx.data_ptr(), dx.stride(0), T, E, k, int(bool(apply_softmax)),
                                      rows_imm, rows_ptr, nt.stream_ptr(x.device)))
    return dx


class TopK(torch.autograd.Function):
    """Differentiable selection (topk.py:88-105): the gate values carry the gradient; indices, bitmatrix words and
    metadata are returned as non-differentiable tensors."""

    @staticmethod
    def forward(ctx, x, k, apply_softmax, y_indx, n_rows):
        y_vals, indx, mask, r = _topk_route(x.detach(), k, apply_softmax, y_indx, n_rows, want_meta=True)
        ctx.save_for_backward(x, indx)
        ctx.k, ctx.apply_softmax, ctx.n_rows = k, apply_softmax, n_rows
        others = (indx, mask.storage.data, r["col_sum"], r["col_sorted_indx"], r["row_sorted_indx"])
        ctx.mark_non_differentiable(*others)
        return (y_vals, *others)

    @staticmethod
    def backward(ctx, dy_vals, *_unused):
        x, indx = ctx.saved_tensors
        return topk_backward(x, indx, dy_vals, ctx.k, ctx.n_rows, ctx.apply_softmax), None, None, None, None


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
    if isinstance(x, torch.Tensor) and x.requires_grad and torch.is_grad_enabled():
        y_vals, y_indx, bm_t, col_sum, col_sorted, row_sorted = TopK.apply(x, k, apply_softmax, y_indx, n_rows)
        T, E = x.shape
        mask = wrap_torch_tensor(bm_t, dtype=BIT, shape=[T if n_rows is None else n_rows, E], shape_max=[T, None])
        r = dict(col_sum=col_sum, col_sorted_indx=col_sorted, row_sorted_indx=row_sorted)
    else:
        y_vals, y_indx, mask, r = _topk_route(x, k, apply_softmax, y_indx, n_rows, want_meta=True)
    meta = BitmatrixMetadata(col_sum=r["col_sum"], col_sorted_indx=r["col_sorted_indx"],
                             row_sorted_indx=r["row_sorted_indx"])
    return SparseMatrix(vals=y_vals, indx=y_indx, mask=mask, mask_metadata=meta)


from .torch_twins import topk_torch  # noqa: E402,F401  (reference twin; never called by `topk`)
