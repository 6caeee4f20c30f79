"""CPU oracle: top-k router, expert histogram / gather-scatter indices, ragged block schedule.

Test infrastructure only.  Follows
  * `topk_torch`                         python/triton_kernels/triton_kernels/topk.py:144-185
  * `make_bitmatrix_metadata_torch`      .../tensor_details/bitmatrix.py:157-168
  * `make_ragged_tensor_metadata_torch`  .../tensor_details/ragged_tensor.py:217-253
    with `n_blocks / max_n_blocks / block_sizes` of .../ragged_tensor.py:73-89 (HIP set 16..256)
  * the routing glue of python/triton_kernels/tests/test_distributed.py:203-210
  * `_topk_backward`                     .../topk_details/_topk_backward.py:5-51 (pinned against torch autograd of the
    forward oracle in tests/test_oracle_routing.py)
  * `remap_ragged_tensor_metadata_torch` .../tensor_details/ragged_tensor.py:388-433 (pinned in
    tests/test_oracle_routing.py by a hand-worked example and by rebuilding the kept slices' metadata from scratch)
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch

BLOCK_SIZES = (16, 32, 64, 128, 256)  # ragged_tensor.py:84-89 on HIP


def topk(logits: torch.Tensor, k: int, apply_softmax: bool = True, n_rows: int | None = None):
    """Returns `(vals [T,k] (logits dtype), indx [T,k] int32, bitmatrix uint32 [T, ceil(E/32)])`.

    Selection = stable descending argsort, so ties go to the lower expert index
    (topk.py:160); softmax over the k kept logits in fp32, cast back (topk.py:170-171).
    Rows `>= n_rows` get index -1 and no bits (topk.py:175).
    """
    x = logits.detach().to("cpu")
    T, E = x.shape
    n_rows = T if n_rows is None else int(n_rows)
    xf = x.to(torch.float32).numpy()
    order = np.argsort(-xf, axis=1, kind="stable")[:, :k]
    vals = np.take_along_axis(xf, order, axis=1)
    if apply_softmax:
        v = torch.softmax(torch.from_numpy(vals), dim=-1).to(x.dtype)
    else:
        v = torch.from_numpy(vals).to(x.dtype)
    indx = order.astype(np.int32)
    indx[n_rows:, :] = -1
    words = (E + 31) // 32
    bits = np.zeros((T, words), dtype=np.uint32)
    for j in range(k):
        col = indx[:n_rows, j].astype(np.int64)
        np.bitwise_or.at(bits, (np.arange(n_rows), col // 32), (np.uint32(1) << (col % 32).astype(np.uint32)))
    return v, torch.from_numpy(indx), torch.from_numpy(bits.view(np.int32)).view(torch.int32)


@dataclass
class BitmatrixMetadata:
    col_sum: torch.Tensor  # [E] int32, tokens routed to each expert
    col_sorted_indx: torch.Tensor  # [R] int32, flat positions t*k+j grouped by expert, -1 padded
    row_sorted_indx: torch.Tensor  # [R] int32, inverse permutation, -1 padded


def make_bitmatrix_metadata(indx: torch.Tensor, n_cols: int) -> BitmatrixMetadata:
    """bitmatrix.py:157-168 with `histc` replaced by a bincount over the valid entries."""
    flat = indx.detach().to("cpu").reshape(-1).to(torch.int64).numpy()
    n = flat.shape[0]
    valid = flat != -1
    col_sorted_valid = np.argsort(flat[valid], kind="stable")
    col_sorted = np.full(n, -1, dtype=np.int64)
    col_sorted[:col_sorted_valid.shape[0]] = col_sorted_valid
    row_sorted_valid = np.argsort(col_sorted_valid, kind="stable")
    row_sorted = np.full(n, -1, dtype=np.int64)
    row_sorted[:row_sorted_valid.shape[0]] = row_sorted_valid
    col_sum = np.bincount(flat[valid], minlength=n_cols)[:n_cols]
    return BitmatrixMetadata(
        col_sum=torch.from_numpy(col_sum.astype(np.int32)),
        col_sorted_indx=torch.from_numpy(col_sorted.astype(np.int32)),
        row_sorted_indx=torch.from_numpy(row_sorted.astype(np.int32)),
    )


def n_blocks(n_slices: int, n_total_rows: int, block_size: int) -> int:
    """Upper bound on the number of row blocks (ragged_tensor.py:73-77); Python floor division."""
    if n_total_rows <= n_slices:
        return n_total_rows
    return n_slices - 1 - ((n_slices - n_total_rows - 1) // block_size)


def max_n_blocks(n_slices: int, n_total_rows: int) -> int:
    return n_blocks(n_slices, n_total_rows, min(BLOCK_SIZES))


@dataclass
class RaggedTensorMetadata:
    slice_sizes: torch.Tensor  # [E] int32
    slice_offs: torch.Tensor  # [E+1] int32
    block_offs_data: torch.Tensor  # [n_bs, E+1] int32
    block_schedule_data: torch.Tensor  # [n_bs, max_n_blocks] int32, (block<<16)|slice, -1 padded


def make_ragged_tensor_metadata(slice_sizes: torch.Tensor, n_total_rows: int) -> RaggedTensorMetadata:
    """ragged_tensor.py:217-253."""
    sizes = slice_sizes.detach().to("cpu").to(torch.int64).numpy()
    E = sizes.shape[0]
    width = max_n_blocks(E, n_total_rows)
    slice_offs = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
    offs_rows, sched_rows = [], []
    for bs in BLOCK_SIZES:
        nb = (sizes + bs - 1) // bs
        offs = np.concatenate([[0], np.cumsum(nb)]).astype(np.int64)
        sched = np.full(width, -1, dtype=np.int64)
        for s in range(E):
            for b in range(int(nb[s])):
                pos = offs[s] + b
                if pos < width:
                    sched[pos] = (b << 16) | s
        offs_rows.append(offs.astype(np.int32))
        sched_rows.append(sched.astype(np.int32))
    return RaggedTensorMetadata(
        slice_sizes=torch.from_numpy(sizes.astype(np.int32)),
        slice_offs=torch.from_numpy(slice_offs),
        block_offs_data=torch.from_numpy(np.stack(offs_rows)),
        block_schedule_data=torch.from_numpy(np.stack(sched_rows)) if width > 0 else torch.empty(
            (len(BLOCK_SIZES), 0), dtype=torch.int32),
    )


def topk_backward(x: torch.Tensor, indx: torch.Tensor, dy_vals: torch.Tensor, apply_softmax: bool = True,
                  n_rows: int | None = None) -> torch.Tensor:
    """_topk_backward.py:5-51: dx is zero except at the kept columns, where it is `y * (dy - sum(y * dy))` with
    `y = softmax(x[kept])` in fp32 (or `dy` without softmax); result in x's dtype.  Rows >= n_rows stay zero."""
    xf = x.detach().to("cpu").to(torch.float32)
    dy = dy_vals.detach().to("cpu").to(torch.float32)
    ix = indx.detach().to("cpu").to(torch.int64)
    T = xf.shape[0]
    rows = T if n_rows is None else int(n_rows)
    dx = torch.zeros_like(xf)
    if rows > 0:
        kept = torch.gather(xf[:rows], 1, ix[:rows])
        if apply_softmax:
            y = torch.softmax(kept, dim=1)
            g = y * (dy[:rows] - (y * dy[:rows]).sum(dim=1, keepdim=True))
        else:
            g = dy[:rows]
        dx[:rows].scatter_(1, ix[:rows], g)
    return dx.to(x.dtype)


def remap_ragged_tensor_metadata(md: RaggedTensorMetadata, slice_map: torch.Tensor) -> RaggedTensorMetadata:
    """ragged_tensor.py:388-433: keep the slices with `slice_map[s] != -1`, in their order.  Kept sizes, offsets and
    block offsets move to the front unchanged, -1 behind them; schedule entries of kept slices are compacted and get
    `slice_map[s]` as slice id; the first -1 of each block-offset row is replaced by the number of entries kept."""
    smap = slice_map.detach().to("cpu").to(torch.int64).numpy()
    n = smap.shape[0]
    keep = smap != -1

    def compact(vals, mask):
        vals = np.asarray(vals, dtype=np.int64)
        return np.concatenate([vals[mask], np.full(int((~mask).sum()), -1, dtype=np.int64)])

    sizes = compact(md.slice_sizes.numpy(), keep)
    keep1 = np.concatenate([keep, [False]])
    offs = compact(md.slice_offs.numpy(), keep1)
    bo_rows, bs_rows = [], []
    for i in range(md.block_offs_data.shape[0]):
        bo = compact(md.block_offs_data[i].numpy(), keep1)
        sched = md.block_schedule_data[i].numpy().astype(np.int64)
        valid = sched != -1
        slice_id = np.where(valid, sched & 0xFFFF, 0)
        kept = valid & keep[slice_id]
        new = (sched & 0xFFFF0000) | np.where(kept, smap[slice_id], 0)
        out = compact(new, kept)
        bo[int(np.nonzero(bo == -1)[0][0])] = int(kept.sum())
        bo_rows.append(bo.astype(np.int32))
        bs_rows.append(out.astype(np.int32))
    return RaggedTensorMetadata(torch.from_numpy(sizes.astype(np.int32)), torch.from_numpy(offs.astype(np.int32)),
                                torch.from_numpy(np.stack(bo_rows)), torch.from_numpy(np.stack(bs_rows)))


@dataclass
class Routing:
    vals: torch.Tensor  # [T,k] gate values (softmax over the kept logits)
    indx: torch.Tensor  # [T,k] int32 expert ids, value-descending
    bitmatrix: torch.Tensor  # [T, words] int32 view of uint32 words
    meta: BitmatrixMetadata
    ragged: RaggedTensorMetadata
    gather_indx: torch.Tensor  # [R] int32 token row feeding sorted row i
    scatter_indx: torch.Tensor  # [R] int32 flat position t*k+j receiving sorted row i
    gammas: torch.Tensor  # [R] gate value of sorted row i


def routing(logits: torch.Tensor, k: int, apply_softmax: bool = True) -> Routing:
    """Router + metadata + glue, composed as tests/test_distributed.py:203-210 composes them."""
    vals, indx, bits = topk(logits, k, apply_softmax)
    E = logits.shape[1]
    meta = make_bitmatrix_metadata(indx, E)
    R = indx.numel()
    ragged = make_ragged_tensor_metadata(meta.col_sum, R)
    col = meta.col_sorted_indx
    gather = torch.div(col, k, rounding_mode="trunc").to(torch.int32)
    scatter = col.clone()
    safe = col.clamp(min=0).to(torch.int64)
    gam = vals.reshape(-1)[safe]
    gam = torch.where(col >= 0, gam, torch.zeros_like(gam))
    return Routing(vals, indx, bits, meta, ragged, gather, scatter, gam)
