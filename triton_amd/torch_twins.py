"""Plain-PyTorch statements of the operators: the `*_torch` names of the reference library.

The reference ships a torch twin next to every kernel-backed operator (`topk_torch` triton_kernels/topk.py:144,
`make_bitmatrix_metadata_torch` tensor_details/bitmatrix.py:157, `make_ragged_tensor_metadata_torch`
tensor_details/ragged_tensor.py:217, `matmul_torch` matmul.py:840, `swiglu_torch` swiglu.py:89, `reduce_torch`
reduce.py:1181, `downcast_to_mxfp_torch` / `upcast_from_mxfp_torch` numerics_details/mxfp.py:192,364) and user code
imports them to check results.  The ones here are written from the operators' definitions with ordinary torch ops on
whatever device their inputs live on.  They are reference implementations for callers to compare against: nothing in
this package's operator path calls them, and an operator whose HIP library is missing raises instead of using one.
"""
from __future__ import annotations

import itertools
from typing import Optional

import torch

from .tensor import BIT, RaggedTensorMetadata, SparseMatrix, Tensor, wrap_torch_tensor
from .tensor_details.bitmatrix import BitmatrixMetadata

_BLOCK = 32  # MX block length


# ---- routing ----------------------------------------------------------------------------------------------

def make_bitmatrix_metadata_torch(nonzero_indx: torch.Tensor, bitmatrix) -> BitmatrixMetadata:
    """Histogram of the selected columns and the two permutations between row-major order (flat position t*k + j) and
    column-grouped order; positions past the selected entries hold -1."""
    n_cols = bitmatrix.shape[1]
    flat = nonzero_indx.reshape(-1).to(torch.int64)
    live = flat >= 0
    n_live = int(live.sum())
    # stable sort by column with the dead entries pushed behind every column
    key = torch.where(live, flat, torch.full_like(flat, n_cols))
    order = torch.sort(key, stable=True).indices
    col_sorted = torch.full_like(flat, -1)
    col_sorted[:n_live] = order[:n_live]
    row_sorted = torch.full_like(flat, -1)
    row_sorted[order[:n_live]] = torch.arange(n_live, device=flat.device)
    col_sum = torch.bincount(flat[live], minlength=n_cols)[:n_cols]
    return BitmatrixMetadata(col_sum=col_sum.to(torch.int32), col_sorted_indx=col_sorted.to(torch.int32),
                             row_sorted_indx=row_sorted.to(torch.int32))


def topk_torch(x, k, apply_softmax: bool = True, dim: int = 1, y_indx: Optional[torch.Tensor] = None,
               n_rows: Optional[int] = None) -> SparseMatrix:
    """k largest entries per row, larger first, ties to the lower column; optional softmax over the kept values (fp32,
    rounded to x's dtype); rows from `n_rows` on select nothing (index -1, no bits)."""
    assert dim == 1 and not isinstance(x, Tensor) and x.ndim == 2
    T, E = x.shape
    n_rows = T if n_rows is None else int(n_rows)
    dev = x.device
    if y_indx is None:
        indx = torch.sort(x.to(torch.float32), dim=1, descending=True, stable=True).indices[:, :k]
    else:
        indx = y_indx.to(torch.int64)
    vals = torch.cat([torch.take_along_dim(x[:n_rows], indx[:n_rows], dim=1), x[n_rows:, :k]], dim=0)
    if apply_softmax:
        vals = torch.softmax(vals.to(torch.float32), dim=-1).to(x.dtype)
    indx = indx.to(torch.int32).clone()
    indx[n_rows:] = -1
    # one bit per (row, selected column), 32 columns to a word, stored word-major like the kernel's output
    words = (E + 31) // 32
    hit = torch.zeros((T, words * 32), dtype=torch.bool, device=dev)
    live = indx >= 0
    rows = torch.arange(T, device=dev)[:, None].expand_as(indx)
    hit[rows[live], indx[live].to(torch.int64)] = True
    weights = torch.ones(32, dtype=torch.int64, device=dev) << torch.arange(32, dtype=torch.int64, device=dev)
    packed = (hit.view(T, words, 32).to(torch.int64) * weights).sum(-1)
    packed = torch.where(packed >= 2**31, packed - 2**32, packed).to(torch.int32)
    data = torch.zeros((words, (T + 31) // 32 * 32), dtype=torch.int32, device=dev)
    data[:, :T] = packed.t()
    bits = torch.transpose(data, 0, 1)[:T].view(torch.uint32)
    mask = wrap_torch_tensor(bits, dtype=BIT, shape=[T, E])
    return SparseMatrix(vals=vals, indx=indx, mask=mask, mask_metadata=make_bitmatrix_metadata_torch(indx, mask))


def make_ragged_tensor_metadata_torch(slice_sizes: torch.Tensor, n_total_rows: int) -> RaggedTensorMetadata:
    """Row offsets of the slices and, for every block size, the block offsets and the block schedule: entry i names the
    slice (low 16 bits) and the block inside it (high 16 bits) of the i-th block, -1 past the last block."""
    assert slice_sizes.ndim == 1
    dev = slice_sizes.device
    n_slices = slice_sizes.shape[0]
    max_n_blocks = RaggedTensorMetadata.max_n_blocks(n_slices, n_total_rows)
    sizes = slice_sizes.to(torch.int64)
    zero = torch.zeros(1, dtype=torch.int64, device=dev)
    slice_offs = torch.cat([zero, torch.cumsum(sizes, 0)])
    block_offs, schedules = [], []
    slot = torch.arange(max_n_blocks, dtype=torch.int64, device=dev)
    for bs in RaggedTensorMetadata.block_sizes():
        offs = torch.cat([zero, torch.cumsum((sizes + bs - 1) // bs, 0)])
        # slot i belongs to the last slice whose first block is <= i (empty slices share an offset with their successor)
        owner = torch.searchsorted(offs[1:], slot, right=True).clamp_max(max(n_slices - 1, 0))
        sched = ((slot - offs[owner]) << 16) | owner
        sched = torch.where(slot < offs[-1], sched, torch.full_like(sched, -1))
        block_offs.append(offs)
        schedules.append(sched)
    return RaggedTensorMetadata(slice_sizes, slice_offs.to(torch.int32), torch.stack(block_offs).to(torch.int32),
                                torch.stack(schedules).to(torch.int32))


def routing_torch(logits, n_expts_act, apply_softmax: bool = True, expt_indx=None, n_rows=None):
    """`legacy.routing` from the torch twins: (RoutingData, GatherIndx, ScatterIndx)."""
    from .legacy import GatherIndx, RoutingData, ScatterIndx
    T, E = logits.shape
    k = n_expts_act
    sm = topk_torch(logits, k, apply_softmax=apply_softmax, y_indx=expt_indx, n_rows=n_rows)
    meta = sm.mask_metadata
    md = make_ragged_tensor_metadata_torch(meta.col_sum, T * k)
    col, row = meta.col_sorted_indx, meta.row_sorted_indx
    live = col >= 0
    safe = col.clamp_min(0).to(torch.int64)
    gate = torch.where(live, sm.vals.reshape(-1)[safe], torch.zeros((), dtype=sm.vals.dtype, device=logits.device))
    token = torch.where(live, (safe // k).to(torch.int32), torch.full_like(col, -1))
    rdata = RoutingData(gate_scal=gate, expt_hist=meta.col_sum, n_expts_tot=E, n_expts_act=k, expt_data=md, token_indx=token,
                        expt_indx=sm.indx, gate_vals=sm.vals)
    return rdata, GatherIndx(src_indx=col, dst_indx=row), ScatterIndx(src_indx=row, dst_indx=col)


# ---- element-wise ------------------------------------------------------------------------------------------

def swiglu_torch(a, alpha, precision_config):
    """out = g * sigmoid(alpha * g) * (l + 1) over interleaved (g, l) column pairs, g clamped from above and l from both
    sides when the config carries a limit."""
    limit = precision_config.limit
    gate, lin = a[..., 0::2], a[..., 1::2]
    if limit is not None:
        gate = gate.clamp(max=limit)
        lin = lin.clamp(min=-limit, max=limit)
    return gate * torch.sigmoid(alpha * gate) * (lin + 1)


def reduce_torch(x: torch.Tensor, dim: int, mask: Optional[torch.Tensor] = None, scale: Optional[torch.Tensor] = None,
                 x_mxscale: Optional[torch.Tensor] = None, x_flex=None, y_flex=None, y_flex_saturate_inf: bool = False,
                 postprocess_fn1=None, unpadded_batch_size=None):
    """Sum over `dim` in fp32 of x (dequantised when MX scales are given), entries weighted by `scale` and dropped where
    `mask` is false; the result takes x's dtype (requantised to MXFP8 along the last axis for MX inputs)."""
    dtype = x.dtype
    v = upcast_from_mxfp_torch(x, x_mxscale, torch.float32, axis=-1) if x_mxscale is not None else x.to(torch.float32)
    if x_flex is not None and getattr(x_flex, "scale", None) is not None:
        v = v * x_flex.scale
    if scale is not None:
        v = v * scale.to(torch.float32)
    if mask is not None:
        v = torch.where(mask.to(torch.bool), v, torch.zeros((), device=v.device))
    out = v.sum(dim=dim)
    if postprocess_fn1 is not None:
        out = postprocess_fn1(out)
    if y_flex is not None and getattr(y_flex, "expected_scale", None) is not None:
        out = out / y_flex.expected_scale
    if x_mxscale is not None:
        q, s = downcast_to_mxfp_torch(out, torch.float8_e4m3fn, axis=-1)
        return q.to(dtype), s
    return out.to(dtype), None


# ---- MX formats --------------------------------------------------------------------------------------------

_MAX_QUANT = {torch.uint8: 6.0, torch.float8_e5m2: 57344.0, torch.float8_e4m3fn: 448.0}
_E2M1_VALUES = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0)


def _e2m1_codes(q: torch.Tensor) -> torch.Tensor:
    """fp32 (already divided by the block scale) -> 4-bit e2m1 codes: round to nearest, ties to the even mantissa,
    magnitudes above 6 saturate."""
    mag = q.abs()
    grid = torch.tensor(_E2M1_VALUES, dtype=torch.float32, device=q.device)
    # nearest grid point; a tie picks the neighbour with an even code (codes 0, 2, 4, 6 have mantissa bit 0)
    hi = torch.searchsorted(grid, mag.contiguous(), right=False).clamp_max(7)
    lo = (hi - 1).clamp_min(0)
    d_lo, d_hi = mag - grid[lo], grid[hi] - mag
    pick_hi = (d_hi < d_lo) | ((d_hi == d_lo) & (hi % 2 == 0))
    code = torch.where(pick_hi, hi, lo)
    code = torch.where(mag.isnan(), torch.full_like(code, 7), code)
    sign = (q.view(torch.int32) >> 31) & 1
    return (code | (sign.to(code.dtype) << 3)).to(torch.uint8)


def downcast_to_mxfp_torch(src_tensor: torch.Tensor, out_quant_type: torch.dtype, axis: int, scale_dtype: torch.dtype = torch.uint8,
                           microblock_size: int = _BLOCK, expected_scale=None, DEQUANT_SCALE_ROUNDING_MODE=None):
    """Blocks of 32 along `axis` share one power-of-two scale (e8m0 byte = biased exponent): the block's largest
    magnitude divided by the format's largest value and rounded up to a power of two (ROUND_UP, the default), or divided
    by the format's largest power of two and rounded down (ROUND_DOWN); the values are divided by it and rounded to e2m1
    (two codes per byte, low nibble first) or fp8 (saturating)."""
    assert src_tensor.dtype in (torch.float32, torch.bfloat16, torch.float16)
    assert scale_dtype == torch.uint8 and microblock_size == _BLOCK
    round_down = DEQUANT_SCALE_ROUNDING_MODE is not None and getattr(DEQUANT_SCALE_ROUNDING_MODE, "name", "") == "ROUND_DOWN"
    fp4 = out_quant_type == torch.uint8
    ndim = src_tensor.ndim
    axis = axis % ndim
    src = src_tensor.transpose(axis, ndim - 1).to(torch.float32)
    if expected_scale is not None:
        es = expected_scale.to(device=src.device, dtype=torch.float32)
        src = src / (es if es.numel() == 1 else es[:, None, None])
    L = src.shape[-1]
    assert not fp4 or L % 2 == 0
    nb = (L + _BLOCK - 1) // _BLOCK
    padded = torch.nn.functional.pad(src, (0, nb * _BLOCK - L)).reshape(*src.shape[:-1], nb, _BLOCK)
    absmax = padded.abs().amax(dim=-1, keepdim=True)
    if round_down:  # the largest power of two the format holds takes the block maximum's place
        top = _MAX_QUANT[out_quant_type]
        bits = (absmax / 2.0**(torch.tensor(top).log2().floor().item())).view(torch.int32) & 0x7F800000
    else:
        bits = ((absmax / _MAX_QUANT[out_quant_type]).view(torch.int32) + 0x007FFFFF) & 0x7F800000
    scale_f = bits.view(torch.float32)
    quant = torch.where(scale_f == 0, torch.zeros_like(padded), padded / scale_f)
    quant = quant.reshape(*src.shape[:-1], nb * _BLOCK)[..., :L]
    if fp4:
        codes = _e2m1_codes(quant)
        out = codes[..., 0::2] | (codes[..., 1::2] << 4)
    else:
        lim = _MAX_QUANT[out_quant_type]
        out = quant.clamp(-lim, lim).to(out_quant_type)  # the conversion saturates
    scales = (bits >> 23).to(torch.uint8).squeeze(-1)
    return out.transpose(axis, ndim - 1), scales.transpose(axis, ndim - 1)


def upcast_from_mxfp_torch(tensor: torch.Tensor, scale: torch.Tensor, target_dtype: torch.dtype, axis: int):
    """value * 2**(scale byte - 127) per block of 32 along `axis`, clamped to the target type's finite range (an e5m2
    infinity stays infinite)."""
    assert scale.dtype == torch.uint8
    ndim = tensor.ndim
    axis = axis % ndim
    t = tensor.transpose(axis, ndim - 1)
    s = scale.transpose(axis, ndim - 1)
    if tensor.dtype == torch.uint8:
        grid = torch.tensor(_E2M1_VALUES + tuple(-v for v in _E2M1_VALUES), dtype=torch.float32, device=tensor.device)
        pair = torch.stack([t & 0xF, t >> 4], dim=-1).to(torch.int64)
        vals = grid[pair].reshape(*t.shape[:-1], t.shape[-1] * 2)
    else:
        vals = t.to(torch.float32)
    L = vals.shape[-1]
    factor = (s.to(torch.int32) << 23).view(torch.float32)
    factor = factor.repeat_interleave(_BLOCK, dim=-1)[..., :L]
    lim = torch.finfo(target_dtype)
    out = (vals * factor).clamp(lim.min, lim.max)
    if tensor.dtype == torch.float8_e5m2:
        out = torch.where(vals.isinf(), vals, out)
    return out.to(target_dtype).contiguous().transpose(axis, ndim - 1)


# ---- GEMM --------------------------------------------------------------------------------------------------

def _operands_as_multiplied(a, b, precision_config):
    """The operands as the GEMM sees them: MX operands dequantised to bf16 along K, flexpoint-scaled ones multiplied by
    their scale in fp32, everything else as stored."""
    from .tensor import convert_layout
    from .tensor_details.layout_details.strided import StridedLayout
    flex = precision_config.flex_ctx

    def plain(t, scale, k_axis, mx_scale):
        if mx_scale is not None:
            if isinstance(t, Tensor):
                t = convert_layout(t, StridedLayout(k_axis)).storage.data
            if isinstance(mx_scale, Tensor):
                mx_scale = convert_layout(mx_scale, StridedLayout(k_axis)).storage.data
            return upcast_from_mxfp_torch(t, mx_scale, torch.bfloat16, axis=k_axis)
        if isinstance(t, Tensor):
            t = t.storage.data
        return t.clone() if scale is None else t.to(torch.float32) * scale

    return (plain(a, flex.lhs_data.scale, a.ndim - 1, precision_config.a_mx_scale),
            plain(b, flex.rhs_data.scale, b.ndim - 2, precision_config.b_mx_scale))


def matmul_torch(a, b, bias, a_ragged_metadata: RaggedTensorMetadata | None = None,
                 b_ragged_metadata: RaggedTensorMetadata | None = None, gather_indx: torch.Tensor = None,
                 scatter_indx: torch.Tensor = None, precision_config=None, betas=None, gammas=None, round_x=None, round_y=None):
    """y[dst(r)] = round_y((x[src(r)] @ w[e(r)] + bias[e(r)] * beta_r) * gamma_r), one expert per slice of rows; with
    `b_ragged_metadata` the slices cut the reduction dimension instead and every slice yields its own [M, N] product."""
    from .matmul import PrecisionConfig
    precision_config = precision_config or PrecisionConfig()
    a, b = _operands_as_multiplied(a, b, precision_config)
    out_scale = precision_config.flex_ctx.out_data.expected_scale

    def finish(v):
        if out_scale is None:
            return v
        return v / out_scale if out_scale.numel() == 1 else v / out_scale[:, None, None]

    if b_ragged_metadata is not None:
        sizes = b_ragged_metadata.slice_sizes.tolist()
        xo, wo = a_ragged_metadata.slice_offs.tolist(), b_ragged_metadata.slice_offs.tolist()
        out = torch.zeros((len(sizes), a.shape[-2], b.shape[-1]), dtype=torch.float32, device=a.device)
        for e, n in enumerate(sizes):
            if n:
                out[e] = a[:, xo[e]:xo[e] + n].to(torch.float32) @ b[wo[e]:wo[e] + n, :].to(torch.float32)
        return finish(out)
    batched = a.ndim == 3
    assert not batched or (gather_indx is None and scatter_indx is None and b.ndim == 3 and b.shape[0] == a.shape[0])
    a3 = a if batched else a[None]
    b3 = b if b.ndim == 3 else b[None]
    if bias is not None and bias.ndim == 1:
        bias = bias[None]
    n_rows = a3.shape[1] if gather_indx is None else gather_indx.shape[0]
    if a_ragged_metadata is not None and not batched:
        ends = torch.cumsum(a_ragged_metadata.slice_sizes.to(torch.int64), 0).tolist()
        bounds = list(itertools.pairwise([0] + ends))
    else:
        bounds = [(0, a3.shape[1])] * b3.shape[0]
    acc_t = torch.float64 if a.dtype == b.dtype == torch.float64 else torch.float32
    y = torch.zeros((a3.shape[0], n_rows, b3.shape[-1]), dtype=a.dtype, device=a.device)
    for e, (lo, hi) in enumerate(bounds):
        src = torch.arange(lo, hi, device=a.device) if gather_indx is None else gather_indx[lo:hi].to(torch.int64)
        xb = a3[e if batched else 0][src]
        if round_x is not None:
            xb = round_x(xb, torch.arange(lo, hi, device=a.device))
        v = xb.to(acc_t) @ b3[e].to(acc_t)
        if bias is not None:
            v = v + (bias[e] if betas is None else bias[e] * betas[lo:hi, None])
        if gammas is not None:
            v = v * gammas[lo:hi, None]
        y[e if batched else 0, lo:hi] = v if round_y is None else round_y(v)
    if not batched:
        y = y[0]
    if scatter_indx is not None:
        out = torch.zeros((scatter_indx.shape[0], y.shape[-1]), dtype=y.dtype, device=a.device)
        live = scatter_indx != -1
        out[scatter_indx[live].to(torch.int64)] = y[live]
        y = out
    return finish(y)


def matmul_ogs_torch(x, w, bias, routing_data=None, gather_indx=None, scatter_indx=None, precision_config=None, betas=None,
                     gammas=None, round_x=None, round_y=None):
    """`legacy.matmul_ogs` from the torch twins (with `scatter_indx`: one row per token, the k expert rows summed)."""
    md = None if routing_data is None else routing_data.expt_data
    k = 1 if routing_data is None else routing_data.n_expts_act
    src = None
    if gather_indx is not None:  # flat position t*k + j of every expert-sorted row -> token t (-1 entries lie past the slices)
        src = torch.div(gather_indx.src_indx.clamp_min(0), k, rounding_mode="trunc")
    y = matmul_torch(x, w, bias, md, None, src, None if scatter_indx is None else scatter_indx.dst_indx, precision_config,
                     betas, gammas, round_x, round_y)
    if scatter_indx is None:
        return y
    return reduce_torch(y.view(y.shape[0] // k, k, -1), dim=1)[0]
