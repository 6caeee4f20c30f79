"""Legacy names of the routing / matmul API (`routing`, `RoutingData`, `GatherIndx`, `ScatterIndx`,
`matmul_ogs`), defined in terms of the current functions exactly as
python/triton_kernels/tests/test_distributed.py:203-220 composes them:

    sparse   = topk(logits, k)                                   vals / indx / histogram / permutations
    metadata = make_ragged_tensor_metadata(col_sum, T*k)
    gather   = col_sorted_indx // k ;  scatter = col_sorted_indx ;  gate_scal = vals.flatten()[col_sorted_indx]
    y        = matmul(x, w, bias, metadata, gather_indx=gather, scatter_indx=scatter, gammas=...)
    out      = reduce(y.view(T, k, -1), dim=1)                   when scattering

`routing` obtains all of it from ONE fused routing pass (three kernel launches).
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from .matmul import FusedActivation, PrecisionConfig, matmul
from .reduce import reduce
from .tensor import RaggedTensorMetadata
from .tensor_details.ragged_tensor import _alloc
from .topk import _topk_route


@dataclass
class GatherIndx:
    src_indx: torch.Tensor  # [R] int32: for expert-sorted row i, the flat position t*k+j it reads
    dst_indx: torch.Tensor  # [R] int32: inverse permutation


@dataclass
class ScatterIndx:
    src_indx: torch.Tensor  # [R] int32: for flat position t*k+j, its expert-sorted row
    dst_indx: torch.Tensor  # [R] int32: for expert-sorted row i, the flat position it writes


@dataclass
class RoutingData:
    gate_scal: torch.Tensor  # [R] gate value of each expert-sorted row
    expt_hist: torch.Tensor  # [E] int32 tokens per expert
    n_expts_tot: int
    n_expts_act: int
    expt_data: RaggedTensorMetadata
    token_indx: torch.Tensor | None = None  # [R] int32 token feeding each expert-sorted row (= src_indx // k)
    expt_indx: torch.Tensor | None = None  # [T, k] int16 selected experts, value-descending
    gate_vals: torch.Tensor | None = None  # [T, k] gate values
    # every token has exactly k routed rows (the router chose them itself: no caller-provided indices, which may hold
    # dropped entries, and no row mask); only then may the scatter-GEMM also sum a token's rows
    all_rows_live: bool = False


def routing(logits, n_expts_act, apply_softmax: bool = True, expt_indx=None, n_rows=None):
    """Router for a mixture-of-experts layer: returns `(RoutingData, GatherIndx, ScatterIndx)`."""
    T, E = logits.shape
    k = n_expts_act
    ragged = _alloc(E, T * k, logits.device)
    vals, indx, _mask, r = _topk_route(logits, k, apply_softmax, expt_indx, n_rows, want_meta=True, want_extras=True,
                                       ragged=ragged)
    slice_offs, block_offs, sched, _ = ragged
    md = RaggedTensorMetadata(r["col_sum"], slice_offs, block_offs, sched)
    col, row = r["col_sorted_indx"], r["row_sorted_indx"]
    rdata = RoutingData(gate_scal=r["gammas"], expt_hist=r["col_sum"], n_expts_tot=E, n_expts_act=k, expt_data=md,
                        token_indx=r["gather_indx"], expt_indx=indx, gate_vals=vals,
                        all_rows_live=expt_indx is None and n_rows is None)
    return rdata, GatherIndx(src_indx=col, dst_indx=row), ScatterIndx(src_indx=row, dst_indx=col)


def matmul_ogs(x, w, bias, routing_data: RoutingData | None = None, gather_indx: GatherIndx | None = None,
               scatter_indx: ScatterIndx | None = None, precision_config: PrecisionConfig | None = None, betas=None,
               gammas=None, fused_activation: FusedActivation | None = None, **kwargs):
    """`matmul` over the experts of `routing_data`; with `scatter_indx` the k expert rows of every token
    are summed, so the result has one row per token.  At decode shapes (tiled MXFP4 weights, a few rows per expert) the
    sum happens inside the GEMM launch; otherwise `reduce` follows it."""
    md = routing_data.expt_data if routing_data is not None else None
    g = None
    if gather_indx is not None:
        k = routing_data.n_expts_act if routing_data is not None else 1
        if routing_data is not None and routing_data.token_indx is not None:
            g = routing_data.token_indx
        else:
            g = torch.div(gather_indx.src_indx, k, rounding_mode="trunc").to(torch.int32)
    s = scatter_indx.dst_indx if scatter_indx is not None else None
    k = routing_data.n_expts_act if (routing_data is not None and scatter_indx is not None) else None
    # The fused combine counts a token's rows as they arrive and needs all k of them: routing with dropped entries
    # or a row mask, and metadata remapped to a rank's own experts, go through `reduce` instead.
    fuse = k if (k is not None and getattr(routing_data, "all_rows_live", False)
                 and getattr(md, "remapped_from", None) is None) else None
    y = matmul(x, w, bias, md, gather_indx=g, scatter_indx=s, precision_config=precision_config, betas=betas,
               gammas=gammas, fused_activation=fused_activation, _combine_k=fuse, **kwargs)
    if scatter_indx is None:
        return y
    combined = getattr(y, "_tk_combined", None)
    if combined is not None:  # decode shapes: the GEMM's last wave per token has already summed its k rows
        return combined
    out, _ = reduce(y.view(y.shape[0] // k, k, y.shape[-1]), dim=1)
    return out


from .torch_twins import matmul_ogs_torch, routing_torch  # noqa: E402,F401  (reference twins)
