"""Ragged expert matmul host driver (mirrors `triton_kernels/matmul.py:40-142,245-766`).

    Y[dst(r), :] = act((X[src(r), :] @ W[e(r)]) * scales + bias[e(r), :]) * gammas[r]

Python validates, picks the tile (`opt_flags`), allocates the output with `torch.empty` and fills one
`tk_gemm_desc`; the HIP kernel behind `tk_moe_gemm` does the rest.  Supported operand combinations:

    activations  weights                        notes
    bf16         bf16                           K-contiguous weights are used in place; N-contiguous
                                                ones are re-laid out once (the copy is cached on the tensor)
    bf16         mxfp4 (uint8 e2m1 + e8m0)      dequantised in registers, bf16 MFMA, fp32 accumulate
    fp8 e4m3     fp8 e4m3 (+ fp32 row/col scales via a/b_mx_tensor_scale)
    mxfp8 e4m3   tiled mxfp4                    both operands in storage format on the scaled MFMA
    fp16         fp16                           fp16 MFMA, fp16 output
    other pairs of {bf16, fp16, e4m3, e5m2, mxfp8, mxfp4} activations x {bf16, fp16, e5m2, mxfp8, mxfp4} weights:
                                                the narrow operand without a native partner is expanded to bf16 / fp16 by
                                                the MX dequantiser kernel (activations per call, weights once, cached)

Options of the reference signature that this build rejects with NotImplementedError: `fused_comm`, the NVFP4 output epilogue, flexpoint
output / accumulator scales, split-k.  `betas`, `out_alpha` and `c_acc_in` are applied in the reference's epilogue order by the kernels with the shared epilogue
(tiled MXFP4 weights then run on the decode kernel's row blocks; `c_acc_in` must have the output's dtype).  Batched 3-D activations run as a ragged problem with equal slices.  Flexpoint input scales (`flex_ctx.lhs_data.scale`,
`flex_ctx.rhs_data.scale`) are folded into the per-row / per-column scales of the epilogue.  MXFP8 / MXFP4 output epilogues run as the bf16 GEMM followed by the
MX quantiser kernel on the same stream.
"""
from __future__ import annotations

import dataclasses
from dataclasses import dataclass
from enum import Enum, auto
from typing import Callable

import torch

from . import _native as nt
from .matmul_details.opt_flags import (InapplicableConstraint, OptFlags, make_opt_flags, scoped_opt_flags,  # noqa: F401
                                        scoped_opt_flags_constraints, set_idle_sms)
from .numerics import InFlexData, OutFlexData
from .specialize import FnSpecs
from .tensor import FP4, RaggedTensorMetadata, Tensor, convert_layout, torch_dtype_to_dtype, wrap_torch_tensor
from .tensor_details.layout_details.cdna4_scale import CDNA4MXScaleLayout
from .tensor_details.layout_details.gfx950_mx import GFX950FP8ValueLayout, GFX950MXScaleLayout, GFX950MXValueLayout
from .tensor_details.layout_details.strided import StridedLayout

MXFP_BLOCK_SIZE = 32


@dataclass(frozen=True)
class FusedActivation:
    specs: FnSpecs = FnSpecs.default()
    fn_args: tuple = tuple()


@dataclass(frozen=True)
class Epilogue:
    specs: FnSpecs = FnSpecs.default()
    fn_arg_values_matmul: tuple = tuple()
    fn_arg_values_finalize: tuple = tuple()
    effective_itemsize: float | None = None


class FnName(Enum):
    QUANTIZE_MXFP8 = auto()
    QUANTIZE_MXFP4 = auto()
    QUANTIZE_NVFP4 = auto()


@dataclass(frozen=True)
class FusedComm:
    """Fused all-gather / reduce-scatter store; multi-GPU only, rejected by `matmul` in this build."""
    out_handles: torch.Tensor
    map_dst_coord: object = None
    all_writes_issued: object = None
    reduce_rank: int = 0
    n_reduce_shards: int = 1


@dataclass(frozen=True)
class FlexCtx:
    lhs_data: InFlexData = InFlexData()
    rhs_data: InFlexData = InFlexData()
    out_data: OutFlexData = OutFlexData()
    acc_data: InFlexData = InFlexData()


@dataclass
class PrecisionConfig:
    max_num_imprecise_acc: int | None = None
    allow_tf32: bool = True
    flex_ctx: FlexCtx = FlexCtx()
    acc_scale: float = 1.0
    flexpoint_saturate_inf: bool = False
    report_quantization_err_fn: Callable | None = None
    a_mx_scale: torch.Tensor | Tensor | None = None
    a_mx_tensor_scale: torch.Tensor | None = None
    a_microblock_size: int | None = None
    b_mx_scale: torch.Tensor | Tensor | None = None
    b_mx_tensor_scale: torch.Tensor | None = None
    b_microblock_size: int | None = None
    c_mx_scale: torch.Tensor | Tensor | None = None
    c_microblock_size: int | None = None
    c_value_pack_factor: int = 1
    out_dtype: torch.dtype | None = None
    intermediate_out_dtype: torch.dtype | None = None
    enforce_bitwise_invariance: bool = False


def matmul_set_idle_sms(num_idle_sms):
    set_idle_sms(num_idle_sms)


_TILE_COUNTERS: dict = {}
_STATIC_TILES = False  # True: the persistent kernels walk their static tile schedule (for comparisons)


def _tile_counters(device: torch.device) -> torch.Tensor:
    """Zeroed int32 words the persistent kernels claim tiles with (`tk_gemm_desc.tile_counters`): one small buffer
    per (device, stream), made on first use and kept for the life of the process.  A kernel leaves the words zero, so
    launches in stream order share them; launches on different streams get different buffers.  (A buffer first made
    while a HIP graph is being captured belongs to the capture stream: graphs captured on one stream must not be
    replayed concurrently with each other.)"""
    key = (device.index, nt.stream_ptr(device))
    buf = _TILE_COUNTERS.get(key)
    if buf is None:
        buf = torch.zeros(32, dtype=torch.int32, device=device)
        _TILE_COUNTERS[key] = buf
    return buf


_COMBINE_COUNTERS: dict = {}
_COMBINE_COUNTER_WORDS = 1 << 16


def _combine_counters(device: torch.device) -> torch.Tensor:
    """Zeroed int32 words for the fused top-k combine (`tk_gemm_desc.combine_counters`), one buffer per (device, stream)
    like the tile counters; the kernel leaves them zero."""
    key = (device.index, nt.stream_ptr(device))
    buf = _COMBINE_COUNTERS.get(key)
    if buf is None:
        buf = torch.zeros(_COMBINE_COUNTER_WORDS, dtype=torch.int32, device=device)
        _COMBINE_COUNTERS[key] = buf
    return buf


def _flex_out_is_trivial(flex: FlexCtx) -> bool:
    return (flex.acc_data.scale is None and flex.out_data.expected_scale is None and flex.out_data.actual_scale is None
            and flex.out_data.checksum_scale is None)


_FP8_TYPES = (torch.float8_e4m3fn, torch.float8_e5m2)


def _strided_scale_data(scale) -> torch.Tensor:
    """The e8m0 bytes of an MX scale operand in logical (strided) order."""
    if isinstance(scale, Tensor):
        if isinstance(scale.storage.layout, CDNA4MXScaleLayout):
            scale = convert_layout(scale, StridedLayout(-2))
        if not isinstance(scale.storage.layout, StridedLayout):
            raise NotImplementedError(f"scale layout {type(scale.storage.layout).__name__} is not supported")
        return scale.storage.data
    return scale


def _cache_key(t: torch.Tensor):
    """What a cached re-layout of `t` is valid for: the storage address and the version counter.  The counter misses
    writes that bypass autograd's bookkeeping (`t.data.add_`, a kernel or collective writing through the raw
    pointer, a DLPack consumer): after such a write call `invalidate_weight_cache(t)`.  Tensors made under
    `torch.inference_mode` have no counter; they are keyed by address alone."""
    try:
        version = t._version
    except RuntimeError:
        version = None
    return (t.data_ptr(), version)


def invalidate_weight_cache(*tensors) -> None:
    """Drops the converted copies `matmul` keeps on weight tensors (the K-contiguous re-layout of N-contiguous bf16 /
    fp16 / fp8 weights, the 16-bit expansion of fp8 / MXFP8 weights, the converted scale layout of a `Tensor`
    wrapper).  Needed after the weights were changed in a way their version counter does not see: `w.data.add_()`,
    `w.data.copy_()`, an optimizer that updates `.data`, a checkpoint load or collective that writes through the raw
    pointer.  In-place torch operations on the tensor itself (`w.add_()`, `w.copy_()`) invalidate on their own."""
    for t in tensors:
        if t is None:
            continue
        for obj in (t, getattr(getattr(t, "storage", None), "data", None)):
            if obj is None:
                continue
            for name in ("_tk_k_contiguous", "_tk_expanded", "_tk_converted"):
                if hasattr(obj, name):
                    try:
                        delattr(obj, name)
                    except AttributeError:
                        pass


def _expanded_weights(w: torch.Tensor, scale, target: torch.dtype) -> torch.Tensor:
    """fp8 weights (with or without e8m0 scales along K) as a 16-bit float tensor, converted by the MX dequantiser ONCE
    and kept on the weight tensor (keyed as `_cache_key` says, for values and scales; `invalidate_weight_cache`)."""
    from .numerics_details.mxfp import upcast_from_mxfp
    sd = _strided_scale_data(scale) if scale is not None else None
    key = (_cache_key(w), None if sd is None else _cache_key(sd), target)
    cached = getattr(w, "_tk_expanded", None)
    if cached is not None and cached[0] == key:
        return cached[1]
    K = w.shape[-2]
    if K % MXFP_BLOCK_SIZE:
        raise NotImplementedError(f"fp8 weights that are expanded to {target} need K % 32 == 0 (got {K})")
    if sd is None:
        sd = torch.full((*w.shape[:-2], K // MXFP_BLOCK_SIZE, w.shape[-1]), 127, dtype=torch.uint8, device=w.device)
    conv = upcast_from_mxfp(w, sd, target, axis=-2)
    try:
        w._tk_expanded = (key, conv)
    except (AttributeError, RuntimeError):
        pass
    return conv


def _expand_operands(a, b, precision_config):
    """Operand pairs that have no kernel of their own run on the 16-bit kernels after the MX dequantiser kernel has
    expanded the narrow operand (exact: an e2m1 / e4m3 / e5m2 value times a power of two is a bf16 value while it stays in
    bf16's range, so the products the MFMA sees are those of the reference's in-kernel conversion):

      * fp8 (e4m3 / e5m2) or MXFP8 / MXFP4 activations with weights other than the native partners (e4m3 x e4m3, and
        MXFP8-e4m3 x tiled MXFP4 on the scaled MFMA) are expanded per call;
      * MXFP8 weights (fp8 values + `b_mx_scale`) and plain e5m2 weights are expanded once and cached on the tensor.

    Returns the (possibly replaced) operands and precision config."""
    from .numerics_details.mxfp import upcast_from_mxfp
    pc = precision_config
    a_data = a.storage.data if isinstance(a, Tensor) else a
    b_data = b.storage.data if isinstance(b, Tensor) else b
    b_strided = not isinstance(b, Tensor) or isinstance(b.storage.layout, StridedLayout)
    b_tiled_mx = isinstance(b, Tensor) and isinstance(b.storage.layout, GFX950MXValueLayout)
    b_tiled_fp8 = isinstance(b, Tensor) and isinstance(b.storage.layout, GFX950FP8ValueLayout)
    a_fp8 = a_data.dtype in _FP8_TYPES
    a_mx = pc.a_mx_scale is not None
    a_fp4 = a_mx and (a_data.dtype == torch.uint8 or (isinstance(a, Tensor) and a.dtype == FP4))
    target = torch.float16 if torch.float16 in (a_data.dtype, b_data.dtype) else torch.bfloat16
    if b_data.dtype in _FP8_TYPES and b_strided:
        native = b_data.dtype == torch.float8_e4m3fn and pc.b_mx_scale is None and a_data.dtype == torch.float8_e4m3fn and not a_mx
        if not native:
            b = _expanded_weights(b_data, pc.b_mx_scale, target)
            b_data = b
            pc = dataclasses.replace(pc, b_mx_scale=None)
    if a_fp8 or a_fp4:
        native = (a_data.dtype == torch.float8_e4m3fn
                  and ((a_mx and b_tiled_mx) or (not a_mx and (b_tiled_fp8 or b_data.dtype == torch.float8_e4m3fn))))
        if not native:
            if a_data.ndim != 2:
                raise NotImplementedError("narrow activations that are expanded must be 2-D")
            K = a_data.shape[-1] * (2 if a_fp4 else 1)
            if K % MXFP_BLOCK_SIZE:
                raise NotImplementedError(f"{a_data.dtype} activations with these weights need K % 32 == 0 (got {K})")
            if a_mx:
                sd = _strided_scale_data(pc.a_mx_scale)
                assert sd.dtype == torch.uint8, f"Unsupported microscale dtype {sd.dtype}"
            else:
                sd = torch.full((a_data.shape[0], K // MXFP_BLOCK_SIZE), 127, dtype=torch.uint8, device=a_data.device)
            a = upcast_from_mxfp(a_data, sd, target, axis=-1)
            pc = dataclasses.replace(pc, a_mx_scale=None)
    return a, b, pc



def _k_contiguous(w: torch.Tensor) -> torch.Tensor:
    """[E, K, N] weights with unit stride along K (each output column contiguous in memory).  Weights that arrive
    N-contiguous (a plain torch [E, K, N] tensor) are re-laid out ONCE: the copy is kept on the tensor object, keyed
    by the tensor's storage address and version counter, so that an in-place torch update of the weights makes a new
    copy.  Writes that the version counter does not see (`w.data.add_()`, raw-pointer writes) need
    `invalidate_weight_cache(w)`.  The copy doubles the memory of such weights; callers that mind convert them up
    front (`w.transpose(-1, -2).contiguous().transpose(-1, -2)`, or `convert_layout(w, StridedLayout(-2))`) and
    drop the original."""
    if w.stride(-2) == 1 and (w.shape[-2] == 1 or w.stride(-1) >= w.shape[-2]):
        return w
    key = _cache_key(w)
    cached = getattr(w, "_tk_k_contiguous", None)
    if cached is not None and cached[0] == key:
        return cached[1]
    conv = w.transpose(-1, -2).contiguous().transpose(-1, -2)
    try:
        w._tk_k_contiguous = (key, conv)
    except (AttributeError, RuntimeError):
        pass  # a tensor subclass without a __dict__: converted per call
    return conv


def _matmul_mx_out(a, b, bias, a_ragged_metadata, gather_indx, scatter_indx, precision_config, gammas, c,
                   fused_activation, epilogue, betas=None, out_alpha=None, c_acc_in=None):
    """`Epilogue(FnSpecs(QUANTIZE_MXFP8 | QUANTIZE_MXFP4, ...))` with `precision_config.c_mx_scale`
    (triton_kernels/matmul.py:53-56,364-369,500-505; kernel side matmul_details/_matmul.py:593-637): the output is
    quantised along N in blocks of 32, values in `out_dtype` (float8 or packed e2m1 in uint8) and one e8m0 scale
    byte per block written to `c_mx_scale` [rows, ceil(N_out / 32)].  Here the GEMM writes bf16 and the MX
    quantiser kernel follows on the same stream, so the values are quantised from the bf16-rounded result (the
    reference quantises the fp32 accumulator: a code can differ by one step where the bf16 rounding crosses a
    quantisation threshold)."""
    import dataclasses
    from .numerics_details.mxfp import downcast_to_mxfp
    scale_out = precision_config.c_mx_scale
    if scale_out is None:
        raise ValueError("an MX-quantising epilogue needs precision_config.c_mx_scale to receive the block scales")
    if precision_config.c_microblock_size not in (None, MXFP_BLOCK_SIZE):
        raise NotImplementedError(f"output microblock size {precision_config.c_microblock_size} is not supported (32 only)")
    fp4 = epilogue.specs.name == FnName.QUANTIZE_MXFP4.name
    out_dtype = precision_config.out_dtype
    if out_dtype not in ((torch.uint8, ) if fp4 else (torch.float8_e4m3fn, torch.float8_e5m2)):
        raise ValueError(f"epilogue {epilogue.specs.name} does not produce out_dtype {out_dtype}")
    if isinstance(scale_out, Tensor):
        if not isinstance(scale_out.storage.layout, StridedLayout):
            raise NotImplementedError(f"output scale layout {type(scale_out.storage.layout).__name__} is not supported")
        scale_data = scale_out.storage.data
    else:
        scale_data = scale_out
    assert scale_data.dtype == torch.uint8, f"Unsupported output microscale dtype {scale_data.dtype}"
    plain = dataclasses.replace(precision_config, c_mx_scale=None, out_dtype=torch.bfloat16)
    y = matmul(a, b, bias, a_ragged_metadata, None, gather_indx, scatter_indx, plain, betas, gammas, out_alpha, None, None,
               fused_activation, None, c_acc_in)
    n_out = y.shape[-1]
    if n_out % MXFP_BLOCK_SIZE != 0:
        raise NotImplementedError(f"MX-quantised output needs N_out % 32 == 0 (got {n_out})")
    assert tuple(scale_data.shape[-2:]) == (y.shape[0], n_out // MXFP_BLOCK_SIZE), \
        f"c_mx_scale must be [{y.shape[0]}, {n_out // MXFP_BLOCK_SIZE}], got {tuple(scale_data.shape)}"
    vals, scales = downcast_to_mxfp(y, out_dtype, axis=-1)
    scale_data.view(scales.shape).copy_(scales)
    # (the reference also records c_microblock_size / c_value_pack_factor on the caller's PrecisionConfig,
    # triton_kernels/matmul.py:364-369; nothing here reads them back, and the caller's object is left as it was given)
    if c is not None:
        assert tuple(c.shape[-2:]) == tuple(vals.shape) and c.dtype == vals.dtype
        c.view(vals.shape).copy_(vals)
        return c
    return vals


def _localise_remapped_metadata(md: RaggedTensorMetadata, n_local: int, n_rows: int) -> RaggedTensorMetadata:
    """Metadata from `remap_ragged_tensor_metadata` as the kernels need it.  The reference's kernel takes the weight
    tensor's slice count as the number of slices (`n_valid_slices`, matmul.py:658), looks rows up through the kept
    slices' unchanged offsets and never uses the (source-tensor) block offsets for scheduling; the kernels here order
    tiles by them, so block offsets and schedule are rebuilt for the `n_local` kept slices (one small launch) while
    sizes and row offsets are taken as remapped.  As in the reference this assumes that `slice_map` numbers the kept
    slices 0..n_local-1 in their original order."""
    from .tensor_details.ragged_tensor import make_ragged_tensor_metadata
    assert n_local <= md.n_slices, f"{n_local} weight slices for metadata remapped from {md.n_slices} slices"
    sizes = md.slice_sizes[:n_local].clamp_min(0)
    local = make_ragged_tensor_metadata(sizes, n_rows)
    return RaggedTensorMetadata(sizes, md.slice_offs[:n_local + 1], local.block_offs_data, local.block_schedule_data)


_BATCH_METADATA = {}


def _matmul_batched(a, b, bias, a_ragged_metadata, gather_indx, scatter_indx, precision_config, betas, gammas, out_alpha, c,
                    fused_comm, fused_activation, epilogue, c_acc_in):
    """Batched mode (triton_kernels/matmul.py:270-277): a [B, M, K] x b [B, K, N] -> [B, M, N], batch i with weight i.
    It is the ragged problem with B slices of exactly M rows, so it runs on the ragged kernels with metadata built
    once per (B, M) and kept; no gather, scatter or ragged metadata of the caller's own."""
    assert gather_indx is None, "gather not supported in batched mode"
    assert scatter_indx is None, "scatter not supported in batched mode"
    assert a_ragged_metadata is None, "x cannot be ragged in batched mode"
    assert fused_comm is None, "fused comm is not supported in batched mode"
    b_data = b.storage.data if isinstance(b, Tensor) else b
    assert len(b.shape) == 3 and b.shape[0] == a.shape[0], "batched mode needs one weight matrix per batch"
    del b_data
    B, M, K = a.shape
    key = (B, M, str(a.device))
    md = _BATCH_METADATA.get(key)
    if md is None:
        from .tensor import make_ragged_tensor_metadata
        md = make_ragged_tensor_metadata(torch.full((B, ), M, dtype=torch.int32, device=a.device), B * M)
        if len(_BATCH_METADATA) >= 16:
            _BATCH_METADATA.pop(next(iter(_BATCH_METADATA)))
        _BATCH_METADATA[key] = md
    if gammas is not None:
        gammas = gammas.repeat(B) if gammas.shape[0] == M else gammas
    if bias is not None and bias.ndim == 1:
        bias = bias[None].expand(B, -1)
    c2 = None
    if c is not None:
        assert c.ndim == 3 and c.shape[0] == B and c.is_contiguous()
        c2 = c.view(B * M, c.shape[-1])
    y = matmul(a.reshape(B * M, K), b, bias, md, None, None, None, precision_config, betas, gammas, out_alpha, c2, None,
               fused_activation, epilogue, c_acc_in)
    return y.view(B, M, y.shape[-1]) if c is None else c


def _matmul_ragged_k(a, b, bias, a_ragged_metadata, b_ragged_metadata, gather_indx, scatter_indx, precision_config, betas,
                     gammas, out_alpha, c, fused_comm, fused_activation, epilogue, c_acc_in):
    """The reduction dimension is ragged (triton_kernels/matmul.py:376-384): one [M, N] output per slice,
    out[e] = a[:, xo[e] : xo[e] + k_e] @ b[wo[e] : wo[e] + k_e, :] with k_e = b_ragged_metadata.slice_sizes[e], xo / wo the
    slice offsets of a's and b's metadata (torch statement: triton_kernels/matmul.py:852-875).  This is the expert
    weight gradient dW[e] = x_e^T @ dy_e.  Dense bf16 / fp16 operands only; no bias (the reference's own test passes
    none for this mode, tests/test_matmul.py:469), gather, scatter, scales or epilogue."""
    assert gather_indx is None and scatter_indx is None  # triton_kernels/matmul.py:279-281
    if a_ragged_metadata is None:
        raise ValueError("ragged-K matmul needs a_ragged_metadata as well (the slice offsets of a along K)")
    for what, v in (("bias", bias), ("betas", betas), ("gammas", gammas), ("out_alpha", out_alpha), ("fused_comm", fused_comm),
                    ("c_acc_in", c_acc_in)):
        if v is not None:
            raise NotImplementedError(f"{what} is not supported with b_ragged_metadata")
    if fused_activation is not None and fused_activation.specs.fn is not None:
        raise NotImplementedError("a fused activation is not supported with b_ragged_metadata")
    if epilogue is not None and (epilogue.specs.fn is not None or epilogue.specs.name != "dflt"):
        raise NotImplementedError("an epilogue is not supported with b_ragged_metadata")
    pc = precision_config or PrecisionConfig()
    if pc.a_mx_scale is not None or pc.b_mx_scale is not None or pc.c_mx_scale is not None:
        raise NotImplementedError("MX operands are not supported with b_ragged_metadata")
    if not (_flex_out_is_trivial(pc.flex_ctx) and pc.flex_ctx.lhs_data.scale is None and pc.flex_ctx.rhs_data.scale is None):
        raise NotImplementedError("flexpoint scales are not supported with b_ragged_metadata")
    if isinstance(a, Tensor):
        a = a.storage.data
    if isinstance(b, Tensor):
        if not isinstance(b.storage.layout, StridedLayout):
            raise NotImplementedError(f"weight layout {type(b.storage.layout).__name__} is not supported with b_ragged_metadata")
        b = b.storage.data
    if a.ndim != 2 or b.ndim != 2:
        raise NotImplementedError("ragged-K matmul takes 2-D operands")
    nt.require_gpu(a, "a")
    if a.dtype != b.dtype or a.dtype not in (torch.bfloat16, torch.float16):
        raise NotImplementedError(f"ragged-K matmul takes bf16 or fp16 operands of one type (got {a.dtype} and {b.dtype})")
    out_dtype = pc.out_dtype or a.dtype
    if out_dtype not in (torch.bfloat16, torch.float16, torch.float32):
        raise NotImplementedError(f"output dtype {out_dtype} is not supported with b_ragged_metadata")
    n_slices = b_ragged_metadata.n_slices
    assert a_ragged_metadata.n_slices == n_slices
    M, N = a.shape[0], b.shape[1]
    if c is None:
        c = torch.empty((n_slices, M, N), dtype=out_dtype, device=a.device)
    else:
        assert c.shape == (n_slices, M, N) and c.dtype == out_dtype and (N == 0 or c.stride(-1) == 1)
    d = nt.RaggedKDesc()
    d.a, d.dtype = a.data_ptr(), nt.TORCH_TO_TK[a.dtype]
    d.a_stride_m, d.a_stride_k = a.stride(0), a.stride(1)
    d.b = b.data_ptr()
    d.b_stride_k, d.b_stride_n = b.stride(0), b.stride(1)
    d.y, d.y_dtype = c.data_ptr(), nt.TORCH_TO_TK[out_dtype]
    d.y_stride_e, d.y_stride_m = c.stride(0), c.stride(1)
    d.M, d.N, d.n_slices = M, N, n_slices
    d.a_k_extent, d.b_k_extent = a.shape[1], b.shape[0]
    sizes, a_offs, b_offs = b_ragged_metadata.slice_sizes, a_ragged_metadata.slice_offs, b_ragged_metadata.slice_offs
    assert sizes.dtype == a_offs.dtype == b_offs.dtype == torch.int32
    assert sizes.is_contiguous() and a_offs.is_contiguous() and b_offs.is_contiguous()
    d.slice_sizes, d.a_slice_offs, d.b_slice_offs = sizes.data_ptr(), a_offs.data_ptr(), b_offs.data_ptr()
    with nt.on_device(a.device):
        nt.check(nt.lib().tk_ragged_k_gemm(d, nt.stream_ptr(a.device)), "tk_ragged_k_gemm")
    return c


def matmul(a, b, bias, a_ragged_metadata: RaggedTensorMetadata | None = None,
           b_ragged_metadata: RaggedTensorMetadata | None = None, gather_indx: torch.Tensor | None = None,
           scatter_indx: torch.Tensor | None = None, precision_config: PrecisionConfig | None = None,
           betas: torch.Tensor | None = None, gammas: torch.Tensor | None = None, out_alpha: float | None = None,
           c: torch.Tensor | None = None, fused_comm: FusedComm | None = None,
           fused_activation: FusedActivation | None = None, epilogue: Epilogue | None = None,
           c_acc_in: torch.Tensor | None = None, *, _combine_k: int | None = None):
    """
    Y[:, :] = 0
    for e in experts:
        Y[idxs_y_m(e), :] += matmul(X[idxs_x_m(e), :], W[e, :, :])

    `_combine_k` (used by `legacy.matmul_ogs`, not part of the reference's signature): with `scatter_indx` mapping rows
    to flat positions t * k + j, the decode kernel may also sum the k rows of every token; the result is then attached to
    the returned tensor as `._tk_combined` ([tokens, N]) and the caller skips its `reduce`.  The caller vouches that
    EVERY token has exactly k routed rows: a token with fewer leaves its arrival counter non-zero for the next launch.
    """
    if b_ragged_metadata is not None:
        return _matmul_ragged_k(a, b, bias, a_ragged_metadata, b_ragged_metadata, gather_indx, scatter_indx, precision_config,
                                betas, gammas, out_alpha, c, fused_comm, fused_activation, epilogue, c_acc_in)
    a_data = a.storage.data if isinstance(a, Tensor) else a
    if a_data.ndim == 3:
        return _matmul_batched(a_data, b, bias, a_ragged_metadata, gather_indx, scatter_indx, precision_config, betas, gammas,
                               out_alpha, c, fused_comm, fused_activation, epilogue, c_acc_in)
    if fused_comm is not None:
        raise NotImplementedError("fused_comm is a multi-GPU feature and is not supported")
    # betas / out_alpha / c_acc_in (triton_kernels/matmul.py:251-258; epilogue order matmul_details/_matmul.py:547-559,
    # 581-591) are served by the kernels with the shared epilogue; see `extras` below
    extras = betas is not None or out_alpha is not None or c_acc_in is not None
    if c_acc_in is not None and scatter_indx is not None:
        raise AssertionError("c_acc_in + scatter is not supported.")  # triton_kernels/matmul.py:531
    if precision_config is None:
        precision_config = PrecisionConfig()
    if fused_activation is None:
        fused_activation = FusedActivation(FnSpecs.default(), tuple())
    if epilogue is None:
        epilogue = Epilogue(FnSpecs.default(), tuple(), tuple(), False)
    a, b, precision_config = _expand_operands(a, b, precision_config)
    # MXFP8 activations (`a_mx_scale`): e4m3 values with one e8m0 scale per 32 k, multiplied with tiled MXFP4 weights
    # on the scaled MFMA (triton_kernels/matmul.py:130-132,783-795)
    a_scale = precision_config.a_mx_scale
    mx_act = a_scale is not None
    if mx_act:
        if isinstance(a_scale, Tensor):
            if not isinstance(a_scale.storage.layout, StridedLayout):
                raise NotImplementedError(f"activation scale layout {type(a_scale.storage.layout).__name__} is not supported")
            a_scale = a_scale.storage.data
        if not (isinstance(b, Tensor) and isinstance(b.storage.layout, GFX950MXValueLayout)):
            raise NotImplementedError("MX-quantised activations (a_mx_scale) need MXFP4 weights in the tiled layout "
                                      "(convert them with make_default_matmul_mxfp4_w_layout)")
        assert a_scale.dtype == torch.uint8, f"Unsupported microscale dtype {a_scale.dtype}"
        assert precision_config.a_microblock_size in (None, MXFP_BLOCK_SIZE), \
            f"Unsupported microscale block size {precision_config.a_microblock_size}"
    mx_out_fused = False
    if epilogue.specs.name in (FnName.QUANTIZE_MXFP8.name, FnName.QUANTIZE_MXFP4.name):
        # with MXFP8 activations the kernel quantises its fp32 accumulator itself; otherwise the bf16 GEMM is followed
        # by the MX quantiser
        mx_out_fused = (mx_act and epilogue.specs.name == FnName.QUANTIZE_MXFP8.name
                        and precision_config.out_dtype == torch.float8_e4m3fn and precision_config.c_mx_scale is not None
                        and precision_config.c_microblock_size in (None, MXFP_BLOCK_SIZE))
        if not mx_act and not extras:
            # bf16 activations x tiled MXFP4 weights: the prefill kernel quantises its fp32 accumulator to e4m3, e5m2 or
            # packed e2m1 (matmul_details/_matmul.py:593-637); other weight layouts take the two-step path below
            fp4_out = epilogue.specs.name == FnName.QUANTIZE_MXFP4.name
            n_out = b.shape[-1] // fused_activation.specs.reduction_n
            a_plain = a.storage.data if isinstance(a, Tensor) else a
            mx_out_fused = (isinstance(b, Tensor) and isinstance(b.storage.layout, GFX950MXValueLayout) and a_plain.dtype == torch.bfloat16
                            and a_plain.ndim == 2 and precision_config.c_mx_scale is not None
                            and precision_config.c_microblock_size in (None, MXFP_BLOCK_SIZE)
                            and precision_config.out_dtype in ((torch.uint8, ) if fp4_out else (torch.float8_e4m3fn, torch.float8_e5m2))
                            and n_out % MXFP_BLOCK_SIZE == 0 and b_ragged_metadata is None
                            and (a_ragged_metadata is None or a_ragged_metadata.n_slices <= 1024)
                            and (c is None or (c.ndim == 2 and c.stride(0) % 8 == 0 and c.data_ptr() % 8 == 0)))
        if mx_out_fused and extras:
            raise NotImplementedError("betas / out_alpha / c_acc_in are not supported together with the fused MX-output epilogue")
        if not mx_out_fused:
            return _matmul_mx_out(a, b, bias, a_ragged_metadata, gather_indx, scatter_indx, precision_config, gammas, c,
                                  fused_activation, epilogue, betas, out_alpha, c_acc_in)
    elif epilogue.specs.fn is not None or epilogue.specs.name != "dflt" or precision_config.c_mx_scale is not None:
        raise NotImplementedError(f"epilogue {epilogue.specs.name!r} is not supported (MXFP8 / MXFP4 output quantisation only)")
    flex = precision_config.flex_ctx
    if not _flex_out_is_trivial(flex):
        raise NotImplementedError("flexpoint output / accumulator scales are not supported (outputs are bf16)")
    if isinstance(a, Tensor):
        a = a.storage.data
    a = flex.lhs_data.reinterpret(a)
    assert a.ndim == 2
    nt.require_gpu(a, "a")
    # ---- weights -------------------------------------------------------------------------------
    b_scale = precision_config.b_mx_scale
    if not isinstance(b, Tensor):
        b = wrap_torch_tensor(b, dtype=FP4 if b.dtype == torch.uint8 else None)
    tiled = isinstance(b.storage.layout, GFX950MXValueLayout)
    tiled_fp8 = isinstance(b.storage.layout, GFX950FP8ValueLayout)
    if not tiled and not tiled_fp8 and not isinstance(b.storage.layout, StridedLayout):
        raise NotImplementedError(f"weight layout {type(b.storage.layout).__name__} is not supported")
    if b_scale is not None and not isinstance(b_scale, Tensor):
        b_scale = wrap_torch_tensor(b_scale)
    if b_scale is not None and isinstance(b_scale.storage.layout, CDNA4MXScaleLayout):
        # the reference's scale pre-shuffle: converted once to the order that goes with the values' layout and
        # kept on the wrapper (weights are static; re-wrap the tensor after changing its storage in place)
        want = GFX950MXScaleLayout() if tiled else StridedLayout(-2)
        cached = getattr(b_scale, "_tk_converted", None)
        if cached is None or cached[0] != want:
            cached = (want, convert_layout(b_scale, want))
            b_scale._tk_converted = cached
        b_scale = cached[1]
    if b_scale is not None:
        if tiled != isinstance(b_scale.storage.layout, GFX950MXScaleLayout):
            raise NotImplementedError("tiled MXFP4 values go with tiled scales (convert both with convert_layout)")
        if not tiled and not isinstance(b_scale.storage.layout, StridedLayout):
            raise NotImplementedError(f"scale layout {type(b_scale.storage.layout).__name__} is not supported")
        assert b_scale.storage.data.dtype == torch.uint8, f"Unsupported microscale dtype {b_scale.storage.data.dtype}"
        assert precision_config.b_microblock_size is None or precision_config.b_microblock_size == MXFP_BLOCK_SIZE, \
            f"Unsupported microscale block size {precision_config.b_microblock_size}"
    w = b.storage.data
    if not tiled and not tiled_fp8 and b.dtype != FP4:
        w = _k_contiguous(w)  # before any view is taken: the converted copy is cached on the caller's tensor
    if w.ndim == 2 and not tiled and not tiled_fp8:
        w = w[None]
    K_W, N = b.shape[-2:]
    M = a.shape[-2] if gather_indx is None else gather_indx.shape[0]
    K = a.shape[-1]
    assert K == K_W, f"reduction dims differ: a has K={K}, b has K={K_W}"
    is_ragged = a_ragged_metadata is not None
    if is_ragged and getattr(a_ragged_metadata, "remapped_from", None) is not None:
        _combine_k = None  # only the local experts' rows arrive: tokens are incomplete
        a_ragged_metadata = _localise_remapped_metadata(a_ragged_metadata, w.shape[0], M)
    n_slices = a_ragged_metadata.n_slices if is_ragged else w.shape[0]
    if not is_ragged and w.shape[0] != 1:
        raise NotImplementedError("batched weights need ragged metadata")
    if is_ragged:
        assert w.shape[0] == n_slices, f"{w.shape[0]} weight slices for {n_slices} ragged slices"
    # ---- output --------------------------------------------------------------------------------
    reduction_n = fused_activation.specs.reduction_n
    act = nt.TK_ACT_NONE
    alpha, limit, has_limit = 0.0, 0.0, 0
    if fused_activation.specs.fn is not None or fused_activation.specs.name != "dflt":
        if fused_activation.specs.name != "swiglu" or reduction_n != 2:
            raise NotImplementedError(f"fused activation {fused_activation.specs.name!r} is not supported")
        act = nt.TK_ACT_SWIGLU
        alpha = float(fused_activation.fn_args[0])
        lim = fused_activation.fn_args[1] if len(fused_activation.fn_args) > 1 else None
        has_limit = int(lim is not None)
        limit = float(lim) if lim is not None else 0.0
    out_dtype = precision_config.out_dtype or a.dtype
    f16 = a.dtype == torch.float16 or w.dtype == torch.float16
    if f16 and not (a.dtype == w.dtype == out_dtype == torch.float16 and not (tiled or tiled_fp8 or mx_act) and b_scale is None):
        raise NotImplementedError(f"fp16 activations go with strided fp16 weights and an fp16 output (got {a.dtype} x {w.dtype} -> {out_dtype})")
    if out_dtype != torch.bfloat16 and not mx_out_fused and not f16:
        raise NotImplementedError(f"output dtype {out_dtype} is not supported (bf16, or fp16 for fp16 operands); set precision_config.out_dtype")
    y_rows = scatter_indx.shape[0] if scatter_indx is not None else M
    out_shape = (y_rows, N // reduction_n)
    c_scale = None
    fp4_out = mx_out_fused and epilogue.specs.name == FnName.QUANTIZE_MXFP4.name
    if mx_out_fused:
        c_scale = precision_config.c_mx_scale
        if isinstance(c_scale, Tensor):
            if not isinstance(c_scale.storage.layout, StridedLayout):
                raise NotImplementedError(f"output scale layout {type(c_scale.storage.layout).__name__} is not supported")
            c_scale = c_scale.storage.data
        if out_shape[1] % MXFP_BLOCK_SIZE != 0:
            raise NotImplementedError(f"MX-quantised output needs N_out % 32 == 0 (got {out_shape[1]})")
        assert c_scale.dtype == torch.uint8 and tuple(c_scale.shape[-2:]) == (y_rows, out_shape[1] // MXFP_BLOCK_SIZE) \
            and c_scale.stride(-1) == 1, f"c_mx_scale must be uint8 [{y_rows}, {out_shape[1] // MXFP_BLOCK_SIZE}]"
        if fp4_out:
            out_shape = (y_rows, out_shape[1] // 2)  # two e2m1 codes per byte
    caller_c = c is not None
    if c is None:
        c = torch.empty(out_shape, dtype=out_dtype, device=a.device)
    else:
        assert tuple(c.shape[-2:]) == out_shape and c.dtype == out_dtype and c.stride(-1) == 1
        c = c.view(out_shape) if c.ndim > 2 else c
    opt_flags = make_opt_flags(torch_dtype_to_dtype(out_dtype), torch_dtype_to_dtype(a.dtype), b.dtype, precision_config,
                               1, M, N, K, a_ragged_metadata, epilogue_reduction_n=reduction_n)
    if M * N == 0:
        return c
    if a.stride(-1) != 1:
        a = a.contiguous()
    d = nt.GemmDesc()
    d.x = a.data_ptr()
    d.x_dtype = nt.TORCH_TO_TK[a.dtype]
    d.x_stride_m = a.stride(0)
    d.x_rows = a.shape[0]
    a_ts = precision_config.a_mx_tensor_scale
    if a_ts is not None:
        a_ts = a_ts.to(torch.float32).reshape(-1).contiguous()
        assert a_ts.numel() == a.shape[0], "a_mx_tensor_scale must hold one scale per row of a"
    if flex.lhs_data.scale is not None:
        # flexpoint input scale (`acc *= x_scale * w_scale` before the bias, matmul_details/_matmul.py:540-547): a
        # one-element device tensor, folded into the per-row scale the kernel already applies (no host read)
        xs = flex.lhs_data.scale.to(torch.float32).reshape(-1)
        if xs.numel() != 1:
            raise NotImplementedError("per-batch flexpoint scales need batched activations, which are not supported")
        a_ts = a_ts * xs if a_ts is not None else xs.expand(a.shape[0]).contiguous()
    if a_ts is not None:
        d.x_row_scale = a_ts.data_ptr()
    keep = [a_ts]
    if mx_act:
        if a.dtype != torch.float8_e4m3fn:
            raise NotImplementedError(f"MX-quantised activations must be float8_e4m3fn (got {a.dtype})")
        if a_ts is not None:
            raise NotImplementedError("a_mx_tensor_scale / flexpoint scales are not supported with a_mx_scale")
        assert tuple(a_scale.shape) == (a.shape[0], (K + MXFP_BLOCK_SIZE - 1) // MXFP_BLOCK_SIZE), \
            f"a_mx_scale must be [{a.shape[0]}, {(K + 31) // 32}], got {tuple(a_scale.shape)}"
        if a_scale.stride(-1) != 1:
            a_scale = a_scale.contiguous()
        d.x_mx_scale = a_scale.data_ptr()
        d.xs_stride_m = a_scale.stride(0)
        keep.append(a_scale)
    if tiled_fp8:
        if b_scale is not None:
            raise NotImplementedError("MX scales are supported with mxfp4 (uint8) weights only")
        if a.dtype != torch.float8_e4m3fn:
            raise NotImplementedError("tiled e4m3 weights take e4m3 activations (quantise with quantize_fp8_rowwise)")
        assert w.is_contiguous() and w.dtype == torch.uint8
        d.w_dtype = nt.TK_E4M3
        d.w_layout = nt.TK_W_TILED
    elif tiled:
        assert b.dtype == FP4 and b_scale is not None, "tiled weights are MXFP4 and need precision_config.b_mx_scale"
        ws = b_scale.storage.data
        assert w.is_contiguous() and ws.is_contiguous() and ws.shape[0] == w.shape[0]
        d.w_dtype = nt.TK_E2M1
        d.w_layout = nt.TK_W_TILED
        d.w_mx_scale = ws.data_ptr()
        d.ws_stride_e = ws.stride(0)
        keep.append(ws)
    elif b.dtype == FP4:
        assert b_scale is not None, "mxfp4 weights need precision_config.b_mx_scale"
        assert w.dtype == torch.uint8
        if w.stride(-2) != 1:
            raise NotImplementedError("mxfp4 weights must be packed along K (stride(-2) == 1)")
        ws = _k_contiguous(b_scale.storage.data)
        ws = ws[None] if ws.ndim == 2 else ws
        d.w_dtype = nt.TK_E2M1
        d.w_mx_scale = ws.data_ptr()
        d.ws_stride_e, d.ws_stride_k, d.ws_stride_n = ws.stride()
        keep.append(ws)
    else:
        if b_scale is not None:
            raise NotImplementedError("MX scales are supported with mxfp4 (uint8) weights only")
        d.w_dtype = nt.TORCH_TO_TK.get(w.dtype, -1)
    d.w = w.data_ptr()
    if tiled or tiled_fp8:
        d.w_stride_e = w.stride(0)
    else:
        d.w_stride_e, d.w_stride_k, d.w_stride_n = w.stride()
    keep.append(w)
    b_ts = precision_config.b_mx_tensor_scale
    if b_ts is not None:
        b_ts = b_ts.to(torch.float32).reshape(w.shape[0], N).contiguous()
    if flex.rhs_data.scale is not None:
        # one scale for all experts or one per expert (PER_BATCH_W_SCALE), folded into the per-column scale
        ws_ = flex.rhs_data.scale.to(torch.float32).reshape(-1)
        if ws_.numel() not in (1, w.shape[0]):
            raise ValueError(f"rhs flexpoint scale must hold 1 or {w.shape[0]} values, got {ws_.numel()}")
        col = ws_.reshape(-1, 1).expand(w.shape[0], N)
        b_ts = b_ts * col if b_ts is not None else col.contiguous()
    if b_ts is not None:
        d.w_col_scale = b_ts.data_ptr()
        d.wcs_stride_e = b_ts.stride(0)
        keep.append(b_ts)
    if bias is not None:
        bias2 = bias[None] if bias.ndim == 1 else bias
        if bias2.stride(-1) != 1 or bias2.dtype not in (torch.float32, torch.bfloat16):
            bias2 = bias2.to(torch.float32).contiguous()
        d.bias = bias2.data_ptr()
        d.bias_dtype = nt.TORCH_TO_TK[bias2.dtype]
        d.bias_stride_e = bias2.stride(0)
        keep.append(bias2)
    if gather_indx is not None:
        assert gather_indx.dtype == torch.int32
        gather_indx = gather_indx.contiguous()
        d.gather_indx = gather_indx.data_ptr()
    if scatter_indx is not None:
        assert scatter_indx.dtype == torch.int32
        scatter_indx = scatter_indx.contiguous()
        d.scatter_indx = scatter_indx.data_ptr()
        d.scatter_len = scatter_indx.shape[0]
    if gammas is not None:
        g = gammas if gammas.dtype in (torch.float32, torch.bfloat16) else gammas.to(torch.float32)
        g = g.contiguous()
        d.gammas = g.data_ptr()
        d.gammas_dtype = nt.TORCH_TO_TK[g.dtype]
        keep.append(g)
    block_m = opt_flags.block_m
    if tiled_fp8:
        from .matmul_details.opt_flags import _get_opt_flags_constraints
        forced = _get_opt_flags_constraints().get("block_m")
        # the FP8 MFMA kernels' row blocks: 256 x 256 tiles from 512 rows per slice on (every row fragment of a block is
        # multiplied there, so blocks should be mostly full) when K is long enough to pay for the larger tile's set-up
        # and epilogue (measured at 16384 rows: K 14336 12 % faster, K 4096 2 % slower), 128-row tiles otherwise
        rows_per_slice = M // max(n_slices, 1) if is_ragged else M
        block_m = 256 if (forced == 256 or (forced is None and rows_per_slice >= 512 and K >= 8192)) else 128
    elif mx_act:
        from .matmul_details.opt_flags import _get_opt_flags_constraints
        forced = _get_opt_flags_constraints().get("block_m")
        block_m = 256 if (forced == 256 or (forced is None and is_ragged and M <= 144 * n_slices)) else 128
    elif tiled and mx_out_fused:
        from .matmul_details.opt_flags import _get_opt_flags_constraints
        forced = _get_opt_flags_constraints().get("block_m")
        block_m = 256 if (forced == 256 or (forced is None and is_ragged and M <= 144 * n_slices)) else 128  # the tile shapes with an MX-output epilogue
    elif tiled and extras:
        block_m = min(block_m, 32)  # the decode kernel carries the shared epilogue; the prefill kernels do not take these options
    elif tiled:
        from .matmul_details.opt_flags import _get_opt_flags_constraints
        if block_m == 128 and _get_opt_flags_constraints().get("block_m") is None and is_ragged and M <= 144 * n_slices:
            block_m = 256  # about 128 rows per expert: one tile per expert, the weights are read once
    elif block_m == 256:
        block_m = 128
    if is_ragged:
        md = a_ragged_metadata
        d.slice_sizes = md.slice_sizes.data_ptr()
        d.slice_offs = md.slice_offs.data_ptr()
        bo, bs = md.block_offs(block_m), md.block_schedule(block_m)
        assert bo.stride(0) == 1 and (bs.numel() == 0 or bs.stride(0) == 1)
        d.block_offs = bo.data_ptr()
        d.block_schedule = bs.data_ptr()
        d.n_slices = n_slices
        d.grid_m = min(RaggedTensorMetadata.n_blocks(n_slices, M, block_m), bs.shape[0])
    else:
        d.n_slices = 1
        d.grid_m = (M + block_m - 1) // block_m
    d.block_m = block_m
    d.M, d.N, d.K = M, N, K
    y_buf = c
    if tiled and block_m >= 64 and not mx_act and not mx_out_fused:
        # the prefill kernels write whole 16-byte pieces through a buffer resource: rows 16-byte aligned and padded to
        # a multiple of 8 columns; an output that is not goes through a padded buffer and is copied.  So does a
        # caller's own `c` whose last piece would spill past its columns (they may belong to a wider tensor).
        n_pad = (out_shape[1] + 7) // 8 * 8
        if c.stride(0) % 8 or c.data_ptr() % 16 or c.stride(0) < n_pad or (caller_c and out_shape[1] % 8):
            y_buf = torch.empty((out_shape[0], n_pad), dtype=c.dtype, device=c.device)[:, :out_shape[1]]
    d.y = y_buf.data_ptr()
    d.y_dtype = nt.TK_E2M1 if fp4_out else nt.TORCH_TO_TK[c.dtype]
    d.y_stride_m = y_buf.stride(0)
    d.activation = act
    d.act_alpha, d.act_limit, d.act_has_limit = alpha, limit, has_limit
    d.idle_cus = max(0, int(opt_flags.idle_sms or 0))
    if c_scale is not None:
        d.y_mx_scale = c_scale.data_ptr()
        d.ys_stride_m = c_scale.stride(-2)
    if betas is not None:
        assert betas.shape[0] == M, f"betas must hold one value per row ({M}), got {tuple(betas.shape)}"
        be = betas if betas.dtype in (torch.float32, torch.bfloat16) else betas.to(torch.float32)
        be = be.contiguous()
        d.betas = be.data_ptr()
        d.betas_dtype = nt.TORCH_TO_TK[be.dtype]
        keep.append(be)
    if out_alpha is not None:
        d.has_out_alpha = 1
        d.out_alpha = float(out_alpha)
    if c_acc_in is not None:
        acc_in = c_acc_in.view(out_shape) if c_acc_in.ndim > 2 else c_acc_in
        if tuple(acc_in.shape) != out_shape or acc_in.dtype != c.dtype or acc_in.stride(-1) != 1:
            raise NotImplementedError(f"c_acc_in must have the output's shape {out_shape} and dtype {c.dtype} with unit stride along N")
        d.acc_in = acc_in.data_ptr()
        d.acc_in_stride_m = acc_in.stride(0)
        keep.append(acc_in)
    if (tiled or tiled_fp8) and block_m >= 64 and not _STATIC_TILES and not mx_act:
        d.tile_counters = _tile_counters(a.device).data_ptr()
    combined = None
    # (not with MXFP8 activations: at the end of that kernel's launch the combine measured 22 us slower than `reduce` in a
    # launch of its own at the gpt-oss shape)
    can_combine = (_combine_k and not extras and tiled and not mx_act and act == nt.TK_ACT_NONE and scatter_indx is not None
                   and scatter_indx.shape[0] % _combine_k == 0 and a.dtype == torch.bfloat16)
    if can_combine and block_m <= 32:
        # decode kernel: the wave that completes a token's rows last sums them (arrival counters per token and fragment)
        can_combine = (scatter_indx.shape[0] // _combine_k) * ((N + 31) // 32) <= _COMBINE_COUNTER_WORDS
    elif can_combine:
        # prefill kernel: the persistent grid sums when all its workgroups have written their tiles
        can_combine = bool(d.tile_counters) and N % 8 == 0 and y_buf is c
    if can_combine:
        combined = torch.empty((scatter_indx.shape[0] // _combine_k, N), dtype=c.dtype, device=c.device)
        d.combine_k = int(_combine_k)
        d.combine_out = combined.data_ptr()
        d.combine_stride_m = combined.stride(0)
        if block_m <= 32:
            d.combine_counters = _combine_counters(a.device).data_ptr()
    with nt.on_device(a.device):
        nt.check(nt.lib().tk_moe_gemm(d, nt.stream_ptr(a.device)))
    del keep
    if y_buf is not c:
        c.copy_(y_buf)
    if combined is not None:
        c._tk_combined = combined
    return c


from .torch_twins import matmul_torch  # noqa: E402,F401  (reference twin; never called by `matmul`)
