"""MX quantise / dequantise (mirrors `triton_kernels/numerics_details/mxfp.py:19-176`).

Both functions call the HIP kernels behind `tk_mx_downcast` / `tk_mx_upcast`; the source (or the
destination) is addressed through its strides, so no transposed temporary is made when the quantised
axis is not the innermost one.
"""
from __future__ import annotations

from enum import Enum

import torch

from .. import _native as nt
from ..tensor import Tensor, empty, wrap_torch_tensor
from ..tensor_details.dtype import FP4, FP8_E4M3FN, FP8_E5M2, UINT8
from ..tensor_details.layout import StridedLayout


class _BlockSize(int):

    @property
    def value(self):
        return int(self)


MXFP_BLOCK_SIZE = _BlockSize(32)
NVFP_BLOCK_SIZE = _BlockSize(16)


class _EpilogueFn:
    """Token carried by `Epilogue(FnSpecs(FnName.QUANTIZE_MXFP8.name, quantize_mxfp8_fn, (), ()), ...)`; the
    reference passes a device function here (`triton_kernels/numerics_details/mxfp.py:432-434`), `matmul` in this
    build recognises the epilogue by its name and runs the MX quantiser kernel."""

    def __init__(self, name):
        self.name = name

    def __repr__(self):
        return self.name


quantize_mxfp8_fn = _EpilogueFn("_quantize_mxfp8_fn")
quantize_mxfp4_fn = _EpilogueFn("_quantize_mxfp4_fn")
quantize_nvfp4_fn = _EpilogueFn("_quantize_nvfp4_fn")


class DequantScaleRoundingMode(Enum):
    ROUND_UP = 0  # 2^ceil(log2(max / max_q)): never clips the block maximum
    ROUND_DOWN = 1  # 2^floor(log2(max / max_pow2_q)): the OCP rule


def get_max_quant_val(dtype: torch.dtype):
    return {torch.uint8: 6.0, torch.float8_e5m2: 57344.0, torch.float8_e4m3fn: 448.0}[dtype]


_KIND = {FP4: nt.TK_E2M1, FP8_E4M3FN: nt.TK_E4M3, FP8_E5M2: nt.TK_E5M2}
_FLOAT_SRC = {torch.float32: nt.TK_F32, torch.bfloat16: nt.TK_BF16, torch.float16: nt.TK_F16}


def _prod(xs):
    r = 1
    for x in xs:
        r *= int(x)
    return r


def _collapse(t: torch.Tensor, axis: int):
    """Views `t` as [outer, axis, inner] and returns (outer, L, inner, s_outer, s_axis, s_inner), or None
    when the dims before / after `axis` do not each collapse to one stride."""
    shape, strides = list(t.shape), list(t.stride())

    def fold(dims):
        dims = [(shape[d], strides[d]) for d in dims if shape[d] != 1]
        if not dims:
            return 1, 0
        n, st = dims[-1]
        for size, stride in reversed(dims[:-1]):
            if stride != st * n:
                return None
            n *= size
        return n, st

    o = fold(range(0, axis))
    i = fold(range(axis + 1, len(shape)))
    if o is None or i is None:
        return None
    return o[0], shape[axis], i[0], o[1], strides[axis], i[1]


def downcast_to_mxfp(x, out_dtype, axis: int, scale_dtype: torch.dtype = torch.uint8,
                     microblock_size: int = MXFP_BLOCK_SIZE.value,
                     DEQUANT_SCALE_ROUNDING_MODE: DequantScaleRoundingMode = DequantScaleRoundingMode.ROUND_UP):
    """Quantises `x` along `axis` in blocks of 32.  Returns `(values, scales)` torch tensors whose
    unit-stride dimension is `axis`; `torch.uint8` output means e2m1 packed two per byte."""
    if not isinstance(x, Tensor):
        x = wrap_torch_tensor(x)
    if scale_dtype != torch.uint8:
        if scale_dtype == torch.float8_e4m3fn:
            raise NotImplementedError("direct float8 (NVFP4) block scales are not supported on gfx950")
        raise AssertionError(f"Invalid scale dtype {scale_dtype=}")
    if microblock_size != MXFP_BLOCK_SIZE.value:
        raise NotImplementedError(f"microblock_size {microblock_size} is not supported (OCP MX uses 32)")
    if isinstance(out_dtype, torch.dtype):
        out_dtype = {torch.uint8: FP4, torch.float8_e4m3fn: FP8_E4M3FN, torch.float8_e5m2: FP8_E5M2}[out_dtype]
    assert out_dtype in (FP4, FP8_E4M3FN, FP8_E5M2), f"Invalid output dtype {out_dtype=}"
    assert -x.ndim <= axis < x.ndim, f"Invalid axis {axis=}"
    assert isinstance(x.storage.layout, StridedLayout), "input data must be strided"
    axis = axis % x.ndim
    L = x.shape[axis]
    assert L % microblock_size == 0, f"axis dim must be divisible by {microblock_size}. Got {L}"
    src = x.storage.data
    if src.dtype not in _FLOAT_SRC:
        raise AssertionError(f"Invalid input tensor dtype {src.dtype}")
    layout = StridedLayout(major_dim=axis - x.ndim)
    scale_shape = (*x.shape[:axis], L // microblock_size, *x.shape[axis + 1:])
    y_value = empty(x.shape, out_dtype, x.device, layout)
    y_scale = empty(scale_shape, UINT8, x.device, layout)
    if src.numel() > 0:
        nt.require_gpu(src, "x")
        view = _collapse(src, axis)
        if view is not None and not (view[5] == 1 or view[2] == 1 and view[4] == 1):
            view = None
        if view is None:
            src = src.contiguous()
            view = _collapse(src, axis)
        outer, L_, inner, so, sa, si = view
        inner_last = src.shape[-1] if axis < src.ndim - 1 else 1
        with nt.on_device(src.device):
            nt.check(
                nt.lib().tk_mx_downcast(src.data_ptr(), _FLOAT_SRC[src.dtype], outer, L_, inner, inner_last, so, sa, si,
                                        y_value.storage.data.data_ptr(), y_scale.storage.data.data_ptr(),
                                        _KIND[out_dtype], DEQUANT_SCALE_ROUNDING_MODE.value, nt.stream_ptr(src.device)))
    return y_value.storage.data, y_scale.storage.data


def upcast_from_mxfp(tensor: torch.Tensor, scale: torch.Tensor, target_dtype: torch.dtype, axis: int,
                     tensor_scale: torch.Tensor | None = None):
    """Dequantises along `axis`; the result is a standard-contiguous tensor of `target_dtype`."""
    ndim = tensor.ndim
    assert -ndim <= axis < ndim, f"Invalid axis {axis=}"
    axis = axis % ndim
    assert tensor.ndim == scale.ndim, (f"Weight and scale must have the same number of dimensions. "
                                       f"Got {tensor.ndim=} and {scale.ndim=}")
    if tensor_scale is not None and tensor_scale.numel() != 1:
        expected = tensor.shape[:axis] + tensor.shape[axis + 1:]
        assert tensor_scale.shape == expected, f"Invalid tensor scale shape: expected {expected}, got {tensor_scale.shape}"
    assert tensor.dtype in {torch.uint8, torch.float8_e5m2, torch.float8_e4m3fn}, f"Invalid tensor dtype {tensor.dtype=}"
    if scale.dtype == torch.float8_e4m3fn:
        raise NotImplementedError("direct float8 (NVFP4) block scales are not supported on gfx950")
    assert scale.dtype == torch.uint8, f"Invalid scale dtype {scale.dtype=}"
    assert target_dtype in (torch.float16, torch.bfloat16, torch.float32), f"Invalid output dtype {target_dtype=}"
    pack = 2 if tensor.dtype == torch.uint8 else 1
    L = tensor.shape[axis] * pack
    out_shape = tensor.shape[:axis] + (L, ) + tensor.shape[axis + 1:]
    out = torch.empty(out_shape, dtype=target_dtype, device=tensor.device)
    if out.numel() > 0:
        nt.require_gpu(tensor, "tensor")
        assert L % MXFP_BLOCK_SIZE == 0 and scale.shape[axis] * MXFP_BLOCK_SIZE == L, \
            "quantised axis must be a multiple of 32 with one scale per block"
        # kernels read values/scales dense with the quantised axis innermost
        v = tensor.transpose(axis, ndim - 1).contiguous()
        s = scale.transpose(axis, ndim - 1).contiguous()
        outer = _prod(out_shape[:axis])
        inner = _prod(out_shape[axis + 1:])
        inner_last = out_shape[-1] if axis < ndim - 1 else 1
        kind = {torch.uint8: nt.TK_E2M1, torch.float8_e4m3fn: nt.TK_E4M3, torch.float8_e5m2: nt.TK_E5M2}[tensor.dtype]
        with nt.on_device(tensor.device):
            nt.check(
                nt.lib().tk_mx_upcast(v.data_ptr(), s.data_ptr(), kind, outer, L, inner, inner_last, out.data_ptr(),
                                      nt.TORCH_TO_TK[target_dtype], L * inner, inner, 1, nt.stream_ptr(tensor.device)))
    if tensor_scale is not None:
        shp = (1, ) * out.ndim if tensor_scale.numel() == 1 else (*tensor_scale.shape[:axis], 1, *tensor_scale.shape[axis:])
        out = out * tensor_scale.to(device=out.device).reshape(shp)
    return out


from ..torch_twins import downcast_to_mxfp_torch, upcast_from_mxfp_torch  # noqa: E402,F401  (reference twins)
