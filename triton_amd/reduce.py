"""Reduction over one dimension (mirrors the forward of `triton_kernels/reduce.py:1143-1165`).

The mixture-of-experts forward uses it as the k-way combine: `reduce(y.view(T, k, d), dim=1)`.
Supported: 3-D input, `dim == 1`, optional `mask` / `scale` (broadcastable), with the backward pass of that subset
(through autograd when `x` requires a gradient).  MX inputs / outputs, flexpoint scales and post-process functions of
the reference are not part of this build.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from . import _native as nt
from .numerics import InFlexData, OutFlexData
from .specialize import FnSpecs


@dataclass(frozen=True)
class PostprocessFn:
    specs: FnSpecs = FnSpecs.default()
    fn_args: tuple = tuple()


def _bcast_strides(t, shape):
    t = t.expand(shape) if t.ndim == len(shape) else t.reshape((1, ) * (len(shape) - t.ndim) + tuple(t.shape)).expand(shape)
    return t, t.stride()


def _mask_scale_args(mask, scale, shape):
    keep = []
    m_ptr, ms = None, (0, 0, 0)
    if mask is not None:
        mask_u8 = mask if mask.dtype in (torch.uint8, torch.bool, torch.int8) else (mask != 0)
        mask_u8, ms = _bcast_strides(mask_u8, shape)
        m_ptr = mask_u8.data_ptr()
        keep.append(mask_u8)
    s_ptr, ss = None, (0, 0, 0)
    if scale is not None:
        scale_f = scale if scale.dtype == torch.float32 else scale.to(torch.float32)
        scale_f, ss = _bcast_strides(scale_f, shape)
        s_ptr = scale_f.data_ptr()
        keep.append(scale_f)
    return m_ptr, ms, s_ptr, ss, keep


def reduce_backward(dy: torch.Tensor, x_shape, dim: int, mask=None, scale=None, dtype=None):
    """dx of `reduce(x, dim=1, mask, scale)` for the gradient `dy [A, C]` (reduce.py:859-1049 for this subset)."""
    A, K, C = x_shape
    assert dim % 3 == 1 and tuple(dy.shape) == (A, C)
    nt.require_gpu(dy, "dy")
    dy = dy.to(dtype) if dtype is not None and dy.dtype != dtype else dy
    if dy.stride(1) != 1:
        dy = dy.contiguous()
    dx = torch.empty((A, K, C), dtype=dy.dtype, device=dy.device)
    m_ptr, ms, s_ptr, ss, keep = _mask_scale_args(mask, scale, (A, K, C))
    with nt.on_device(dy.device):
        nt.check(
            nt.lib().tk_reduce_mid_backward(dy.data_ptr(), nt.TORCH_TO_TK[dy.dtype], A, K, C, dy.stride(0) if A else 0, m_ptr, *ms, s_ptr,
                                            *ss, dx.data_ptr(), nt.stream_ptr(dy.device)))
    del keep
    return dx


class _ReduceAutograd(torch.autograd.Function):

    @staticmethod
    def forward(ctx, x, mask, scale, y):
        out, _ = _reduce_forward(x.detach(), mask, scale, y)
        ctx.x_shape, ctx.x_dtype, ctx.mask, ctx.scale = tuple(x.shape), x.dtype, mask, scale
        return out

    @staticmethod
    def backward(ctx, grad_y):
        return reduce_backward(grad_y, ctx.x_shape, 1, ctx.mask, ctx.scale, ctx.x_dtype), None, None, None


def reduce(x: torch.Tensor, dim: int, mask: Optional[torch.Tensor] = None, scale: Optional[torch.Tensor] = None,
           x_mxscale: Optional[torch.Tensor] = None, x_flex: Optional[InFlexData] = InFlexData(),
           x_global_scale: Optional[torch.Tensor] = None, y: Optional[torch.Tensor] = None,
           y_dtype: Optional[torch.dtype] = None, y_flex: Optional[OutFlexData] = OutFlexData(),
           y_flex_saturate_inf: bool = False, y_has_mx: Optional[bool] = None,
           y_mx_scale_dtype: Optional[torch.dtype] = None, y_microblock_size: int = 32, y_value_pack_factor: int = 1,
           postprocess_fn1: Optional[PostprocessFn] = None, postprocess_fn2: Optional[PostprocessFn] = None,
           unpadded_batch_size: Optional[torch.Tensor] = None):
    """Returns `(y, y_mxscale)` with `y = sum over dim of where(mask, x * scale, 0)` in fp32, cast to x's dtype."""
    if x_mxscale is not None or y_has_mx or x_global_scale is not None:
        raise NotImplementedError("MX inputs / outputs are not supported by reduce")
    if (x_flex is not None and x_flex.scale is not None) or (y_flex is not None and
                                                              (y_flex.expected_scale is not None or y_flex.actual_scale is not None)):
        raise NotImplementedError("flexpoint scales are not supported by reduce")
    for fn in (postprocess_fn1, postprocess_fn2):
        if fn is not None and fn.specs.fn is not None:
            raise NotImplementedError("post-process functions are not supported by reduce")
    if unpadded_batch_size is not None:
        raise NotImplementedError("unpadded_batch_size is not supported by reduce")
    if x.ndim != 3:
        raise NotImplementedError("reduce supports 3-D inputs")
    dim = dim % 3
    if dim != 1:
        raise NotImplementedError("reduce supports dim == 1 (the k-way combine)")
    if y_dtype is not None and y_dtype != x.dtype:
        raise NotImplementedError("reduce keeps the input dtype")
    if x.requires_grad and torch.is_grad_enabled():
        return _ReduceAutograd.apply(x, mask, scale, y), None
    return _reduce_forward(x, mask, scale, y)


def _reduce_forward(x, mask, scale, y):
    nt.require_gpu(x, "x")
    if x.stride(2) != 1:
        x = x.contiguous()
    A, K, C = x.shape
    if y is None:
        y = torch.empty((A, C), dtype=x.dtype, device=x.device)
    else:
        assert y.shape == (A, C) and y.dtype == x.dtype and y.stride(1) == 1
    m_ptr, ms, s_ptr, ss, keep = _mask_scale_args(mask, scale, x.shape)
    with nt.on_device(x.device):
        nt.check(
            nt.lib().tk_reduce_mid(x.data_ptr(), nt.TORCH_TO_TK[x.dtype], A, K, C, x.stride(0), x.stride(1), m_ptr, *ms, s_ptr,
                                   *ss, y.data_ptr(), y.stride(0) if A else 0, nt.stream_ptr(x.device)))
    return y, None


from .torch_twins import reduce_torch  # noqa: E402,F401  (reference twin; never called by `reduce`)
