"""Layouts accepted for matmul operands (mirrors `triton_kernels/tensor_details/layout.py`).

Only the strided layout exists on gfx950 in this build; the default-layout helpers therefore return
`StridedLayout(-2)` (K-major weights / scales), which is what the reference returns when no
architecture-specific swizzle applies (layout.py:40,54).
"""
from .layout_details.base import Layout
from .layout_details.strided import StridedLayout

__all__ = ["Layout", "StridedLayout"]


def make_default_matmul_mxfp4_w_layout(mx_axis: int, **_unused):
    return StridedLayout(-2)


def make_default_matmul_mxfp4_w_scale_layout(mx_axis: int, num_warps: int = 8):
    return StridedLayout(-2)


def make_default_matmul_mx_act_scale_layout(ragged_metadata=None):
    return StridedLayout(-2)
