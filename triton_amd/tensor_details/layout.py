"""Layouts accepted for matmul operands (mirrors `triton_kernels/tensor_details/layout.py`).

Two families exist on gfx950 in this build: the strided layout (what `downcast_to_mxfp` returns) and the
pre-tiled MXFP4 pair `GFX950MXValueLayout` / `GFX950MXScaleLayout`, which the default-layout helpers return
for weights whose MX axis is K, as the reference's helpers return its architecture-specific layouts
(layout.py:26-54).  Both are accepted by `matmul`; the tiled pair is the fast path.  `CDNA4MXScaleLayout`, the
reference's own scale pre-shuffle for this GPU, is accepted too: `matmul` converts such scales once to the order
that goes with the weight values' layout.
"""
from .layout_details.base import Layout
from .layout_details.cdna4_scale import CDNA4MXScaleLayout
from .layout_details.gfx950_mx import GFX950FP8ValueLayout, GFX950MXScaleLayout, GFX950MXValueLayout
from .layout_details.strided import StridedLayout

__all__ = ["Layout", "StridedLayout", "GFX950MXValueLayout", "GFX950MXScaleLayout", "GFX950FP8ValueLayout", "CDNA4MXScaleLayout"]


def make_default_matmul_fp8_w_layout():
    """Layout `matmul` prefers for e4m3 expert weights `[E, K, N]` on this GPU (no counterpart in the reference, which
    takes plain strided fp8 weights; those stay accepted)."""
    return GFX950FP8ValueLayout()


def make_default_matmul_mxfp4_w_layout(mx_axis: int, **_unused):
    return GFX950MXValueLayout() if mx_axis in (1, -2) else StridedLayout(-2)


def make_default_matmul_mxfp4_w_scale_layout(mx_axis: int, num_warps: int = 8):
    return GFX950MXScaleLayout() if mx_axis in (1, -2) else StridedLayout(-2)


def make_default_matmul_mx_act_scale_layout(ragged_metadata=None):
    return StridedLayout(-2)
