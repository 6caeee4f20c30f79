"""swiglu activation (mirrors `triton_kernels/swiglu.py:10-100`).

`swiglu_fn` is the token a `FusedActivation(FnSpecs("swiglu", swiglu_fn, ("alpha", "limit"), reduction_n=2),
(alpha, limit))` carries; `matmul` recognises it and runs the activation in the GEMM epilogue."""
from __future__ import annotations

from dataclasses import dataclass

import torch

from . import _native as nt
from .numerics import InFlexData, OutFlexData


@dataclass(frozen=True)
class FlexCtx:
    out_data: OutFlexData = OutFlexData()
    inp_data: InFlexData = InFlexData()
    saturate_inf: bool = False


@dataclass(frozen=True)
class PrecisionConfig:
    limit: float | None
    flex_ctx: FlexCtx = FlexCtx()


class _SwigluFn:
    """Marker for the fused activation: out = s * (linear + 1), s = gate * sigmoid(alpha * gate)."""
    name = "swiglu"

    def __repr__(self):
        return "_swiglu"


swiglu_fn = _SwigluFn()


def swiglu(a, alpha, precision_config, routing_data=None):
    """`a [..., 2n]` with interleaved (gate, linear) columns -> `[..., n]`, same dtype."""
    nt.require_gpu(a, "a")
    flex = precision_config.flex_ctx
    if flex.out_data.expected_scale is not None or flex.inp_data.scale is not None or flex.out_data.actual_scale is not None:
        raise NotImplementedError("flexpoint scales are not supported by swiglu")
    N = a.shape[-1]
    assert a.stride()[-1] == 1
    assert N % 2 == 0
    M = a.numel() // N if N else 0
    a2 = a.reshape(M, N)
    out = torch.empty((M, N // 2), dtype=a.dtype, device=a.device)
    n_tokens = None
    if routing_data is not None:
        # rows actually routed = the last entry of the experts' row offsets (the reference reads
        # `expt_data.token_offs[n_expts_tot]`, swiglu.py:53-55; here the same array is called `slice_offs`)
        offs = routing_data.expt_data.slice_offs
        n_tokens = offs[routing_data.n_expts_tot:routing_data.n_expts_tot + 1]
        assert n_tokens.dtype == torch.int32 and n_tokens.numel() == 1
    limit = precision_config.limit
    with nt.on_device(a.device):
        nt.check(
            nt.lib().tk_swiglu(a2.data_ptr(), nt.TORCH_TO_TK[a.dtype], M, N // 2, a2.stride(0) if M else 0, out.data_ptr(),
                               out.stride(0), float(alpha), float(limit) if limit is not None else 0.0,
                               int(limit is not None), nt.ptr(n_tokens), nt.stream_ptr(a.device)))
    return out.view(a.shape[:-1] + out.shape[-1:])


from .torch_twins import swiglu_torch  # noqa: E402,F401  (reference twin; never called by `swiglu`)
