"""Per-row dynamic quantisation of activations to OCP e4m3.

The reference has no function of its own for this (its benchmark casts activations with `.to(float8)`,
bench/bench_mlp.py:169); the Mixtral-shaped FP8 configuration needs it, so it lives here.  The scales feed
`PrecisionConfig.a_mx_tensor_scale` (one fp32 per row of `a`).
"""
from __future__ import annotations

import torch

from .. import _native as nt


def quantize_fp8_rowwise(x: torch.Tensor):
    """`x [M, K]` bf16 -> `(q [M, K] float8_e4m3fn, scale [M] fp32)` with `scale = amax/448` (1 for a zero
    row) and `q = saturating_cast(x / scale)`."""
    nt.require_gpu(x, "x")
    assert x.ndim == 2 and x.dtype == torch.bfloat16
    if x.stride(1) != 1:
        x = x.contiguous()
    M, K = x.shape
    q = torch.empty((M, K), dtype=torch.float8_e4m3fn, device=x.device)
    s = torch.empty((M, ), dtype=torch.float32, device=x.device)
    with nt.on_device(x.device):
        nt.check(
            nt.lib().tk_quant_fp8_rows(x.data_ptr(), nt.TK_BF16, M, K, x.stride(0) if M else 0, q.data_ptr(), q.stride(0) if M else 0,
                                       s.data_ptr(), nt.stream_ptr(x.device)))
    return q, s
