"""GPU parity of `reduce` (dim = 1, the k-way combine) and its backward through the C ABI.

Mirrors the subset of python/triton_kernels/tests/test_reduce.py:38-131 that this build supports: float16 / float32 /
bfloat16, the five mask modes, an optional broadcast scale, forward and backward, tolerances atol = rtol = 1e-3 as there
(1e-2 for bf16).  The reference value is the closed form `sum_j where(mask, x * scale, 0)` (reduce.py:1181-1214)
evaluated by torch on the CPU in fp32, and its gradient by torch autograd."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _mask(mode, B, M, N, g):
    if mode == "none":
        return None
    shape = {"full": (B, M, N), "broadcast_b": (1, M, N), "broadcast_m": (B, 1, N), "broadcast_n": (B, M, 1)}[mode]
    return (torch.rand(shape, generator=g) > 0.3).to(torch.int8).expand(B, M, N)


@pytest.mark.parametrize("B, M, N", [(311, 4, 384), (64, 311, 40), (4, 4, 4), (3, 15, 25), (4096, 4, 2880), (5, 2, 0), (0, 2, 5)])
@pytest.mark.parametrize("dt", [torch.float16, torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mask_mode", ["none", "full", "broadcast_b", "broadcast_m", "broadcast_n"])
@pytest.mark.parametrize("with_scale", [False, True])
def test_reduce_forward_backward(device, B, M, N, dt, mask_mode, with_scale):
    from triton_amd.reduce import reduce
    if B * M * N > 10**7 and (mask_mode not in ("none", "full") or dt == torch.float16):
        pytest.skip("large shape: one mask mode per dtype is enough")
    g = torch.Generator().manual_seed(B + M + N)
    x = torch.randn((B, M, N), generator=g).to(dt)
    mask = _mask(mask_mode, B, M, N, g)
    scale = torch.rand((B, M, 1), generator=g).expand(B, M, N) if with_scale else None
    x_ref = x.float().clone().requires_grad_()
    v = x_ref * scale if scale is not None else x_ref
    if mask is not None:
        v = torch.where(mask != 0, v, torch.zeros_like(v))
    y_ref = v.sum(dim=1)
    dv = lambda t: None if t is None else t.to(device)
    x_dev = x.to(device).requires_grad_()
    y, y_mx = reduce(x_dev, dim=1, mask=dv(mask), scale=dv(scale))
    assert y_mx is None and y.shape == (B, N) and y.dtype == dt
    tol = 1e-2 if dt == torch.bfloat16 else 1e-3
    assert torch.allclose(y.detach().cpu().float(), y_ref.detach().to(dt).float(), atol=tol * max(1, M**0.5), rtol=tol)
    dy = torch.randn((B, N), generator=g).to(dt)
    y.backward(dy.to(device))
    y_ref.backward(dy.float())
    assert x_dev.grad.shape == x.shape and x_dev.grad.dtype == dt
    assert torch.allclose(x_dev.grad.cpu().float(), x_ref.grad.to(dt).float(), atol=tol, rtol=tol)
