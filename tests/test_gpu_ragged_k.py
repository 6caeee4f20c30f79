"""GPU parity of the ragged-K GEMM (the expert weight gradient, `matmul(..., b_ragged_metadata=...)`) through the C ABI
against the CPU oracle.

Mirrors the `inner_expt_opt` cases of python/triton_kernels/tests/test_matmul.py:311-320,469-500: the reduction
dimension is split into slices (10, one of them empty), either operand's slices may be padded ("pad_a" / "pad_b", so
the two operands carry different slice offsets), no bias.  Operands are bf16 or fp16; a is taken both k-slow (x^T of a
row-major x: the weight-gradient layout) and k-contiguous, b both row-major and transposed.  Tolerance: the rtol 2e-2 /
atol 1e-2 gate for 16-bit outputs (accumulation order differs from torch's), tighter for fp32 outputs."""
import pytest
import torch

from oracle import moe as omoe
from oracle.checks import assert_allclose_gate

pytestmark = pytest.mark.gpu


def _slices(k_total, n_slices, g):
    cuts = torch.sort(torch.randint(0, k_total + 1, (n_slices - 1, ), generator=g)).values
    sizes = torch.diff(torch.cat([torch.tensor([0]), cuts, torch.tensor([k_total])]))
    if n_slices > 2:
        sizes[n_slices // 2 + 1] += sizes[n_slices // 2]  # one empty slice
        sizes[n_slices // 2] = 0
    return sizes.to(torch.int32)


def _metadata(sizes, offs, device):
    from triton_amd.tensor import RaggedTensorMetadata, make_ragged_tensor_metadata
    md = make_ragged_tensor_metadata(sizes.to(device), int(offs[-1]))
    return RaggedTensorMetadata(md.slice_sizes, offs.to(torch.int32).to(device), md.block_offs_data, md.block_schedule_data)


def _offsets(sizes, pad):
    """Start of every slice (+ the end): dense, or each slice padded to a multiple of `pad`."""
    offs = [0]
    for s in sizes.tolist():
        step = s if pad is None else (s + pad - 1) // pad * pad
        offs.append(offs[-1] + step)
    return torch.tensor(offs, dtype=torch.int32)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("m, n, k", [(300, 400, 416), (128, 256, 1024), (720, 576, 768), (17, 40, 100), (256, 8, 64)])
@pytest.mark.parametrize("pad", [None, "pad_a", "pad_b"])
@pytest.mark.parametrize("a_k_slow, b_transposed", [(True, False), (False, False), (True, True), (False, True)])
def test_ragged_k_matmul(device, dtype, m, n, k, pad, a_k_slow, b_transposed):
    import triton_amd.matmul as mm
    g = torch.Generator().manual_seed(m * 31 + n * 7 + k)
    sizes = _slices(k, 10, g)
    a_offs = _offsets(sizes, 16 if pad == "pad_a" else None)
    b_offs = _offsets(sizes, 16 if pad == "pad_b" else None)
    ka, kb = int(a_offs[-1]), int(b_offs[-1])
    # the padding holds garbage that must not reach the output (NaN would poison a sum that read it)
    a = torch.randn((m, ka), generator=g).to(dtype)
    b = torch.randn((kb, n), generator=g).to(dtype)
    for e, s in enumerate(sizes.tolist()):
        a[:, int(a_offs[e]) + s:int(a_offs[e + 1])] = float("nan")
        b[int(b_offs[e]) + s:int(b_offs[e + 1]), :] = float("nan")
    ref = omoe.matmul_ragged_k(a, b, sizes, a_offs, b_offs)
    a_dev = a.to(device)
    if a_k_slow:  # x^T of a row-major [k, m] tensor
        a_dev = a.t().contiguous().to(device).t()
        assert a_dev.stride(0) == 1
    b_dev = b.to(device)
    if b_transposed:
        b_dev = b.t().contiguous().to(device).t()
    out = mm.matmul(a_dev, b_dev, None, a_ragged_metadata=_metadata(sizes, a_offs, device),
                    b_ragged_metadata=_metadata(sizes, b_offs, device))
    assert out.shape == (10, m, n) and out.dtype == dtype
    assert not torch.isnan(out).any()
    assert_allclose_gate(ref, out, what="ragged-K matmul")
    assert out[5].abs().max() == 0  # the empty slice


def test_ragged_k_fp32_output_and_weight_gradient_identity(device):
    """dW[e] = x_e^T @ dy_e at a MoE-like shape with fp32 output, and the identity sum_e dW[e] = x^T @ dy."""
    import triton_amd.matmul as mm
    g = torch.Generator().manual_seed(3)
    rows, hidden, n, E = 1024, 360, 200, 8
    sizes = _slices(rows, E, g)
    offs = _offsets(sizes, None)
    x = torch.randn((rows, hidden), generator=g).to(torch.bfloat16)
    dy = torch.randn((rows, n), generator=g).to(torch.bfloat16)
    md = _metadata(sizes, offs, device)
    pc = mm.PrecisionConfig(out_dtype=torch.float32)
    out = mm.matmul(x.to(device).t(), dy.to(device), None, a_ragged_metadata=md, b_ragged_metadata=md, precision_config=pc)
    ref = omoe.matmul_ragged_k(x.t(), dy, sizes, offs, offs, out_dtype=torch.float32)
    torch.testing.assert_close(out.cpu(), ref, rtol=1e-4, atol=1e-3)
    torch.testing.assert_close(out.cpu().sum(0).double(), x.double().t() @ dy.double(), rtol=1e-4, atol=2e-3)


def test_ragged_k_rejections(device):
    import triton_amd.matmul as mm
    sizes = torch.tensor([4, 4], dtype=torch.int32)
    md = _metadata(sizes, _offsets(sizes, None), device)
    a = torch.zeros((8, 8), dtype=torch.bfloat16, device=device)
    with pytest.raises(NotImplementedError):
        mm.matmul(a, a, torch.zeros((2, 8), device=device), a_ragged_metadata=md, b_ragged_metadata=md)
    with pytest.raises(NotImplementedError):
        mm.matmul(a.float(), a.float(), None, a_ragged_metadata=md, b_ragged_metadata=md)
    with pytest.raises(ValueError):
        mm.matmul(a, a, None, b_ragged_metadata=md)
