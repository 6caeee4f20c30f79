"""The `*_torch` twins exported under the reference's names (CPU): importable where the reference has them, equal to the
CPU oracle on seeded inputs, and not wired into the operators."""
import inspect

import pytest
import torch

from oracle import moe as omoe
from oracle import mxfp as omx
from oracle import routing as ort


def test_twins_are_importable_under_the_reference_names():
    from triton_kernels.legacy import matmul_ogs_torch, routing_torch  # noqa: F401
    from triton_kernels.matmul import matmul_torch  # noqa: F401
    from triton_kernels.numerics_details.mxfp import downcast_to_mxfp_torch, upcast_from_mxfp_torch  # noqa: F401
    from triton_kernels.reduce import reduce_torch  # noqa: F401
    from triton_kernels.swiglu import swiglu_torch  # noqa: F401
    from triton_kernels.tensor_details.bitmatrix import make_bitmatrix_metadata_torch  # noqa: F401
    from triton_kernels.tensor_details.ragged_tensor import make_ragged_tensor_metadata_torch  # noqa: F401
    from triton_kernels.topk import topk_torch  # noqa: F401


def test_operators_never_call_a_twin_and_twins_never_import_the_oracle():
    import triton_amd.legacy as legacy
    import triton_amd.matmul as mm
    import triton_amd.reduce as red
    import triton_amd.swiglu as sw
    import triton_amd.topk as tk
    import triton_amd.torch_twins as twins
    from triton_amd.numerics_details import mxfp
    assert "oracle" not in inspect.getsource(twins).replace("the CPU oracle", "")
    for mod in (legacy, mm, red, sw, tk, mxfp):
        src = inspect.getsource(mod)
        body = "\n".join(l for l in src.splitlines() if not l.startswith("from .torch_twins import") and not l.startswith("from ..torch_twins import"))
        assert "_torch(" not in body.replace("wrap_torch_tensor(", ""), mod.__name__


@pytest.mark.parametrize("T, E, k", [(33, 128, 4), (7, 40, 2), (64, 9, 8)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_routing_twins_match_oracle(T, E, k, dtype):
    from triton_amd.torch_twins import make_ragged_tensor_metadata_torch, topk_torch
    g = torch.Generator().manual_seed(T * E + k)
    logits = torch.randn((T, E), generator=g).to(dtype)
    n_rows = T - 3
    sm = topk_torch(logits, k, n_rows=n_rows)
    vals, indx, bits = ort.topk(logits, k, n_rows=n_rows)
    assert torch.equal(sm.indx, indx)
    assert torch.equal(sm.vals[:n_rows], vals[:n_rows])
    assert torch.equal(sm.mask.storage.data.view(torch.int32), bits)
    meta = ort.make_bitmatrix_metadata(indx, E)
    assert torch.equal(sm.mask_metadata.col_sum, meta.col_sum)
    assert torch.equal(sm.mask_metadata.col_sorted_indx, meta.col_sorted_indx)
    assert torch.equal(sm.mask_metadata.row_sorted_indx, meta.row_sorted_indx)
    md = make_ragged_tensor_metadata_torch(meta.col_sum, T * k)
    want = ort.make_ragged_tensor_metadata(meta.col_sum, T * k)
    assert torch.equal(md.slice_offs, want.slice_offs)
    assert torch.equal(md.block_offs_data, want.block_offs_data)
    assert torch.equal(md.block_schedule_data, want.block_schedule_data)


@pytest.mark.parametrize("out_dtype", [torch.uint8, torch.float8_e4m3fn, torch.float8_e5m2])
@pytest.mark.parametrize("axis", [0, 1])
@pytest.mark.parametrize("src_dtype", [torch.bfloat16, torch.float32])
def test_mx_twins_match_oracle(out_dtype, axis, src_dtype):
    from triton_amd.numerics_details.mxfp import DequantScaleRoundingMode
    from triton_amd.torch_twins import downcast_to_mxfp_torch, upcast_from_mxfp_torch
    g = torch.Generator().manual_seed(11)
    x = (torch.randn((64, 96), generator=g) * torch.exp2(torch.randint(-20, 20, (64, 96), generator=g).float())).to(src_dtype)
    x[3, 5] = 0
    x[:, 40] = 0
    for mode, code in ((DequantScaleRoundingMode.ROUND_UP, omx.ROUND_UP), (DequantScaleRoundingMode.ROUND_DOWN, omx.ROUND_DOWN)):
        q, s = downcast_to_mxfp_torch(x, out_dtype, axis, DEQUANT_SCALE_ROUNDING_MODE=mode)
        qo, so = omx.downcast_to_mxfp(x, out_dtype, axis, rounding=code)
        assert torch.equal(s, so)
        assert torch.equal(q.contiguous().view(torch.uint8), qo.contiguous().view(torch.uint8))
        for target in (torch.bfloat16, torch.float32):
            up = upcast_from_mxfp_torch(qo, so, target, axis)
            assert torch.equal(up, omx.upcast_from_mxfp(qo, so, target, axis))


def test_matmul_swiglu_reduce_twins_match_oracle():
    from triton_amd.matmul import PrecisionConfig
    from triton_amd.swiglu import PrecisionConfig as SwigluConfig
    from triton_amd.torch_twins import matmul_torch, reduce_torch, swiglu_torch
    g = torch.Generator().manual_seed(2)
    T, K, N, E, k = 24, 64, 48, 5, 2
    x = torch.randn((T, K), generator=g).to(torch.bfloat16)
    w = (torch.randn((E, K, N), generator=g) * 0.1).to(torch.bfloat16)
    bias = torch.randn((E, N), generator=g)
    r = ort.routing(torch.randn((T, E), generator=g), k)
    from triton_amd.torch_twins import make_ragged_tensor_metadata_torch
    md = make_ragged_tensor_metadata_torch(r.meta.col_sum, T * k)
    got = matmul_torch(x, w, bias, md, gather_indx=r.gather_indx, scatter_indx=r.scatter_indx, precision_config=PrecisionConfig(),
                       gammas=r.gammas)
    want = omoe.matmul(x, w, bias, r.meta.col_sum, gather_indx=r.gather_indx, scatter_indx=r.scatter_indx, gammas=r.gammas)
    assert torch.equal(got, want)
    q, s = omx.downcast_to_mxfp(w, torch.uint8, axis=1)
    got4 = matmul_torch(x, q, bias, md, gather_indx=r.gather_indx, precision_config=PrecisionConfig(b_mx_scale=s))
    want4 = omoe.matmul(x, q, bias, r.meta.col_sum, gather_indx=r.gather_indx, w_mx_scale=s)
    assert torch.equal(got4, want4)
    a = torch.randn((T, 2 * N), generator=g)
    assert torch.allclose(swiglu_torch(a, 1.702, SwigluConfig(limit=7.0)), omoe.swiglu(a, 1.702, 7.0), rtol=1e-6, atol=1e-6)
    y = torch.randn((T, k, N), generator=g).to(torch.bfloat16)
    assert torch.equal(reduce_torch(y, dim=1)[0], omoe.reduce_k(y.reshape(T * k, N), k))
    # ragged K
    sizes = torch.tensor([10, 0, 30, 24], dtype=torch.int32)
    from triton_amd.tensor import RaggedTensorMetadata
    offs = torch.tensor([0, 10, 10, 40, 64], dtype=torch.int32)
    mdk = make_ragged_tensor_metadata_torch(sizes, 64)
    mdk = RaggedTensorMetadata(sizes, offs, mdk.block_offs_data, mdk.block_schedule_data)
    a2 = torch.randn((9, 64), generator=g).to(torch.bfloat16)
    b2 = torch.randn((64, 7), generator=g).to(torch.bfloat16)
    got_k = matmul_torch(a2, b2, None, mdk, mdk)
    assert torch.equal(got_k, omoe.matmul_ragged_k(a2, b2, sizes, offs[:4], offs[:4], out_dtype=torch.float32))
