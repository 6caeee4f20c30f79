"""Round trips of the pre-tiled MXFP4 layouts (CPU) and element placement against the documented formula."""
import pytest
import torch

from triton_kernels.tensor import FP4, UINT8, convert_layout, wrap_torch_tensor
from triton_kernels.tensor_details.layout import (GFX950FP8ValueLayout, GFX950MXScaleLayout, GFX950MXValueLayout, StridedLayout,
                                                  make_default_matmul_mxfp4_w_layout, make_default_matmul_mxfp4_w_scale_layout)


@pytest.mark.parametrize("E, K, N", [(1, 128, 32), (3, 96, 40), (2, 2880, 96), (2, 320, 33 * 2)])
def test_value_layout_round_trip_and_placement(E, K, N):
    g = torch.Generator().manual_seed(K + N)
    packed = torch.randint(0, 256, (E, N, K // 2), generator=g, dtype=torch.uint8).transpose(1, 2)  # [E, K/2, N], K-contiguous
    t = wrap_torch_tensor(packed, dtype=FP4)
    assert t.shape == [E, K, N]
    tiled = convert_layout(t, GFX950MXValueLayout())
    nfr, nst = (N + 31) // 32, (K + 127) // 128
    assert list(tiled.storage.data.shape) == [E, nfr * nst * 2048] == GFX950MXValueLayout().storage_shape([E, K, N], True)
    back = convert_layout(tiled, StridedLayout(-2))
    assert torch.equal(back.storage.data, packed)
    raw = tiled.storage.data
    for (e, k, n) in [(0, 0, 0), (E - 1, K - 2, N - 1), (0, 70, 5), (E - 1, (K // 2) & ~1, N // 2)]:
        F, c, s, kk = n // 32, n % 32, k // 128, k % 128
        h, q, b = kk // 64, (kk % 64) // 32, (kk % 32) // 2
        off = (F * nst + s) * 2048 + q * 1024 + (h * 32 + c) * 16 + b
        assert raw[e, off] == packed[e, k // 2, n]
    # padding holds zero weights
    if K % 128 or N % 32:
        total = int(raw.to(torch.int64).sum())
        assert total == int(packed.to(torch.int64).sum())


@pytest.mark.parametrize("E, K, N", [(1, 128, 32), (3, 96, 40), (2, 2880, 96)])
def test_scale_layout_round_trip_and_placement(E, K, N):
    g = torch.Generator().manual_seed(K * N)
    sc = torch.randint(100, 140, (E, N, K // 32), generator=g, dtype=torch.uint8).transpose(1, 2)  # [E, K/32, N]
    t = wrap_torch_tensor(sc)
    tiled = convert_layout(t, GFX950MXScaleLayout())
    nfr, nst = (N + 31) // 32, (K // 32 + 3) // 4
    assert list(tiled.storage.data.shape) == [E, nfr * nst * 128]
    back = convert_layout(tiled, StridedLayout(-2))
    assert torch.equal(back.storage.data, sc)
    raw = tiled.storage.data
    for (e, kb, n) in [(0, 0, 0), (E - 1, K // 32 - 1, N - 1), (0, 1, 7)]:
        F, c, s, j = n // 32, n % 32, kb // 4, kb % 4
        assert raw[e, (F * nst + s) * 128 + c * 4 + j] == sc[e, kb, n]


def test_default_layout_helpers():
    assert isinstance(make_default_matmul_mxfp4_w_layout(mx_axis=1), GFX950MXValueLayout)
    assert isinstance(make_default_matmul_mxfp4_w_scale_layout(mx_axis=1), GFX950MXScaleLayout)
    assert isinstance(make_default_matmul_mxfp4_w_layout(mx_axis=2), StridedLayout)
    with pytest.raises(ValueError):
        GFX950MXValueLayout().storage_shape([2, 64, 32], False)
    assert UINT8.bitwidth == 8


@pytest.mark.parametrize("E, K, N", [(1, 128, 32), (3, 96, 40), (2, 4096 + 16, 96), (2, 320, 70)])
def test_fp8_value_layout_round_trip_and_placement(E, K, N):
    g = torch.Generator().manual_seed(K + N)
    raw8 = torch.randint(1, 120, (E, N, K), generator=g, dtype=torch.uint8)
    w = raw8.view(torch.float8_e4m3fn).transpose(1, 2)  # [E, K, N], K-contiguous as the GEMM takes strided fp8 weights
    t = wrap_torch_tensor(w)
    assert t.shape == [E, K, N]
    tiled = convert_layout(t, GFX950FP8ValueLayout())
    nfr, nst = (N + 31) // 32, 2 * ((K + 255) // 256)
    assert list(tiled.storage.data.shape) == [E, nfr * nst * 4096] == GFX950FP8ValueLayout().storage_shape([E, K, N], False)
    back = convert_layout(tiled, StridedLayout(-2))
    assert torch.equal(back.storage.data.view(torch.uint8), w.view(torch.uint8))
    raw = tiled.storage.data
    for (e, k, n) in [(0, 0, 0), (E - 1, K - 1, N - 1), (0, 70, 5), (E - 1, K // 2 + 3, N // 2)]:
        F, c, s, kk = n // 32, n % 32, k // 128, k % 128
        tt, h, half, b = kk // 64, (kk % 64) // 32, (kk % 32) // 16, kk % 16
        off = (F * nst + s) * 4096 + (tt * 2 + half) * 1024 + (h * 32 + c) * 16 + b
        assert raw[e, off] == raw8[e, n, k]
    assert int((raw != 0).sum()) == raw8.numel()  # padding holds zero weights
