"""`CDNA4MXScaleLayout` (the reference's scale pre-shuffle for this GPU): round trips on the reference's shapes
(tests/test_tensor_details/test_layout_cdna4.py:12-38), zero-sized tensors, storage shape, and element placement
against the kernel-side inverse the reference documents (cdna4_scale.py:80-86: a [BLOCK_N/32, KS/8, 4, 16, 2, 2]
view permuted to (n32, a, r, k8, b, d) gives back [BLOCK_N, KS])."""
import pytest
import torch

from triton_kernels.tensor import convert_layout, wrap_torch_tensor
from triton_kernels.tensor_details.layout import CDNA4MXScaleLayout, GFX950MXScaleLayout, StridedLayout


@pytest.mark.parametrize("shape", [(0, 64), (64, 0), (2, 0), (0, 2), (0, 64, 64)])
def test_zero_sized_roundtrip(shape):
    x = torch.empty(shape, dtype=torch.uint8)
    src = wrap_torch_tensor(x)
    swizzled = convert_layout(src, CDNA4MXScaleLayout())
    back = convert_layout(swizzled, src.storage.layout)
    assert back.storage.data.shape == x.shape


@pytest.mark.parametrize("shape", [(3, 512, 1024), (10, 254, 60), (1, 320, 160), (2, 16, 512), (3, 2, 36), (90, 96)])
def test_roundtrip_shape_and_padding(shape):
    g = torch.Generator().manual_seed(sum(shape))
    x = torch.randint(1, 256, shape, dtype=torch.uint8, generator=g)
    tr = CDNA4MXScaleLayout().make_transformation(x.shape, is_fp4=False)
    sw = tr.swizzle_data(x)
    ks, n = shape[-2:]
    b = x.numel() // (ks * n)
    ks_pad, n_pad = -(-ks // 8) * 8, -(-n // 32) * 32
    assert list(sw.shape) == tr.storage_shape == [b, ks_pad * 32, n_pad // 32]
    assert sw.stride(-2) == 1
    assert int((sw != 0).sum()) == x.numel()  # padding bytes are zero, every real scale (>= 1) is kept
    assert torch.equal(tr.unswizzle_data(sw), x)


def test_placement_matches_kernel_side_inverse():
    """One [BLOCK_N = 64, KS = 16] block: reading the stored bytes through the reference's kernel-side view must
    give scale[n, ks]."""
    ks, n = 16, 64
    x = (torch.arange(ks * n, dtype=torch.int32).reshape(ks, n) % 251).to(torch.uint8)  # [KS, N]
    sw = CDNA4MXScaleLayout().make_transformation([1, ks, n], False).swizzle_data(x[None])
    flat = sw.transpose(-1, -2).reshape(-1)  # memory order
    v = flat.view(n // 32, ks // 8, 4, 16, 2, 2, 1).permute(0, 5, 3, 1, 4, 2, 6).reshape(n, ks)
    assert torch.equal(v, x.T)


def test_convert_to_kernel_layouts():
    g = torch.Generator().manual_seed(5)
    x = torch.randint(100, 140, (2, 96, 90), dtype=torch.uint8, generator=g).transpose(1, 2)  # [E, KS=90, N=96], KS-contiguous
    cd = convert_layout(wrap_torch_tensor(x), CDNA4MXScaleLayout())
    assert torch.equal(convert_layout(cd, StridedLayout(-2)).storage.data, x)
    direct = convert_layout(wrap_torch_tensor(x), GFX950MXScaleLayout())
    assert torch.equal(convert_layout(cd, GFX950MXScaleLayout()).storage.data, direct.storage.data)
