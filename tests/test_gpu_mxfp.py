"""GPU parity of the MX quantise / dequantise kernels (through the C ABI) against the CPU oracle.

Cases mirror python/triton_kernels/tests/test_mxfp.py:92-291; the full benchmark shape
[32, 2880, 5760] is checked through size-independent properties plus oracle comparison on slices."""
import pytest
import torch

from oracle import mxfp as omx
from oracle.checks import assert_close, assert_equal

pytestmark = pytest.mark.gpu

DTYPES = [torch.float16, torch.bfloat16, torch.float32]
QTYPES = [torch.uint8, torch.float8_e5m2, torch.float8_e4m3fn]


@pytest.fixture(scope="module")
def mx(device):
    from triton_amd.numerics_details import mxfp
    return mxfp


def _same(a, b, what):
    assert_equal(a.view(torch.uint8) if a.dtype.itemsize == 1 else a, b.view(torch.uint8) if b.dtype.itemsize == 1 else b, what)


@pytest.mark.parametrize("dt", DTYPES)
def test_rounding_cases(mx, device, dt):
    ulp = {torch.bfloat16: 0.251953125, torch.float16: 0.250244140625, torch.float32: 0.2500000298023223877}[dt]
    x = torch.tensor([6, 0, 0.24, 0.25, 0.75, 0.99, 1.2, 1.3, -1.25, ulp] + [0] * 22, dtype=dt, device=device).view(1, -1, 1)
    q, s = mx.downcast_to_mxfp(x, torch.uint8, axis=1)
    d = mx.upcast_from_mxfp(q, s, dt, axis=1)
    assert d.flatten().tolist() == [6, 0, 0, 0.0, 1.0, 1.0, 1.0, 1.5, -1.0, 0.5] + [0] * 22
    qo, so = omx.downcast_to_mxfp(x, torch.uint8, axis=1)
    _same(qo, q, "values")
    _same(so, s, "scales")
    x = torch.tensor([33.0, 24.0, 16.0, 8.0, 4.0, 0.0, -32.0, 0.0] + [0] * 24, device=device).bfloat16().view(1, -1, 1)
    q, s = mx.downcast_to_mxfp(x, torch.uint8, axis=1, DEQUANT_SCALE_ROUNDING_MODE=mx.DequantScaleRoundingMode.ROUND_DOWN)
    assert s.item() == 130
    d = mx.upcast_from_mxfp(q, s, dt, axis=1)
    assert torch.equal(d[0, 1:, :].float(), x[0, 1:, :].float())


@pytest.mark.parametrize("src", QTYPES)
@pytest.mark.parametrize("dt", DTYPES)
def test_extreme_values(mx, device, src, dt):
    big = 65470 if dt == torch.float16 else 3.3895e38
    x = torch.tensor([big, big] + [0] * 30, dtype=dt, device=device)
    q, s = mx.downcast_to_mxfp(x, src, axis=-1)
    d = mx.upcast_from_mxfp(q, s, dt, axis=-1)
    _same(omx.upcast_from_mxfp(q, s, dt, axis=-1), d, "dequant")
    assert not d.isinf().any()


@pytest.mark.parametrize("src", QTYPES)
@pytest.mark.parametrize("dt", DTYPES)
def test_exact_round_trip_set(mx, device, src, dt):
    max_val = mx.get_max_quant_val(src)
    if src == torch.float8_e5m2 and dt == torch.float16:
        max_val = 128
    pos = torch.tensor([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, max_val], dtype=dt, device=device)
    kdim = torch.cat([pos, -pos]).reshape(-1, 1)
    scales = (2.0**torch.arange(-8, 8, dtype=dt, device=device)).reshape(1, -1)
    w = (kdim * scales).repeat((9, 32)).unsqueeze(0)
    w = torch.nn.functional.pad(w.mT.contiguous().mT, (0, 0, 0, 16))
    q, s = mx.downcast_to_mxfp(w, src, axis=1)
    d = mx.upcast_from_mxfp(q, s, dt, axis=1)
    assert torch.equal(w, d)


def test_pitched_input(mx, device):
    torch.manual_seed(0)
    dense = torch.randn((64, 128), device=device, dtype=torch.bfloat16)
    pitched = torch.empty_strided(dense.shape, (256, 1), device=device, dtype=dense.dtype)
    pitched.copy_(dense)
    q, s = mx.downcast_to_mxfp(pitched, torch.uint8, axis=-1)
    qe, se = mx.downcast_to_mxfp(dense, torch.uint8, axis=-1)
    assert torch.equal(q, qe) and torch.equal(s, se)


CASES = [
    ((0, 4096, 1024), 1, torch.uint8, 0),
    ((3, 4096, 0), 1, torch.uint8, 1),
    ((10, 0, 1024), 2, torch.float8_e5m2, 0),
    ((0, 0, 1024), 2, torch.float8_e4m3fn, 1),
    ((3, 4096, 1024), 1, torch.uint8, 0),
    ((32, 254, 60), 0, torch.uint8, 1),
    ((1, 320, 160), 2, torch.float8_e5m2, 0),
    ((2, 16, 512), -1, torch.float8_e4m3fn, 1),
    ((5, 96, 33), 1, torch.uint8, 0),  # odd inner: one column per lane
    ((2, 64, 130), 1, torch.float8_e4m3fn, 0),
    ((3, 96, 516), 1, torch.uint8, 1),  # tile kernels: partial column tile, 3 of 8 blocks
    ((2, 160, 260), 1, torch.float8_e4m3fn, 0),  # 5 blocks = one full fp8 tile of 4 + 1
    ((2, 352, 1028), 1, torch.float8_e5m2, 1),
    ((4, 288, 8, 36), 1, torch.uint8, 0),  # two inner dims
    ((7, 2880), 1, torch.uint8, 0),
    ((2880, 6), 0, torch.uint8, 0),
]


@pytest.mark.parametrize("shape, axis, qdt, rounding", CASES)
@pytest.mark.parametrize("dt", DTYPES)
def test_casting_matches_oracle(mx, device, shape, axis, qdt, rounding, dt):
    torch.manual_seed(0)
    x = torch.randn(shape, dtype=dt, device=device)
    mode = mx.DequantScaleRoundingMode(rounding)
    q, s = mx.downcast_to_mxfp(x, qdt, axis, DEQUANT_SCALE_ROUNDING_MODE=mode)
    qo, so = omx.downcast_to_mxfp(x, qdt, axis, rounding=rounding)
    _same(qo, q, "values")
    _same(so, s, "scales")
    if x.numel() > 0:
        assert q.stride(axis) == 1 and s.stride(axis) == 1
    d = mx.upcast_from_mxfp(q, s, dt, axis)
    do = omx.upcast_from_mxfp(qo, so, dt, axis)
    _same(do.contiguous(), d, "dequant")
    assert d.is_contiguous()
    if x.numel() > 0:
        assert_close(x, d, maxtol=0.5, rmstol=0.15)


def test_wide_dynamic_range_and_denormals(mx, device):
    # exponents spread over the whole fp32 range, including blocks that are all zero or denormal
    g = torch.Generator().manual_seed(3)
    e = torch.randint(-140, 120, (64, 96), generator=g).float()
    x = (torch.randn(64, 96 * 32, generator=g).view(64, 96, 32) * (2.0**e)[..., None]).view(64, -1)
    x[3, :64] = 0
    x = x.to(device)
    for qdt in QTYPES:
        q, s = mx.downcast_to_mxfp(x, qdt, axis=1)
        qo, so = omx.downcast_to_mxfp(x, qdt, axis=1)
        _same(qo, q, "values")
        _same(so, s, "scales")
        d = mx.upcast_from_mxfp(q, s, torch.float32, axis=1)
        _same(omx.upcast_from_mxfp(qo, so, torch.float32, axis=1).contiguous(), d, "dequant")


def test_baseline_shape_round_trip(mx, device):
    """[32, 2880, 5760] bf16, N(0, .02) with 0.1% +-U(4,16) outliers, quantised along axis 1."""
    g = torch.Generator(device="cpu").manual_seed(1)
    E, K, N = 32, 2880, 5760
    w = torch.empty((E, K, N), dtype=torch.bfloat16, device=device)
    for e in range(E):  # generated per expert on the CPU so the oracle sees identical bits
        we = torch.randn((K, N), generator=g) * 0.02
        mask = torch.rand((K, N), generator=g) < 1e-3
        out = (torch.rand((K, N), generator=g) * 12 + 4) * torch.where(torch.rand((K, N), generator=g) < 0.5, -1.0, 1.0)
        w[e] = torch.where(mask, out, we).to(torch.bfloat16).to(device)
    q, s = mx.downcast_to_mxfp(w, torch.uint8, axis=1)
    assert q.shape == (E, K // 2, N) and s.shape == (E, K // 32, N)
    assert q.stride() == (K // 2 * N, 1, K // 2) and s.stride() == (K // 32 * N, 1, K // 32)
    d = mx.upcast_from_mxfp(q, s, torch.bfloat16, axis=1)
    assert d.shape == w.shape and d.is_contiguous()
    # oracle on two whole experts
    for e in (0, 31):
        qo, so = omx.downcast_to_mxfp(w[e:e + 1], torch.uint8, axis=1)
        _same(qo, q[e:e + 1], f"values[{e}]")
        _same(so, s[e:e + 1], f"scales[{e}]")
        _same(omx.upcast_from_mxfp(qo, so, torch.bfloat16, axis=1).contiguous(), d[e:e + 1], f"dequant[{e}]")
    # size-independent properties on the whole tensor
    # dequantise o quantise is idempotent: every dequantised value is representable again (the block
    # scale may drop by a power of two when the block maximum rounded down, the values do not move)
    q2, s2 = mx.downcast_to_mxfp(d, torch.uint8, axis=1)
    d2 = mx.upcast_from_mxfp(q2, s2, torch.bfloat16, axis=1)
    assert torch.equal(d2, d)
    assert bool((s2 <= s).all())
    del q2, s2, d2
    # ROUND_UP never clips, and the widest e2m1 gap is 2 (4 -> 6): |error| <= 1 * block scale everywhere
    for e in range(E):
        err = (d[e].float() - w[e].float()).abs().view(K // 32, 32, N)
        step = torch.exp2(s[e].float() - 127)  # [K/32, N]
        assert bool((err <= step[:, None, :]).all())


@pytest.mark.parametrize("M, K, view", [(37, 4096, "plain"), (5, 1000, "plain"), (9, 1003, "plain"), (6, 520, "offset"), (3, 7, "plain"),
                                        (4, 14336, "plain"), (3, 8256, "plain"), (2, 20000, "plain"),
                                        # rows that a workgroup keeps in registers between the two passes (2048 < K <= 32768,
                                        # aligned), with a partly filled last piece, and the same length unaligned (two-pass kernel)
                                        (5, 2056, "plain"), (3, 3000, "plain"), (3, 4096, "offset"), (3, 8192, "plain"),
                                        # long rows: eight pieces per thread up to 16384 elements, sixteen up to 32768, the two-pass
                                        # kernel beyond
                                        (2, 16384, "plain"), (3, 14344, "plain"), (2, 16392, "plain"), (2, 32768, "plain"), (2, 32776, "plain")])
def test_quantize_fp8_rowwise_bit_exact(device, M, K, view):
    """Per-row e4m3 quantiser (the FP8 configuration's activation path): bytes bit-exact and scales equal to the
    oracle's, on rows that take the vector path, rows with a scalar tail, and rows that are not 16-byte aligned;
    one row is all zero (scale 1) and one holds the value that must saturate to 448."""
    from oracle import moe as omoe
    from triton_amd.numerics_details.rowwise_fp8 import quantize_fp8_rowwise
    g = torch.Generator().manual_seed(M * 1000 + K)
    base = (torch.randn((M, K + 8), generator=g) * 3).to(torch.bfloat16)
    base[0] = 0
    x = base[:, 1:K + 1] if view == "offset" else base[:, :K]
    xd = base.to(device)
    xd = xd[:, 1:K + 1] if view == "offset" else xd[:, :K]
    q, s = quantize_fp8_rowwise(xd)
    q_ref, s_ref = omoe.quantize_fp8_rowwise(x)
    assert torch.equal(s.cpu(), s_ref)
    assert torch.equal(q.cpu().view(torch.uint8), q_ref.view(torch.uint8))


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16])
def test_infinite_inputs_match_oracle(mx, device, dt):
    """+-inf elements: the block scale becomes 2^128 (byte 255), inf * 0 is NaN and saturates to +-6 with the sign of its
    bit pattern, the finite elements of the block become 0 (mxfp.py:255-327); checked on the strided-axis kernels
    (LDS-transposed tile path and the plain one) against the oracle.  NaN inputs are left out: whether the block
    maximum propagates them differs between the reference's own two implementations."""
    g = torch.Generator().manual_seed(9)
    x = torch.randn((2, 64, 260), generator=g).to(dt)
    x[0, 3, 5] = float("inf")
    x[0, 40, 7] = float("-inf")
    x[1, 33, 259] = float("-inf")
    for xs in (x, x[:, :, :131].contiguous()):  # inner 260: tile kernels; inner 131: one column per lane
        q, s = mx.downcast_to_mxfp(xs.to(device), torch.uint8, axis=1)
        qo, so = omx.downcast_to_mxfp(xs, torch.uint8, axis=1)
        _same(qo, q, "values")
        _same(so, s, "scales")
