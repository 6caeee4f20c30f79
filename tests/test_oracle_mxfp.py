"""Pins the MX oracle (oracle/mxfp.py) against the reference's own golden vectors
(python/triton_kernels/tests/test_mxfp.py:92-205), closed forms and brute force; also checks the
library's host-evaluated scalar conversions against the oracle.  CPU only."""
import numpy as np
import pytest
import torch

from oracle import mxfp

DTYPES = [torch.float16, torch.bfloat16, torch.float32]
E2M1 = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]


@pytest.mark.parametrize("dt", DTYPES)
def test_rounding_golden(dt):
    # tests/test_mxfp.py:95-114
    ulp = {torch.bfloat16: 0.251953125, torch.float16: 0.250244140625, torch.float32: 0.2500000298023223877}[dt]
    x = torch.tensor([6, 0, 0.24, 0.25, 0.75, 0.99, 1.2, 1.3, -1.25, ulp] + [0] * 22, dtype=dt).view(1, -1, 1)
    q, s = mxfp.downcast_to_mxfp(x, torch.uint8, axis=1)
    d = mxfp.upcast_from_mxfp(q, s, dt, axis=1)
    assert d.flatten().tolist() == [6, 0, 0, 0.0, 1.0, 1.0, 1.0, 1.5, -1.0, 0.5] + [0] * 22
    assert s.flatten().tolist() == [127]
    assert q.stride(1) == 1 and s.stride(1) == 1


@pytest.mark.parametrize("dt", DTYPES)
def test_round_down_golden(dt):
    # tests/test_mxfp.py:128-141
    x = torch.tensor([33.0, 24.0, 16.0, 8.0, 4.0, 0.0, -32.0, 0.0] + [0] * 24).bfloat16().view(1, -1, 1)
    q, s = mxfp.downcast_to_mxfp(x, torch.uint8, axis=1, rounding=mxfp.ROUND_DOWN)
    assert s.item() == 127 + 3
    d = mxfp.upcast_from_mxfp(q, s, dt, axis=1)
    assert torch.equal(d[0, 1:, :].float(), x[0, 1:, :].float())


@pytest.mark.parametrize("src", [torch.uint8, torch.float8_e5m2, torch.float8_e4m3fn])
@pytest.mark.parametrize("dt", DTYPES)
def test_extreme_values_stay_finite(src, dt):
    # tests/test_mxfp.py:154-168
    big = 65470 if dt == torch.float16 else 3.3895e38
    x = torch.tensor([big, big] + [0] * 30, dtype=dt)
    q, s = mxfp.downcast_to_mxfp(x, src, axis=-1)
    d = mxfp.upcast_from_mxfp(q, s, dt, axis=-1)
    assert not d.isinf().any() and not d.isnan().any()


@pytest.mark.parametrize("src", [torch.uint8, torch.float8_e5m2, torch.float8_e4m3fn])
@pytest.mark.parametrize("dt", DTYPES)
def test_exact_round_trip_set(src, dt):
    # tests/test_mxfp.py:173-205: representable values times power-of-two scales survive exactly
    max_val = mxfp._MAX_Q[mxfp._kind(src)]
    if src == torch.float8_e5m2 and dt == torch.float16:
        max_val = 128
    pos = torch.tensor(E2M1[:-1] + [max_val], dtype=dt)
    kdim = torch.cat([pos, -pos]).reshape(-1, 1)
    scales = (2.0**torch.arange(-8, 8, dtype=dt)).reshape(1, -1)
    w = (kdim * scales).repeat((9, 32)).unsqueeze(0)
    w = torch.nn.functional.pad(w.mT.contiguous().mT, (0, 0, 0, 16))
    q, s = mxfp.downcast_to_mxfp(w, src, axis=1)
    d = mxfp.upcast_from_mxfp(q, s, dt, axis=1)
    assert torch.equal(w, d)


def test_scale_closed_form():
    # ROUND_UP scale = smallest power of two s with max/s <= max_q; ROUND_DOWN = 2^floor(log2(max/max_pow2)).
    rng = np.random.default_rng(1)
    m = np.abs(rng.standard_normal(20000).astype(np.float32)) * np.float32(2.0)**rng.integers(-60, 60, 20000)
    m = np.concatenate([m, np.float32([6.0, 3.0, 1.5, 0.75, 448.0, 224.0, 4.0, 8.0, 1.0])]).astype(np.float32)
    for kind in ("e2m1", "e4m3", "e5m2"):
        up = mxfp.scale_bits_from_absmax(m, kind, mxfp.ROUND_UP).view(np.float32).astype(np.float64)
        mq = mxfp._MAX_Q[kind]
        assert np.all(m / up <= mq) and np.all(m / (up / 2) > mq)
        dn = mxfp.scale_bits_from_absmax(m, kind, mxfp.ROUND_DOWN).view(np.float32).astype(np.float64)
        expect = 2.0**np.floor(np.log2(m.astype(np.float64) / mxfp._MAX_POW2_Q[kind]))
        assert np.array_equal(dn, expect)
    assert mxfp.scale_bits_from_absmax(np.float32([0.0]), "e2m1", mxfp.ROUND_UP)[0] == 0


def _nearest_even_e2m1(a: np.ndarray) -> np.ndarray:
    """Independent statement: nearest representable magnitude, ties to the even code, saturate at 6."""
    cand = np.array(E2M1, dtype=np.float64)
    a = np.minimum(np.abs(a.astype(np.float64)), 6.0)
    d = np.abs(a[:, None] - cand[None, :])
    best = d.min(axis=1, keepdims=True)
    is_best = d == best
    code = np.argmax(is_best, axis=1)
    tie = is_best.sum(axis=1) > 1
    code = np.where(tie & (code % 2 == 1), code + 1, code)
    return code


def test_e2m1_rounding_brute_force():
    bits = (np.arange(65536, dtype=np.uint32) << 16).view(np.float32)  # every bf16 value
    bits = bits[np.isfinite(bits)]
    extra = np.float32(np.linspace(0, 8, 200001))
    x = np.concatenate([bits, extra, -extra])
    got = mxfp.e2m1_codes_from_f32(x)
    assert np.array_equal(got & 7, _nearest_even_e2m1(x))
    assert np.array_equal((got >> 3).astype(bool), np.signbit(x))


def test_packing_and_layout():
    x = torch.arange(64, dtype=torch.float32).view(1, 64, 1).repeat(3, 1, 5) / 16
    q, s = mxfp.downcast_to_mxfp(x, torch.uint8, axis=1)
    assert q.shape == (3, 32, 5) and s.shape == (3, 2, 5)
    assert q.stride(1) == 1 and s.stride(1) == 1
    codes = mxfp.e2m1_codes_from_f32((x[0, :32, 0] / 2.0**(int(s[0, 0, 0]) - 127)).numpy())
    assert int(q[0, 0, 0]) == int(codes[0]) | (int(codes[1]) << 4)  # even element in the low nibble


def test_library_host_conversions_match_oracle():
    nt = pytest.importorskip("triton_amd._native")
    L = nt.lib()
    rng = np.random.default_rng(0)
    bf = (np.arange(65536, dtype=np.uint32) << 16).view(np.float32)
    rnd = rng.integers(0, 2**32, size=1_000_000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    x = np.concatenate([bf, rnd, np.float32(rng.uniform(-8, 8, 500_000))]).astype(np.float32)
    x = np.ascontiguousarray(x[~np.isnan(x)])
    out = np.zeros(x.shape[0], dtype=np.uint8)
    assert L.tk_host_mx_convert(x.ctypes.data, x.shape[0], nt.TK_E2M1, out.ctypes.data) == 0
    assert np.array_equal(out, mxfp.e2m1_codes_from_f32(x))
    for kind, dt, mq in [(nt.TK_E4M3, torch.float8_e4m3fn, 448.0), (nt.TK_E5M2, torch.float8_e5m2, 57344.0)]:
        assert L.tk_host_mx_convert(x.ctypes.data, x.shape[0], kind, out.ctypes.data) == 0
        ref = torch.from_numpy(x).clamp(-mq, mq).to(dt).view(torch.uint8).numpy()
        assert np.array_equal(out, ref)
    m = np.abs(x[np.isfinite(x)])[:200000].copy()
    sc = np.zeros(m.shape[0], dtype=np.uint8)
    for kind, name in [(nt.TK_E2M1, "e2m1"), (nt.TK_E4M3, "e4m3"), (nt.TK_E5M2, "e5m2")]:
        for r in (0, 1):
            assert L.tk_host_mx_scale(m.ctypes.data, m.shape[0], kind, r, sc.ctypes.data) == 0
            ref = (mxfp.scale_bits_from_absmax(m, name, r) >> 23).astype(np.uint8)
            assert np.array_equal(sc, ref)
