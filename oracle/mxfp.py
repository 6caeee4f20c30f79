"""CPU oracle: microscaling (MX) quantise / dequantise.  Test infrastructure only.

Follows `python/triton_kernels/triton_kernels/numerics_details/mxfp.py`:
  * `downcast_to_mxfp`  <- `downcast_to_mxfp_torch`  (mxfp.py:192-343)
  * `upcast_from_mxfp`  <- `upcast_from_mxfp_torch` + `cvt_e2m1_to_fp32` (mxfp.py:346-429)

Integer / byte arithmetic is done in numpy; torch is used only to convert
bf16 / fp16 / fp8 to and from fp32.
"""
from __future__ import annotations

import numpy as np
import torch

MX_BLOCK = 32  # OCP microscaling block (mxfp_details/_downcast_to_mxfp.py:9)

ROUND_UP = 0  # DequantScaleRoundingMode.ROUND_UP   (mxfp.py:19-24)
ROUND_DOWN = 1  # DequantScaleRoundingMode.ROUND_DOWN

# largest finite value of each element format (mxfp.py:187-189)
_MAX_Q = {"e2m1": 6.0, "e4m3": 448.0, "e5m2": 57344.0}
# largest power of two of each element format (_downcast_to_mxfp.py:24-30)
_MAX_POW2_Q = {"e2m1": 4.0, "e4m3": 256.0, "e5m2": 32768.0}

_KIND_OF = {torch.uint8: "e2m1", torch.float8_e4m3fn: "e4m3", torch.float8_e5m2: "e5m2"}
_TORCH_OF = {"e4m3": torch.float8_e4m3fn, "e5m2": torch.float8_e5m2}

E2M1_VALUES = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0], dtype=np.float32)


def _kind(out_dtype) -> str:
    if isinstance(out_dtype, str):
        return out_dtype
    return _KIND_OF[out_dtype]


def scale_bits_from_absmax(absmax: np.ndarray, kind: str, rounding: int) -> np.ndarray:
    """fp32 block maxima -> int32 bit pattern of the power-of-two dequant scale.

    mxfp.py:255-268: ROUND_UP adds 0x007FFFFF before masking the exponent field,
    ROUND_DOWN masks only.
    """
    absmax = absmax.astype(np.float32)
    if rounding == ROUND_UP:
        d = (absmax / np.float32(_MAX_Q[kind])).astype(np.float32)
        bits = d.view(np.int32)
        return (bits + np.int32(0x007FFFFF)) & np.int32(0x7F800000)
    d = (absmax / np.float32(_MAX_POW2_Q[kind])).astype(np.float32)
    return d.view(np.int32) & np.int32(0x7F800000)


def e2m1_codes_from_f32(q: np.ndarray) -> np.ndarray:
    """fp32 (already divided by the scale) -> 4-bit e2m1 codes, round-to-nearest-even, saturating.

    Bit algorithm of mxfp.py:298-327.
    """
    u = np.ascontiguousarray(q, dtype=np.float32).view(np.uint32)
    sign = (u >> np.uint32(28)) & np.uint32(0x8)
    exp = ((u >> np.uint32(23)) & np.uint32(0xFF)).astype(np.int64)
    man = (u & np.uint32(0x7FFFFF)).astype(np.int64)
    sub = exp < 127
    shift = np.clip(127 - exp - 1, 0, 63)
    man_pre = np.int64(0x400000) | (man >> 1)
    dropped0 = (man & 1) != 0
    mask = (np.int64(1) << np.minimum(shift, 31)) - 1
    dropped_post = (man_pre & mask) != 0
    sticky = sub & (dropped0 | dropped_post)
    mant = np.where(sub, man_pre >> shift, man)
    e_out = np.maximum(exp, 126) - 126
    m2 = (mant >> 21) & 3
    lsb = (m2 >> 1) & 1
    guard = m2 & 1
    sticky = sticky | ((mant & 0x1FFFFF) != 0)
    inc = guard & (sticky.astype(np.int64) | lsb)
    code = np.minimum((((e_out << 2) | m2) + inc) >> 1, 7)
    return (sign.astype(np.uint8) | code.astype(np.uint8)).astype(np.uint8)


def downcast_to_mxfp(x: torch.Tensor, out_dtype, axis: int, rounding: int = ROUND_UP):
    """Quantise `x` along `axis` in blocks of 32.

    Returns `(values, scales)` as torch tensors with `x`'s dimension order and
    `stride(axis) == 1` (mxfp.py:335-343).  e2m1 values are packed two per uint8
    along `axis`, even index in the low nibble (mxfp.py:329-333).
    """
    kind = _kind(out_dtype)
    ndim = x.ndim
    axis = axis if axis >= 0 else axis + ndim
    assert x.dtype in (torch.float32, torch.bfloat16, torch.float16)
    src = x.detach().to("cpu").transpose(axis, ndim - 1).to(torch.float32).contiguous().numpy()
    L = src.shape[-1]
    assert L % MX_BLOCK == 0, "quantised axis must be a multiple of 32"
    lead = src.shape[:-1]
    if src.size == 0:
        vshape = lead + ((L // 2) if kind == "e2m1" else L, )
        vdt = torch.uint8 if kind == "e2m1" else _TORCH_OF[kind]
        vals = torch.empty(vshape, dtype=vdt)
        scl = torch.empty(lead + (L // MX_BLOCK, ), dtype=torch.uint8)
        return vals.transpose(axis, ndim - 1), scl.transpose(axis, ndim - 1)
    blocks = src.reshape(-1, L // MX_BLOCK, MX_BLOCK)
    absmax = np.abs(blocks).max(axis=-1, keepdims=True)
    sbits = scale_bits_from_absmax(absmax, kind, rounding)
    s = sbits.view(np.float32)
    with np.errstate(divide="ignore"):
        inv = np.where(s == 0, np.float32(0), (np.float32(1.0) / s).astype(np.float32)).astype(np.float32)
    with np.errstate(invalid="ignore"):  # inf * 0 (an infinite element in a block whose scale overflowed) is NaN on purpose
        q = (blocks * inv).astype(np.float32)
    scale_bytes = (sbits >> 23).astype(np.uint8).reshape(lead + (L // MX_BLOCK, ))
    if kind == "e2m1":
        codes = e2m1_codes_from_f32(q).reshape(-1, L // 2, 2)
        packed = (codes[..., 0] | (codes[..., 1] << 4)).astype(np.uint8).reshape(lead + (L // 2, ))
        vals = torch.from_numpy(packed)
    else:
        mq = np.float32(_MAX_Q[kind])
        qc = np.clip(q, -mq, mq).reshape(lead + (L, ))  # saturating cast (mxfp.py:293-296)
        vals = torch.from_numpy(qc).to(_TORCH_OF[kind])
    scl = torch.from_numpy(scale_bytes)
    return vals.transpose(axis, ndim - 1), scl.transpose(axis, ndim - 1)


def e2m1_unpack_to_f32(packed: np.ndarray) -> np.ndarray:
    """uint8 [..., n] -> fp32 [..., 2n]; low nibble first (mxfp.py:346-361)."""
    lut = np.concatenate([E2M1_VALUES, -E2M1_VALUES]).astype(np.float32)
    lo = lut[packed & 0xF]
    hi = lut[(packed >> 4) & 0xF]
    return np.stack([lo, hi], axis=-1).reshape(packed.shape[:-1] + (packed.shape[-1] * 2, ))


def upcast_from_mxfp(values: torch.Tensor, scales: torch.Tensor, target_dtype: torch.dtype, axis: int):
    """Dequantise.  Product in fp32, clamp to the target's finite range, cast (mxfp.py:364-429).

    Returns a tensor in `values`' dimension order with `stride(axis) == 1`
    (the twin returns the transposed view of a contiguous buffer).
    """
    ndim = values.ndim
    axis = axis if axis >= 0 else axis + ndim
    v = values.detach().to("cpu").transpose(axis, ndim - 1).contiguous()
    s = scales.detach().to("cpu").transpose(axis, ndim - 1).contiguous().numpy()
    if v.dtype == torch.uint8:
        f = e2m1_unpack_to_f32(v.numpy())
    else:
        f = v.to(torch.float32).numpy()
    L = f.shape[-1]
    if L == 0:
        return torch.from_numpy(f).to(target_dtype).transpose(axis, ndim - 1)
    assert L % MX_BLOCK == 0 and s.shape[-1] == L // MX_BLOCK
    dq = (s.astype(np.int32) << 23).view(np.float32)
    blocks = f.reshape(f.shape[:-1] + (L // MX_BLOCK, MX_BLOCK))
    finfo = torch.finfo(target_dtype)
    with np.errstate(invalid="ignore", over="ignore"):
        out = (blocks * dq[..., None]).astype(np.float32)
        out = np.clip(out, np.float32(finfo.min), np.float32(finfo.max))
    if values.dtype == torch.float8_e5m2:
        isinf = np.isinf(blocks)
        out = np.where(isinf, blocks, out)  # infinities pass through (mxfp.py:416-418)
    out = out.reshape(f.shape)
    return torch.from_numpy(out).to(target_dtype).transpose(axis, ndim - 1)
