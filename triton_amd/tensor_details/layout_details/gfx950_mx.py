"""Pre-tiled MXFP4 weight layouts for the gfx950 expert GEMM.

The counterpart of the reference's architecture-specific weight layouts
(`triton_kernels/tensor_details/layout.py:26-54`; e.g. `CDNA4MXScaleLayout`,
`layout_details/cdna4_scale.py:11-86`): the weights are re-ordered once, with `convert_layout`, into the order
the kernel's wavefronts read them, so that every load instruction fetches one contiguous KiB.

Logical operand `[E, K, N]` (K = reduction, packed e2m1 along K).  Per expert, per fragment F of 32 output
columns (N padded to 32) and per K-stage s of 128 (K padded to 128 with zero weights):

  values  one 2048-byte block ordered [q:2][h:2][c:32][16 bytes]: the 16 packed bytes of column F*32 + c for
          k in [s*128 + h*64 + q*32, +32); blocks ordered [F][s];
  scales  one 128-byte block ordered [c:32][4]: the stage's four e8m0 bytes of column F*32 + c.

Storage is a `[E, bytes]` uint8 tensor for both.

`GFX950FP8ValueLayout` is the same idea for e4m3 weights (one byte per element, no MX scales) feeding the FP8 MFMA
`v_mfma_f32_32x32x64_f8f6f4`: K is padded to 256 (an even number of 128-blocks) and per (F, s) one 4096-byte block ordered [t:2][half:2][h:2][c:32][16 bytes] with the
bytes of column F*32 + c for k in [s*128 + t*64 + h*32 + half*16, +16).
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from .base import Layout, LayoutTransformation
from .strided import repack

FRAG_N = 32
STAGE_K = 128


def _cdiv(a, b):
    return (a + b - 1) // b


@dataclass(frozen=True)
class GFX950MXValueLayout(Layout):

    @property
    def name(self):
        return "GFX950_MX_VALUE"

    def make_transformation(self, shape, is_fp4: bool) -> LayoutTransformation:
        if not is_fp4:
            raise ValueError("GFX950MXValueLayout holds packed e2m1 (FP4) values")
        return GFX950MXValueLayoutTransformation(list(shape), is_fp4)

    def swizzle_block_shape(self, block_shape):
        return block_shape


@dataclass(frozen=True)
class GFX950MXValueLayoutTransformation(LayoutTransformation):

    def _dims(self):
        *lead, K, N = self.shape
        E = 1
        for v in lead:
            E *= v
        return E, K, N, _cdiv(N, FRAG_N), _cdiv(K, STAGE_K)

    @property
    def storage_shape(self) -> list:
        E, K, N, nfr, nst = self._dims()
        return [E, nfr * nst * 2048]

    def swizzle_data(self, data):
        """`data`: canonical form `[..., K, N/2]` (packed along the last dim)."""
        E, K, N, nfr, nst = self._dims()
        if K % 2:
            raise ValueError(f"FP4 packing dimension K must have an even size, got {K}")
        kmaj = repack(data.reshape(E, K, N // 2), -1, -2, True)  # [E, K/2, N], packed along K
        pad = torch.zeros((E, nst * 64, nfr * FRAG_N), dtype=torch.uint8, device=data.device)
        pad[:, :K // 2, :N] = kmaj
        # byte index along K/2 = s*64 + h*32 + q*16 + b ; column = F*32 + c
        t = pad.view(E, nst, 2, 2, 16, nfr, FRAG_N)  # [E, s, h, q, b, F, c]
        t = t.permute(0, 5, 1, 3, 2, 6, 4)  # [E, F, s, q, h, c, b]
        return t.contiguous().view(E, nfr * nst * 2048)

    def unswizzle_data(self, data):
        E, K, N, nfr, nst = self._dims()
        t = data.view(E, nfr, nst, 2, 2, FRAG_N, 16).permute(0, 2, 4, 3, 6, 1, 5)  # [E, s, h, q, b, F, c]
        kmaj = t.reshape(E, nst * 64, nfr * FRAG_N)[:, :K // 2, :N].contiguous()
        out = repack(kmaj, -2, -1, True)  # [E, K, N/2]
        return out.view(*self.shape[:-1], N // 2)


@dataclass(frozen=True)
class GFX950MXScaleLayout(Layout):

    @property
    def name(self):
        return "GFX950_MX_SCALE"

    def make_transformation(self, shape, is_fp4: bool) -> LayoutTransformation:
        if is_fp4:
            raise ValueError("GFX950MXScaleLayout holds e8m0 scale bytes")
        return GFX950MXScaleLayoutTransformation(list(shape), is_fp4)

    def swizzle_block_shape(self, block_shape):
        return block_shape


@dataclass(frozen=True)
class GFX950MXScaleLayoutTransformation(LayoutTransformation):
    """Logical scale tensor `[..., K/32, N]`."""

    def _dims(self):
        *lead, KB, N = self.shape
        E = 1
        for v in lead:
            E *= v
        return E, KB, N, _cdiv(N, FRAG_N), _cdiv(KB, 4)

    @property
    def storage_shape(self) -> list:
        E, KB, N, nfr, nst = self._dims()
        return [E, nfr * nst * 128]

    def swizzle_data(self, data):
        E, KB, N, nfr, nst = self._dims()
        pad = torch.full((E, nst * 4, nfr * FRAG_N), 127, dtype=torch.uint8, device=data.device)  # 2^0 over zero weights
        pad[:, :KB, :N] = data.reshape(E, KB, N)
        t = pad.view(E, nst, 4, nfr, FRAG_N).permute(0, 3, 1, 4, 2)  # [E, F, s, c, 4]
        return t.contiguous().view(E, nfr * nst * 128)

    def unswizzle_data(self, data):
        E, KB, N, nfr, nst = self._dims()
        t = data.view(E, nfr, nst, FRAG_N, 4).permute(0, 2, 4, 1, 3)  # [E, s, 4, F, c]
        out = t.reshape(E, nst * 4, nfr * FRAG_N)[:, :KB, :N].contiguous()
        return out.view(*self.shape)


@dataclass(frozen=True)
class GFX950FP8ValueLayout(Layout):

    @property
    def name(self):
        return "GFX950_FP8_VALUE"

    def make_transformation(self, shape, is_fp4: bool) -> LayoutTransformation:
        if is_fp4:
            raise ValueError("GFX950FP8ValueLayout holds one-byte (e4m3) values")
        return GFX950FP8ValueLayoutTransformation(list(shape), is_fp4)

    def swizzle_block_shape(self, block_shape):
        return block_shape


@dataclass(frozen=True)
class GFX950FP8ValueLayoutTransformation(LayoutTransformation):
    """Logical operand `[..., K, N]` of one-byte values; storage `[E, nfr * nst * 4096]` uint8."""

    def _dims(self):
        *lead, K, N = self.shape
        E = 1
        for v in lead:
            E *= v
        return E, K, N, _cdiv(N, FRAG_N), 2 * _cdiv(K, 2 * STAGE_K)  # K padded to 256: an even number of 128-blocks

    @property
    def storage_shape(self) -> list:
        E, K, N, nfr, nst = self._dims()
        return [E, nfr * nst * 4096]

    def swizzle_data(self, data):
        """`data`: canonical `[..., K, N]` with unit stride along N (float8 or uint8 bytes)."""
        E, K, N, nfr, nst = self._dims()
        pad = torch.zeros((E, nst * STAGE_K, nfr * FRAG_N), dtype=torch.uint8, device=data.device)
        pad[:, :K, :N] = data.reshape(E, K, N).view(torch.uint8)
        # k = s*128 + t*64 + h*32 + half*16 + b ; column = F*32 + c
        t = pad.view(E, nst, 2, 2, 2, 16, nfr, FRAG_N)  # [E, s, t, h, half, b, F, c]
        t = t.permute(0, 6, 1, 2, 4, 3, 7, 5)  # [E, F, s, t, half, h, c, b]
        return t.contiguous().view(E, nfr * nst * 4096)

    def unswizzle_data(self, data):
        E, K, N, nfr, nst = self._dims()
        t = data.view(E, nfr, nst, 2, 2, 2, FRAG_N, 16).permute(0, 2, 3, 5, 4, 7, 1, 6)  # [E, s, t, h, half, b, F, c]
        out = t.reshape(E, nst * STAGE_K, nfr * FRAG_N)[:, :K, :N].contiguous()
        return out.view(*self.shape)
