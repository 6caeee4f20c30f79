"""The reference's pre-shuffled MX scale layout for CDNA4 (`triton_kernels/tensor_details/layout_details/
cdna4_scale.py:11-86`), kept so that scale tensors prepared for the reference load here unchanged.

Logical operand `[..., KS, N]` (KS = K / 32 scale rows).  KS is padded to a multiple of 8 and N to a multiple of
32; within a batch the byte at flat position

    p = ((((n32 * (KS_pad / 8) + k8) * 4 + d) * 16 + r) * 2 + b) * 2 + a

holds the scale of row ks = k8 * 8 + b * 4 + d and column n = n32 * 32 + a * 16 + r, i.e. each 32-column by
8-row block is stored as 256 consecutive bytes.  The storage tensor is `[B, KS_pad * 32, N_pad / 32]` with unit
stride along dim -2 (flat position = column-block * KS_pad * 32 + row), padding bytes are zero.

`matmul` consumes this layout by converting it once to the kernel's own scale order (the converted tensor is
cached on the wrapper), since the kernels here read either strided scales or `GFX950MXScaleLayout`.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from .base import Layout, LayoutTransformation

N_BLOCK = 32
KS_BLOCK = 8


@dataclass(frozen=True)
class CDNA4MXScaleLayout(Layout):

    @property
    def name(self):
        return "CDNA4_SCALE"

    def make_transformation(self, shape, is_fp4: bool) -> LayoutTransformation:
        return CDNA4MXScaleLayoutTransformation(list(shape), is_fp4)

    def swizzle_block_shape(self, block_shape):
        ks, n = block_shape[-2:]
        return list(block_shape[:-2]) + [n // N_BLOCK, ks * N_BLOCK]


@dataclass(frozen=True)
class CDNA4MXScaleLayoutTransformation(LayoutTransformation):

    def _dims(self):
        *lead, ks, n = self.shape
        b = 1
        for v in lead:
            b *= v
        ks_pad = -(-ks // KS_BLOCK) * KS_BLOCK
        n_pad = -(-n // N_BLOCK) * N_BLOCK
        return lead, b, ks, n, ks_pad, n_pad

    @property
    def storage_shape(self) -> list:
        _, b, _, _, ks_pad, n_pad = self._dims()
        return [b, ks_pad * N_BLOCK, n_pad // N_BLOCK]

    def _source_of_position(self, device):
        """(ks, n) held by every flat storage position of one batch entry."""
        _, _, _, _, ks_pad, n_pad = self._dims()
        p = torch.arange(ks_pad * n_pad, device=device)
        a, b, r, d = p % 2, (p // 2) % 2, (p // 4) % 16, (p // 64) % 4
        k8 = (p // 256) % (ks_pad // KS_BLOCK)
        n32 = p // (256 * (ks_pad // KS_BLOCK))
        return k8 * 8 + b * 4 + d, n32 * 32 + a * 16 + r

    def swizzle_data(self, data):
        """`data`: canonical `[..., KS, N]` with unit stride along N."""
        assert not self.is_fp4, "MX scales are bytes, not packed FP4"
        _, b, ks, n, ks_pad, n_pad = self._dims()
        padded = torch.zeros((b, ks_pad, n_pad), dtype=data.dtype, device=data.device)
        padded[:, :ks, :n] = data.reshape(b, ks, n)
        src_ks, src_n = self._source_of_position(data.device)
        flat = padded[:, src_ks, src_n]  # [B, KS_pad * N_pad] in storage order
        return flat.view(b, n_pad // N_BLOCK, ks_pad * N_BLOCK).transpose(-1, -2)

    def unswizzle_data(self, data):
        lead, b, ks, n, ks_pad, n_pad = self._dims()
        flat = data.transpose(-1, -2).reshape(b, ks_pad * n_pad)
        src_ks, src_n = self._source_of_position(data.device)
        padded = torch.empty((b, ks_pad, n_pad), dtype=data.dtype, device=data.device)
        padded[:, src_ks, src_n] = flat
        return padded[:, :ks, :n].reshape(*lead, ks, n).contiguous()
