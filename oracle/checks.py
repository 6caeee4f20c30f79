"""Comparison helpers for the parity tests.  Test infrastructure only.

`rel_errors` / `assert_close` restate `assert_close` of
python/triton_kernels/triton_kernels/testing.py:27-88; `assert_equal` restates testing.py:18-24.
"""
from __future__ import annotations

import torch


def assert_equal(ref, got, what=""):
    if isinstance(ref, torch.Tensor):
        ref = ref.detach().to("cpu")
        got = got.detach().to("cpu")
        assert ref.shape == got.shape, f"{what}: shape {tuple(ref.shape)} vs {tuple(got.shape)}"
        if ref.dtype != got.dtype:
            got = got.to(ref.dtype) if not ref.dtype.is_floating_point else got
        same = ref.view(torch.uint8) == got.view(torch.uint8) if ref.dtype.itemsize == 1 and ref.dtype.is_floating_point else ref == got
        n_bad = int((~same).sum())
        assert n_bad == 0, f"{what}: {n_bad} / {ref.numel()} elements differ"
    else:
        assert ref == got, f"{what}: {ref} != {got}"


def rel_errors(ref: torch.Tensor, got: torch.Tensor):
    """(max, rms) of |ref-got| / max(rms(ref), |ref|) after normalising by max|ref|."""
    ref = ref.detach().to("cpu").to(torch.float32)
    got = got.detach().to("cpu").to(torch.float32)
    assert ref.shape == got.shape
    if ref.numel() == 0:
        return 0.0, 0.0
    inf_ref, inf_got = torch.isinf(ref), torch.isinf(got)
    assert torch.equal(inf_ref, inf_got), "infinite elements differ"
    refn = torch.where(inf_ref, torch.zeros_like(ref), ref)
    gotn = torch.where(inf_got, torch.zeros_like(got), got)
    eps = 1.0e-30
    mult = 1.0 / (refn.abs().max() + eps)
    refn = refn * mult
    gotn = gotn * mult
    ref_rms = torch.sqrt(torch.square(refn).mean()) + eps
    rel = (refn - gotn).abs() / torch.maximum(ref_rms, refn.abs())
    return float(rel.max()), float(torch.sqrt(torch.square(rel).mean()))


def assert_close(ref, got, maxtol=2e-2, rmstol=4e-3, what=""):
    mx, rms = rel_errors(ref, got)
    assert mx <= maxtol, f"{what}: max relative error {mx:.4g} > {maxtol}"
    assert rms <= rmstol, f"{what}: rms relative error {rms:.4g} > {rmstol}"
    return mx, rms


def assert_allclose_gate(ref, got, rtol=2e-2, atol=1e-2, what="", max_bad_frac=0.0):
    """The `torch.allclose`-style gate stated for bf16 GEMM outputs: |got-ref| <= atol + rtol*|ref|.
    `max_bad_frac` tolerates that fraction of elements outside the gate; it is zero for single GEMMs and
    set only where k bf16-rounded partial rows cancel in a sum (one bf16 ulp of a partial row can exceed
    atol + rtol*|sum| there)."""
    ref = ref.detach().to("cpu").to(torch.float32)
    got = got.detach().to("cpu").to(torch.float32)
    bad = (got - ref).abs() > (atol + rtol * ref.abs())
    n_bad = int(bad.sum())
    assert n_bad <= max_bad_frac * ref.numel(), f"{what}: {n_bad} / {ref.numel()} outside rtol={rtol} atol={atol}; worst {float((got-ref).abs().max()):.4g}"
