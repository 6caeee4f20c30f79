"""Tile selection for the ragged GEMM and the constraint-scoping API
(mirrors the user interface of `triton_kernels/matmul_details/opt_flags.py:20-38,482-603`).

The HIP GEMM is compiled for a fixed set of tile shapes, selected by `block_m` (rows of one expert per
workgroup) and the weight format:

    block_m   mxfp4 / fp8 weights        bf16 weights           use
              block_n  block_k  waves    block_n  block_k
      16        128      256      4        128      128         decode: a few rows per expert
      32        128      256      4        128      128
      64        256      128      4        128      128
     128        256      128      4        128      128         prefill: ~128 rows per expert
     256        256      128      4         -        -          pre-tiled MXFP4 only: a whole expert (<= 160 rows) per tile

so only `block_m` can be forced; `block_n`, `block_k` and `num_warps` constraints must match the table.
`split_k > 1` and `is_persistent=True` cannot be honoured and raise `InapplicableConstraint`, which is
what the reference's own tests skip on AMD (tests/test_matmul.py:377-383).
"""
from __future__ import annotations

from contextlib import contextmanager
from contextvars import ContextVar
from dataclasses import dataclass

TILE_TABLE = {  # narrow (4-bit / 8-bit) weights
    16: dict(block_n=128, block_k=256, num_warps=4),
    32: dict(block_n=128, block_k=256, num_warps=4),
    64: dict(block_n=256, block_k=128, num_warps=4),
    128: dict(block_n=256, block_k=128, num_warps=4),
    256: dict(block_n=256, block_k=128, num_warps=4),  # pre-tiled MXFP4 weights only: one tile per expert of <= 160 rows
}
TILE_TABLE_16BIT = {bm: dict(block_n=128, block_k=128, num_warps=4) for bm in TILE_TABLE}


def tile_for(block_m: int, rhs_dtype=None) -> dict:
    """The compiled tile for `block_m` and a weight dtype (torch dtype, package dtype or None = narrow)."""
    bits = getattr(rhs_dtype, "bitwidth", None)
    if bits is None:
        bits = getattr(rhs_dtype, "itemsize", 1) * 8
    return (TILE_TABLE_16BIT if bits >= 16 else TILE_TABLE)[block_m]


@dataclass
class OptFlags:
    block_m: int
    block_n: int
    block_k: int
    num_warps: int
    num_stages: int
    group_m: int
    xcd_swizzle: int
    w_cache_modifier: str | None
    split_k: int
    is_persistent: bool
    idle_sms: int
    epilogue_subtile: int | None
    arch: str | None
    occupancy_target: int
    target_kernel_kwargs: dict
    clc: bool = False
    swap_xw: bool | None = None
    use_output_tma: bool | None = None


class InapplicableConstraint(Exception):
    pass


_SUPPORTED = {
    "block_m", "block_n", "block_k", "split_k", "is_persistent", "epilogue_subtile", "idle_sms", "max_allowable_mn",
    "num_warps", "disable_mx4_block_swap"
}

_opt_flags_constraints: ContextVar = ContextVar("opt_flags_constraints", default=None)
_opt_flags: ContextVar = ContextVar("opt_flags", default=None)
_idle_sms = 0


def _get_idle_sms() -> int:
    return _idle_sms


def set_idle_sms(num_idle_sms: int):
    global _idle_sms
    _idle_sms = num_idle_sms


def _get_opt_flags_constraints() -> dict:
    c = _opt_flags_constraints.get()
    return {} if c is None else c


def update_opt_flags_constraints(constraints: dict):
    updated = dict(_get_opt_flags_constraints())
    updated.update(constraints)
    _opt_flags_constraints.set(updated)


def reset_opt_flags_constraints():
    _opt_flags_constraints.set(None)


@contextmanager
def scoped_opt_flags_constraints(constraints):
    updated = dict(_get_opt_flags_constraints())
    updated.update(constraints)
    token = _opt_flags_constraints.set(updated)
    try:
        yield
    finally:
        _opt_flags_constraints.reset(token)


def reset_opt_flags():
    _opt_flags.set(None)


def set_opt_flags(opt_flags: OptFlags):
    assert not _get_opt_flags_constraints(), "setting constraints is incompatible with manual flags override"
    assert _opt_flags.get() is None, "opt_flags already set; please reset to None first"
    _opt_flags.set(opt_flags)


@contextmanager
def scoped_opt_flags(opt_flags: OptFlags):
    token = _opt_flags.set(opt_flags)
    try:
        yield
    finally:
        _opt_flags.reset(token)


def default_block_m(m, ragged_metadata) -> int:
    """Rows of one expert per workgroup, from the expected rows per expert."""
    if ragged_metadata is None:
        slice_size = m
    elif ragged_metadata.expected_slice_size is None:
        slice_size = max(1, m // max(1, ragged_metadata.n_slices))
    else:
        slice_size = ragged_metadata.expected_slice_size
    if slice_size <= 16:
        return 16
    if slice_size <= 32:
        return 32
    if slice_size <= 64:
        return 64
    return 128


def make_opt_flags(out_dtype, lhs_dtype, rhs_dtype, precision_config, batch_size, m, n, k, ragged_metadata,
                   can_use_persistent_tma=False, can_use_split_k=False, epilogue_effective_itemsize=None,
                   x_transpose=False, has_y_acc_in=False, block_k=None, intermediate_out_dtype=None, mx_block_size=None,
                   x_uses_tma_when_persistent=True, w_transpose=False, rhs_layout=None, epilogue_reduction_n=1):
    constraints = _get_opt_flags_constraints()
    unsupported = set(constraints.keys()) - _SUPPORTED
    assert not unsupported, f"Given unsupported constraint: {unsupported}"
    if constraints.get("is_persistent", False):
        raise InapplicableConstraint("cannot enforce `is_persistent=True` constraint")
    if constraints.get("split_k") is not None and constraints.get("split_k") > 1:
        if not constraints.get("max_allowable_mn"):
            raise InapplicableConstraint("cannot enforce `split_k=True` constraint")
    if constraints.get("max_allowable_mn") and not constraints.get("split_k"):
        raise InapplicableConstraint("split_k also needs to be provided with max_allowable_mn")
    forced = _opt_flags.get()
    if forced is not None:
        assert not constraints
        assert block_k is None
        if forced.block_m not in TILE_TABLE:
            raise InapplicableConstraint(f"block_m={forced.block_m} is not one of {sorted(TILE_TABLE)}")
        return forced
    block_m = constraints.get("block_m") or default_block_m(m, ragged_metadata)
    if block_m not in TILE_TABLE:
        raise InapplicableConstraint(f"block_m={block_m} is not one of {sorted(TILE_TABLE)}")
    tile = tile_for(block_m, rhs_dtype)
    for key in ("block_n", "block_k", "num_warps"):
        want = constraints.get(key)
        if want is not None and want != tile[key]:
            raise InapplicableConstraint(f"{key}={want} does not match the compiled tile for block_m={block_m} ({tile[key]})")
    return OptFlags(
        block_m=block_m,
        block_n=tile["block_n"],
        block_k=tile["block_k"],
        num_warps=tile["num_warps"],
        num_stages=2,
        group_m=1,
        xcd_swizzle=8,
        w_cache_modifier=None,
        split_k=1,
        is_persistent=False,
        idle_sms=constraints.get("idle_sms", _get_idle_sms()),
        epilogue_subtile=constraints.get("epilogue_subtile") or 1,
        arch="gfx950",
        occupancy_target=1,
        target_kernel_kwargs={},
    )
