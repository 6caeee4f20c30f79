"""Host-side mirror of the reference's operator interface: names, data classes, layouts, tile constraints and
the argument checks that run before any kernel is launched.  CPU only."""
import importlib

import pytest
import torch

import triton_kernels  # noqa: F401  (alias package: triton_kernels.X is triton_amd.X)
from triton_kernels.matmul_details import opt_flags as of
from triton_kernels.tensor import (BIT, FP4, UINT8, RaggedTensorMetadata, Tensor, convert_layout, empty, wrap_torch_tensor)
from triton_kernels.tensor_details.layout import StridedLayout
from triton_kernels.tensor_details.layout_details.strided import repack


def test_reference_module_names_resolve():
    # the import lines of the reference's benchmark and tests (bench/bench_mlp.py:1-25, tests/test_matmul.py:1-40)
    names = {
        "triton_kernels.matmul": ["matmul", "PrecisionConfig", "FlexCtx", "FnSpecs", "FusedActivation", "Epilogue"],
        "triton_kernels.topk": ["topk"],
        "triton_kernels.reduce": ["reduce"],
        "triton_kernels.swiglu": ["swiglu", "swiglu_fn", "PrecisionConfig"],
        "triton_kernels.numerics_details.mxfp": ["downcast_to_mxfp", "upcast_from_mxfp", "DequantScaleRoundingMode", "MXFP_BLOCK_SIZE"],
        "triton_kernels.tensor": ["SparseMatrix", "RaggedTensor", "make_ragged_tensor_metadata", "make_bitmatrix_metadata", "wrap_torch_tensor",
                                  "convert_layout", "FP4", "Tensor", "Storage"],
        "triton_kernels.tensor_details.layout": ["StridedLayout", "make_default_matmul_mxfp4_w_layout", "make_default_matmul_mxfp4_w_scale_layout"],
        "triton_kernels.matmul_details.opt_flags": ["make_opt_flags", "scoped_opt_flags_constraints", "update_opt_flags_constraints",
                                                    "reset_opt_flags_constraints", "InapplicableConstraint", "OptFlags"],
        "triton_kernels.legacy": ["routing", "RoutingData", "GatherIndx", "ScatterIndx", "matmul_ogs"],
        "triton_kernels.target_info": ["is_hip", "is_hip_cdna4", "is_cuda"],
    }
    for mod, attrs in names.items():
        m = importlib.import_module(mod)
        for a in attrs:
            assert hasattr(m, a), f"{mod}.{a}"
    import triton_amd.matmul
    assert importlib.import_module("triton_kernels.matmul") is triton_amd.matmul


@pytest.mark.parametrize(("logical_shape", "is_fp4", "layout", "storage_shape"), [
    ((3, 258, 514), True, StridedLayout(-2), [3, 129, 514]),
    ((0, 64), True, StridedLayout(-2), [0, 64]),
    ((3, 258, 514), True, StridedLayout(-1), [3, 258, 257]),
    ((3, 70, 65), False, StridedLayout(-2), [3, 70, 65]),
])
def test_layout_storage_shape_matches_conversion(logical_shape, is_fp4, layout, storage_shape):
    # tests/test_tensor.py:85-118 (the strided rows of its table)
    t = empty(logical_shape, dtype=FP4 if is_fp4 else UINT8, device="meta")
    converted = convert_layout(t, layout)
    assert layout.storage_shape(list(logical_shape), is_fp4) == storage_shape
    assert list(converted.storage.data.shape) == storage_shape


@pytest.mark.parametrize("major_dim", [-1, -2])
@pytest.mark.parametrize("other_size", [0, 2])
def test_strided_layout_rejects_odd_fp4_packing_dim(major_dim, other_size):
    # tests/test_tensor.py:128-135
    shape = [other_size, other_size]
    shape[major_dim] = 1
    with pytest.raises(ValueError):
        StridedLayout(major_dim).storage_shape(shape, True)


def test_strided_layout_order_and_errors():
    assert StridedLayout(-1).order(3) == [2, 1, 0]
    assert StridedLayout(-2).order(3) == [1, 2, 0]
    assert StridedLayout(0).order(3) == [0, 1, 2]
    with pytest.raises(ValueError):
        StridedLayout(3).order(3)
    with pytest.raises(TypeError):
        StridedLayout("k")


def test_wrap_fp4_doubles_the_unit_stride_dim():
    # tensor.py:216-233: uint8 storage of FP4 has two elements per byte along the contiguous dimension
    w = torch.zeros((4, 16, 6), dtype=torch.uint8).transpose(1, 2).contiguous().transpose(1, 2)  # strides (96, 1, 16)
    t = wrap_torch_tensor(w, dtype=FP4)
    assert t.shape == [4, 32, 6] and t.storage.layout == StridedLayout(-2)
    t = wrap_torch_tensor(torch.zeros((4, 16, 6), dtype=torch.uint8), dtype=FP4)
    assert t.shape == [4, 16, 12] and t.storage.layout == StridedLayout(-1)
    with pytest.raises(ValueError):
        Tensor(t.storage, dtype=FP4)  # sub-byte types need an explicit shape
    assert BIT.bitwidth == 1 and FP4.bitwidth == 4


def test_repack_moves_nibbles_between_dims():
    g = torch.Generator().manual_seed(0)
    vals = torch.randint(0, 16, (3, 8, 6), generator=g, dtype=torch.uint8)  # one nibble per logical element
    pack_last = vals[..., 0::2] | (vals[..., 1::2] << 4)  # [3, 8, 3]
    pack_mid = vals[:, 0::2, :] | (vals[:, 1::2, :] << 4)  # [3, 4, 6]
    assert torch.equal(repack(pack_last, -1, -2, True), pack_mid)
    assert torch.equal(repack(pack_mid, -2, -1, True), pack_last)
    assert repack(pack_last, -1, -1, True) is pack_last
    with pytest.raises(TypeError):
        repack(pack_last.to(torch.float32), -1, -2, True)


def test_convert_layout_round_trip_fp4():
    g = torch.Generator().manual_seed(1)
    data = torch.randint(0, 256, (2, 6, 8), generator=g, dtype=torch.uint8)
    t = wrap_torch_tensor(data, dtype=FP4)  # logical [2, 6, 16], packed along the last dim
    k_major = convert_layout(t, StridedLayout(-2))
    assert list(k_major.storage.data.shape) == [2, 3, 16] and k_major.storage.data.stride(1) == 1
    back = convert_layout(k_major, StridedLayout(-1))
    assert torch.equal(back.storage.data, data)
    assert convert_layout(t, StridedLayout(-1)) is t


def test_ragged_metadata_static_helpers():
    # ragged_tensor.py:73-89
    assert RaggedTensorMetadata.block_sizes() == [16, 32, 64, 128, 256]
    assert RaggedTensorMetadata.n_blocks(128, 16384, 16) == 1144
    assert RaggedTensorMetadata.max_n_blocks(128, 16384) == 1144
    assert RaggedTensorMetadata.n_blocks(8, 3, 64) == 3


def test_opt_flags_constraints_scope_and_tiles():
    of.reset_opt_flags_constraints()
    flags = of.make_opt_flags(None, None, FP4, None, 1, 16384, 5760, 2880, None)
    assert (flags.block_m, flags.block_n, flags.block_k, flags.split_k, flags.is_persistent) == (128, 256, 128, 1, False)
    with of.scoped_opt_flags_constraints({"block_m": 16}):
        f = of.make_opt_flags(None, None, FP4, None, 1, 16384, 5760, 2880, None)
        assert (f.block_m, f.block_n, f.block_k) == (16, 128, 256)
        f = of.make_opt_flags(None, None, torch.bfloat16, None, 1, 16384, 5760, 2880, None)
        assert (f.block_m, f.block_n, f.block_k) == (16, 128, 128)
        with of.scoped_opt_flags_constraints({"block_n": 64}):
            with pytest.raises(of.InapplicableConstraint):
                of.make_opt_flags(None, None, FP4, None, 1, 64, 64, 64, None)
    assert of._get_opt_flags_constraints() == {}
    for bad in ({"is_persistent": True}, {"split_k": 4}, {"block_m": 48}, {"max_allowable_mn": 1024}):
        with of.scoped_opt_flags_constraints(bad):
            with pytest.raises(of.InapplicableConstraint):
                of.make_opt_flags(None, None, FP4, None, 1, 64, 64, 64, None)
    with of.scoped_opt_flags_constraints({"no_such_knob": 1}):
        with pytest.raises(AssertionError):
            of.make_opt_flags(None, None, FP4, None, 1, 64, 64, 64, None)
    of.update_opt_flags_constraints({"block_m": 32})
    assert of.make_opt_flags(None, None, FP4, None, 1, 4096, 64, 64, None).block_m == 32
    of.reset_opt_flags_constraints()


def test_default_block_m_follows_rows_per_expert():
    class Md:
        n_slices = 128
        expected_slice_size = None

    assert of.default_block_m(16384, Md()) == 128
    assert of.default_block_m(64 * 4, Md()) == 16
    assert of.default_block_m(40, None) == 64
    Md.expected_slice_size = 20
    assert of.default_block_m(16384, Md()) == 32


def test_constraints_are_per_context():
    import contextvars
    of.reset_opt_flags_constraints()

    def inner():
        of.update_opt_flags_constraints({"block_m": 64})
        return of._get_opt_flags_constraints()

    assert contextvars.copy_context().run(inner) == {"block_m": 64}
    assert of._get_opt_flags_constraints() == {}


def test_cpu_tensors_are_refused_not_computed():
    # there is no CPU path: every operator refuses host tensors before doing anything
    from triton_kernels.matmul import matmul
    from triton_kernels.numerics_details.mxfp import downcast_to_mxfp, upcast_from_mxfp
    from triton_kernels.reduce import reduce
    from triton_kernels.swiglu import PrecisionConfig, swiglu
    from triton_kernels.topk import topk
    x = torch.zeros((32, 64), dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="HIP device"):
        matmul(x, torch.zeros((64, 32), dtype=torch.bfloat16), None)
    with pytest.raises(RuntimeError, match="HIP device"):
        topk(torch.zeros((4, 8)), 2)
    with pytest.raises(RuntimeError, match="HIP device"):
        downcast_to_mxfp(x, torch.uint8, axis=1)
    with pytest.raises(RuntimeError, match="HIP device"):
        upcast_from_mxfp(torch.zeros((32, 32), dtype=torch.uint8), torch.zeros((32, 2), dtype=torch.uint8), torch.bfloat16, axis=1)
    with pytest.raises(RuntimeError, match="HIP device"):
        swiglu(x, 1.0, PrecisionConfig(limit=None))
    with pytest.raises(RuntimeError, match="HIP device"):
        reduce(x.view(16, 2, 64), dim=1)


def test_mx_argument_checks_match_the_reference():
    # mxfp.py:39-47: axis range and divisibility are checked before any work
    from triton_kernels.numerics_details.mxfp import downcast_to_mxfp
    with pytest.raises((AssertionError, ValueError)):
        downcast_to_mxfp(torch.zeros((4, 8), dtype=torch.bfloat16), torch.uint8, axis=2)
    with pytest.raises((AssertionError, ValueError)):
        downcast_to_mxfp(torch.zeros((4, 7), dtype=torch.bfloat16), torch.uint8, axis=1)


def test_weight_relayout_cache_key_and_invalidation():
    """The K-contiguous copy `matmul` keeps on an N-contiguous weight tensor follows in-place torch updates through the
    version counter; writes through `.data` do not bump it (checked here), so `invalidate_weight_cache` is the
    documented way to drop the copy after such a write.  Inference-mode tensors have no counter and must not raise."""
    from triton_amd.matmul import _cache_key, _k_contiguous, invalidate_weight_cache
    w = torch.randn(2, 8, 16)
    c0 = _k_contiguous(w)
    assert c0.stride(-2) == 1 and torch.equal(c0, w)
    assert _k_contiguous(w) is c0  # cached
    w.add_(1.0)  # visible to the version counter: a new copy
    c1 = _k_contiguous(w)
    assert c1 is not c0 and torch.equal(c1, w)
    v = w._version
    w.data.mul_(2.0)  # NOT visible
    assert w._version == v and _k_contiguous(w) is c1 and not torch.equal(c1, w)
    invalidate_weight_cache(w)
    c2 = _k_contiguous(w)
    assert c2 is not c1 and torch.equal(c2, w)
    # a different storage under the same Python object (set_) changes the key as well
    w.set_(torch.randn(2, 8, 16))
    assert torch.equal(_k_contiguous(w), w)
    with torch.inference_mode():
        wi = torch.randn(2, 8, 16)
    assert _cache_key(wi)[1] is None
    assert torch.equal(_k_contiguous(wi), wi)
    # already K-contiguous weights are used in place
    wk = torch.randn(2, 16, 8).transpose(1, 2)
    assert _k_contiguous(wk) is wk


def test_routing_data_records_whether_every_token_has_all_its_rows():
    from triton_amd.legacy import RoutingData
    assert RoutingData.__dataclass_fields__["all_rows_live"].default is False
