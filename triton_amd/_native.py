"""ctypes binding of `libtriton_amd.so` (the C ABI declared in include/triton_amd.h).

The library is loaded lazily on first use and a missing library is a hard error: there is no
fallback implementation.
"""
from __future__ import annotations

import ctypes
import os
import threading

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libtriton_amd.so")

TK_OK, TK_ERR_INVALID, TK_ERR_UNSUPPORTED, TK_ERR_LAUNCH = 0, 1, 2, 3

# enum tk_dtype
TK_F32, TK_BF16, TK_F16, TK_E4M3, TK_E5M2, TK_E2M1, TK_U8, TK_I16, TK_I32 = range(9)

TORCH_TO_TK = {
    torch.float32: TK_F32,
    torch.bfloat16: TK_BF16,
    torch.float16: TK_F16,
    torch.float8_e4m3fn: TK_E4M3,
    torch.float8_e5m2: TK_E5M2,
    torch.uint8: TK_U8,
    torch.int16: TK_I16,
    torch.int32: TK_I32,
}

_c = ctypes
_i32, _i64, _ptr, _f32 = _c.c_int32, _c.c_int64, _c.c_void_p, _c.c_float

TK_ACT_NONE, TK_ACT_SWIGLU = 0, 1
TK_W_STRIDED, TK_W_TILED = 0, 1


class RouteDesc(_c.Structure):
    """struct tk_route_desc (field order and types follow include/triton_amd.h)."""
    _fields_ = [
        ("logits", _ptr), ("logits_dtype", _i32), ("logits_stride_m", _i64), ("n_tokens", _i32), ("n_rows", _i32),
        ("n_rows_ptr", _ptr), ("n_experts", _i32), ("k", _i32), ("apply_softmax", _i32), ("use_provided_indx", _i32),
        ("vals", _ptr), ("indx", _ptr), ("indx_dtype", _i32), ("bitmatrix", _ptr), ("bitmatrix_stride_w", _i64),
        ("col_sum", _ptr), ("col_sorted_indx", _ptr), ("row_sorted_indx", _ptr), ("gather_indx", _ptr),
        ("gammas", _ptr), ("slice_offs", _ptr), ("block_offs", _ptr), ("block_offs_stride", _i64),
        ("block_schedule", _ptr), ("block_schedule_stride", _i64), ("max_n_blocks", _i32), ("workspace", _ptr),
    ]


class GemmDesc(_c.Structure):
    """struct tk_gemm_desc (field order and types follow include/triton_amd.h)."""
    _fields_ = [
        ("x", _ptr), ("x_dtype", _i32), ("x_stride_m", _i64), ("x_row_scale", _ptr),
        ("w", _ptr), ("w_dtype", _i32), ("w_stride_e", _i64), ("w_stride_k", _i64), ("w_stride_n", _i64),
        ("w_mx_scale", _ptr), ("ws_stride_e", _i64), ("ws_stride_k", _i64), ("ws_stride_n", _i64),
        ("w_col_scale", _ptr), ("wcs_stride_e", _i64),
        ("bias", _ptr), ("bias_dtype", _i32), ("bias_stride_e", _i64),
        ("gather_indx", _ptr), ("scatter_indx", _ptr), ("scatter_len", _i32),
        ("gammas", _ptr), ("gammas_dtype", _i32),
        ("slice_sizes", _ptr), ("slice_offs", _ptr), ("block_offs", _ptr), ("block_schedule", _ptr),
        ("n_slices", _i32), ("block_m", _i32), ("grid_m", _i32), ("M", _i32), ("N", _i32), ("K", _i32),
        ("y", _ptr), ("y_dtype", _i32), ("y_stride_m", _i64),
        ("activation", _i32), ("act_alpha", _f32), ("act_limit", _f32), ("act_has_limit", _i32),
        ("w_layout", _i32), ("idle_cus", _i32), ("tile_counters", _ptr), ("x_rows", _i64),
        ("x_mx_scale", _ptr), ("xs_stride_m", _i64), ("y_mx_scale", _ptr), ("ys_stride_m", _i64),
        ("combine_k", _i32), ("combine_out", _ptr), ("combine_stride_m", _i64), ("combine_counters", _ptr),
        ("betas", _ptr), ("betas_dtype", _i32), ("has_out_alpha", _i32), ("out_alpha", _f32), ("acc_in", _ptr), ("acc_in_stride_m", _i64),
    ]


class RaggedKDesc(_c.Structure):
    """struct tk_ragged_k_desc (field order and types follow include/triton_amd.h)."""
    _fields_ = [
        ("a", _ptr), ("dtype", _i32), ("a_stride_m", _i64), ("a_stride_k", _i64),
        ("b", _ptr), ("b_stride_k", _i64), ("b_stride_n", _i64),
        ("y", _ptr), ("y_dtype", _i32), ("y_stride_e", _i64), ("y_stride_m", _i64),
        ("M", _i32), ("N", _i32), ("n_slices", _i32),
        ("slice_sizes", _ptr), ("a_slice_offs", _ptr), ("b_slice_offs", _ptr), ("a_k_extent", _i64), ("b_k_extent", _i64),
    ]


class DecodeLayerDesc(_c.Structure):
    """struct tk_decode_layer_desc (field order and types follow include/triton_amd.h)."""
    _fields_ = [
        ("x", _ptr), ("x_stride_m", _i64), ("logits", _ptr), ("logits_dtype", _i32), ("logits_stride_m", _i64),
        ("n_tokens", _i32), ("n_experts", _i32), ("k", _i32), ("apply_softmax", _i32), ("d_model", _i32), ("d_ff", _i32),
        ("w1", _ptr), ("w1_mx_scale", _ptr), ("w1_stride_e", _i64), ("w1s_stride_e", _i64),
        ("b1", _ptr), ("b1_dtype", _i32), ("b1_stride_e", _i64),
        ("w2", _ptr), ("w2_mx_scale", _ptr), ("w2_stride_e", _i64), ("w2s_stride_e", _i64),
        ("b2", _ptr), ("b2_dtype", _i32), ("b2_stride_e", _i64),
        ("act_alpha", _f32), ("act_limit", _f32), ("act_has_limit", _i32),
        ("out", _ptr), ("out_stride_m", _i64), ("indx_out", _ptr), ("vals_out", _ptr), ("workspace", _ptr), ("spin_limit", _i32),
    ]


# name -> (restype, argtypes); must list every symbol include/triton_amd.h declares.
SIGNATURES = {
    "tk_version": (_i32, []),
    "tk_last_error": (_c.c_char_p, []),
    "tk_mx_downcast": (_i32, [_ptr, _i32, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _ptr, _ptr, _i32, _i32, _ptr]),
    "tk_route_workspace_bytes": (_i64, [_i32, _i32]),
    "tk_route": (_i32, [_c.POINTER(RouteDesc), _ptr]),
    "tk_route_static": (_i32, [_c.POINTER(RouteDesc), _ptr]),
    "tk_route_static_prepare": (_i32, []),
    "tk_topk_backward": (_i32, [_ptr, _i32, _i64, _ptr, _i64, _ptr, _i64, _ptr, _i64, _i32, _i32, _i32, _i32, _i32, _ptr, _ptr]),
    "tk_ragged_metadata": (_i32, [_ptr, _i32, _ptr, _ptr, _i64, _ptr, _i64, _i32, _ptr]),
    "tk_ragged_remap": (_i32, [_ptr, _ptr, _ptr, _i64, _ptr, _i64, _ptr, _i32, _i32, _i32, _ptr, _ptr, _ptr, _i64, _ptr, _i64, _ptr]),
    "tk_moe_gemm": (_i32, [_c.POINTER(GemmDesc), _ptr]),
    "tk_ragged_k_gemm": (_i32, [_c.POINTER(RaggedKDesc), _ptr]),
    "tk_moe_decode_layer_workspace_bytes": (_i64, [_i32, _i32, _i32, _i32, _i32]),
    "tk_moe_decode_layer": (_i32, [_c.POINTER(DecodeLayerDesc), _ptr]),
    "tk_probe_mfma": (_i32, [_ptr, _i32, _i32, _i32, _ptr]),
    "tk_swiglu": (_i32, [_ptr, _i32, _i64, _i64, _i64, _ptr, _i64, _f32, _f32, _i32, _ptr, _ptr]),
    "tk_reduce_mid": (_i32, [_ptr, _i32, _i64, _i64, _i64, _i64, _i64, _ptr, _i64, _i64, _i64, _ptr, _i64, _i64, _i64, _ptr, _i64, _ptr]),
    "tk_reduce_mid_backward": (_i32, [_ptr, _i32, _i64, _i64, _i64, _i64, _ptr, _i64, _i64, _i64, _ptr, _i64, _i64, _i64, _ptr, _ptr]),
    "tk_quant_fp8_rows": (_i32, [_ptr, _i32, _i64, _i64, _i64, _ptr, _i64, _ptr, _ptr]),
    "tk_mx_upcast": (_i32, [_ptr, _ptr, _i32, _i64, _i64, _i64, _i64, _ptr, _i32, _i64, _i64, _i64, _ptr]),
    # host check hooks (no device work)
    "tk_host_mx_convert": (_i32, [_ptr, _i64, _i32, _ptr]),
    "tk_host_mx_scale": (_i32, [_ptr, _i64, _i32, _i32, _ptr]),
}

_lib = None
_lock = threading.Lock()


class NativeLibraryMissing(RuntimeError):
    pass


def lib():
    """The loaded library; raises NativeLibraryMissing when it has not been built."""
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                if not os.path.exists(LIB_PATH):
                    raise NativeLibraryMissing(
                        f"{LIB_PATH} not found: build it with `python -m triton_amd.build` (needs hipcc). "
                        "There is no fallback implementation.")
                handle = ctypes.CDLL(LIB_PATH)
                for name, (res, args) in SIGNATURES.items():
                    fn = getattr(handle, name)
                    fn.restype = res
                    fn.argtypes = args
                _lib = handle
    return _lib


def last_error() -> str:
    return lib().tk_last_error().decode("utf-8", "replace")


def check(status: int, what: str = ""):
    """Maps a status code of the C ABI to the exception the reference raises in the same situation."""
    if status == TK_OK:
        return
    msg = last_error() or what
    if status == TK_ERR_INVALID:
        raise ValueError(msg)
    if status == TK_ERR_UNSUPPORTED:
        raise NotImplementedError(msg)
    raise RuntimeError(msg)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_ptr(device=None) -> int:
    """The current PyTorch HIP stream of `device` as a raw hipStream_t."""
    if _raw_stream is not None:  # the direct binding: a fraction of a microsecond instead of several
        idx = device.index if isinstance(device, torch.device) and device.index is not None else torch.cuda.current_device()
        return _raw_stream(idx)
    return torch.cuda.current_stream(device).cuda_stream


class on_device:
    """`with on_device(t.device):` makes that device current for the launch, like `torch.cuda.device`, but costs
    next to nothing in the common case that it already is."""
    __slots__ = ("ctx", )

    def __init__(self, device):
        idx = device.index if isinstance(device, torch.device) else device
        self.ctx = None if idx is None or idx == torch.cuda.current_device() else torch.cuda.device(idx)

    def __enter__(self):
        if self.ctx is not None:
            self.ctx.__enter__()
        return self

    def __exit__(self, *exc):
        if self.ctx is not None:
            return self.ctx.__exit__(*exc)
        return False


def require_gpu(t: torch.Tensor, name: str = "tensor"):
    if not t.is_cuda:
        raise RuntimeError(f"{name} must live on a HIP device (got {t.device}); this package has no CPU path")


def ptr(t) -> int | None:
    return None if t is None else t.data_ptr()
