"""One-launch MoE FFN layer for decode-sized batches (no counterpart function in the reference).

The reference's MoE block is a sequence of calls (python/triton_kernels/bench/bench_mlp.py:72-79):

    rdata, gather, scatter = routing(logits, k)
    h   = matmul_ogs(x, w1, b1, rdata, gather_indx=gather, precision_config=pc1, fused_activation=swiglu)
    out = matmul_ogs(h, w2, b2, rdata, scatter_indx=scatter, precision_config=pc2, gammas=rdata.gate_scal)

`moe_mlp` computes the same `out` from the same arguments.  With a handful of tokens (T * k <= 256 routed rows), tiled
MXFP4 weights and d_model, d_ff <= 3072 it is ONE kernel launch (`tk_moe_decode_layer`: router, both expert GEMMs and
the top-k combine in a persistent grid); any other case runs the three calls above.  At these sizes the layer is a
stream of the active experts' weights, and launch boundaries plus the serial router in front of the first weight byte
cost a third of the three-call time.
"""
from __future__ import annotations

import torch

from . import _native as nt
from .matmul import FusedActivation, PrecisionConfig, _flex_out_is_trivial
from .tensor import FP4, Tensor
from .tensor_details.layout_details.gfx950_mx import GFX950MXScaleLayout, GFX950MXValueLayout

MAX_ROWS = 256
MIN_ROWS = 8  # below this `moe_mlp` prefers the three calls
MAX_EXPERTS = 512
MAX_DIM = 3072

_WORKSPACES: dict = {}


def _workspace(device, T, k, E, d_ff, d_model) -> torch.Tensor:
    """Scratch of the launch (hidden activations, the k partial rows, counters), one per (device, stream, shape), made
    on first use with its counter words zero; the kernel leaves them zero, so launches in stream order share it."""
    key = (device.index, nt.stream_ptr(device), T, k, E, d_ff, d_model)
    ws = _WORKSPACES.get(key)
    if ws is None:
        nbytes = nt.lib().tk_moe_decode_layer_workspace_bytes(T, k, E, d_ff, d_model)
        ws = torch.zeros(nbytes, dtype=torch.uint8, device=device)
        if len(_WORKSPACES) >= 64:
            _WORKSPACES.pop(next(iter(_WORKSPACES)))
        _WORKSPACES[key] = ws
    return ws


def workspace_error_word(x, logits, n_expts_act, w1) -> int:
    """The sticky error word of the workspace `moe_mlp` uses for these arguments on the current stream (synchronises;
    for tests): 0 = fine, bit 0 = a bounded wait ran out, bit 1 = the unit table overflowed."""
    T, E = logits.shape
    d_model, n1 = w1.shape[-2:]
    ws = _workspace(x.device, T, n_expts_act, E, n1 // 2, d_model)
    words = ws[-(2 + (MAX_ROWS + MAX_ROWS // 16) * 32 + T * ((d_model + 31) // 32)) * 4:].view(torch.int32)
    return int(words[1].item())


def _swiglu_args(act: FusedActivation | None):
    if act is None or act.specs.name != "swiglu" or act.specs.reduction_n != 2:
        return None
    alpha = float(act.fn_args[0])
    lim = act.fn_args[1] if len(act.fn_args) > 1 else None
    return alpha, (0.0 if lim is None else float(lim)), int(lim is not None)


def one_launch_reason(x, logits, n_expts_act, w1, b1, w2, b2, pc1, pc2, act) -> str | None:
    """None when `tk_moe_decode_layer` can run these arguments, else the reason it cannot."""
    if not (isinstance(x, torch.Tensor) and x.ndim == 2 and x.dtype == torch.bfloat16 and x.is_cuda):
        return "activations must be a 2-D bf16 device tensor"
    if logits.ndim != 2 or logits.dtype not in (torch.float32, torch.bfloat16) or logits.shape[0] != x.shape[0]:
        return "logits must be [tokens, experts] in fp32 or bf16"
    T, E = logits.shape
    if T * n_expts_act > MAX_ROWS or E > MAX_EXPERTS or n_expts_act > min(E, 32):
        return "more routed rows or experts than the single launch handles"
    for w, pc in ((w1, pc1), (w2, pc2)):
        if not (isinstance(w, Tensor) and isinstance(w.storage.layout, GFX950MXValueLayout) and w.dtype == FP4):
            return "weights must be MXFP4 in the tiled layout"
        s = pc.b_mx_scale if pc is not None else None
        if not (isinstance(s, Tensor) and isinstance(s.storage.layout, GFX950MXScaleLayout)):
            return "weight scales must be in the tiled layout"
        if pc.a_mx_scale is not None or pc.a_mx_tensor_scale is not None or pc.b_mx_tensor_scale is not None or pc.c_mx_scale is not None:
            return "only MX weight scales are supported"
        if not _flex_out_is_trivial(pc.flex_ctx) or pc.flex_ctx.lhs_data.scale is not None or pc.flex_ctx.rhs_data.scale is not None:
            return "flexpoint scales are not supported"
        if pc.out_dtype not in (None, torch.bfloat16):
            return "outputs are bf16"
    if _swiglu_args(act) is None:
        return "the first GEMM's fused activation must be swiglu"
    d_model, n1 = w1.shape[-2:]
    d_ff, n2 = w2.shape[-2:]
    if w1.shape[0] != E or w2.shape[0] != E or x.shape[1] != d_model or n1 != 2 * d_ff or n2 != d_model:
        return "weight shapes do not form an FFN over these activations"
    if d_model > MAX_DIM or d_ff > MAX_DIM or d_model % 8 or d_ff % 8:
        return "d_model and d_ff must be multiples of 8 up to 3072"
    # (the kernel reads the rows of x through a 32-bit buffer resource, 16 bytes at a time)
    if T and (x.stride(1) != 1 or x.stride(0) < d_model or x.stride(0) % 8 or x.data_ptr() % 16
              or ((T - 1) * x.stride(0) + d_model) * 2 > 0x7FFFFFFF):
        return "activation rows must be contiguous, 16-byte aligned, non-overlapping and within 2 GiB"
    for b, n in ((b1, n1), (b2, n2)):
        if b is not None and not (b.ndim == 2 and b.shape == (E, n) and b.stride(-1) == 1 and b.dtype in (torch.float32, torch.bfloat16)):
            return "biases must be [experts, N] in fp32 or bf16"
    return None


def moe_decode_layer(x, logits, n_expts_act, w1, b1, w2, b2, pc1: PrecisionConfig, pc2: PrecisionConfig,
                     fused_activation: FusedActivation, *, apply_softmax: bool = True, out=None, return_routing: bool = False):
    """The layer in one launch; raises NotImplementedError when `one_launch_reason` names an obstacle."""
    why = one_launch_reason(x, logits, n_expts_act, w1, b1, w2, b2, pc1, pc2, fused_activation)
    if why is not None:
        raise NotImplementedError(f"moe_decode_layer: {why}")
    T, E = logits.shape
    k = n_expts_act
    d_model, n1 = w1.shape[-2:]
    d_ff = n1 // 2
    alpha, limit, has_limit = _swiglu_args(fused_activation)
    if x.stride(-1) != 1:
        x = x.contiguous()
    if logits.stride(-1) != 1:
        logits = logits.contiguous()
    if out is None:
        out = torch.empty((T, d_model), dtype=torch.bfloat16, device=x.device)
    else:
        assert out.shape == (T, d_model) and out.dtype == torch.bfloat16 and out.stride(-1) == 1
    if T == 0:
        return (out, None, None) if return_routing else out
    ws = _workspace(x.device, T, k, E, d_ff, d_model)
    d = nt.DecodeLayerDesc()
    d.x, d.x_stride_m = x.data_ptr(), x.stride(0)
    d.logits, d.logits_dtype, d.logits_stride_m = logits.data_ptr(), nt.TORCH_TO_TK[logits.dtype], logits.stride(0)
    d.n_tokens, d.n_experts, d.k, d.apply_softmax = T, E, k, int(apply_softmax)
    d.d_model, d.d_ff = d_model, d_ff
    keep = []
    for name, w, pc, b in (("1", w1, pc1, b1), ("2", w2, pc2, b2)):
        wd, sd = w.storage.data, pc.b_mx_scale.storage.data
        assert wd.is_contiguous() and sd.is_contiguous() and wd.dtype == torch.uint8 and sd.dtype == torch.uint8
        setattr(d, "w" + name, wd.data_ptr())
        setattr(d, f"w{name}_mx_scale", sd.data_ptr())
        setattr(d, f"w{name}_stride_e", wd.stride(0))
        setattr(d, f"w{name}s_stride_e", sd.stride(0))
        if b is not None:
            setattr(d, "b" + name, b.data_ptr())
            setattr(d, f"b{name}_dtype", nt.TORCH_TO_TK[b.dtype])
            setattr(d, f"b{name}_stride_e", b.stride(0))
        keep += [wd, sd, b]
    d.act_alpha, d.act_limit, d.act_has_limit = alpha, limit, has_limit
    d.out, d.out_stride_m = out.data_ptr(), out.stride(0)
    indx = vals = None
    if return_routing:
        indx = torch.empty((T, k), dtype=torch.int16, device=x.device)
        vals = torch.empty((T, k), dtype=torch.float32, device=x.device)
        d.indx_out, d.vals_out = indx.data_ptr(), vals.data_ptr()
    d.workspace = ws.data_ptr()
    with nt.on_device(x.device):
        nt.check(nt.lib().tk_moe_decode_layer(d, nt.stream_ptr(x.device)), "tk_moe_decode_layer")
    del keep
    return (out, indx, vals) if return_routing else out


def moe_mlp(x, logits, n_expts_act, w1, b1, w2, b2, pc1: PrecisionConfig, pc2: PrecisionConfig,
            fused_activation: FusedActivation):
    """`routing` + gather-`matmul_ogs` (+ fused activation) + scatter-`matmul_ogs` (gate weighted, k rows summed) as one
    call: one kernel launch at decode sizes, the three calls otherwise.  Returns `[tokens, d_model]`."""
    # (with fewer than 8 routed rows the launch's fixed part, every workgroup routing the batch before its first weight
    # byte, outweighs the two launch boundaries it saves: 41 against 29 us for one token at the gpt-oss shape)
    if logits.shape[0] * n_expts_act >= MIN_ROWS and one_launch_reason(x, logits, n_expts_act, w1, b1, w2, b2, pc1, pc2, fused_activation) is None:
        return moe_decode_layer(x, logits, n_expts_act, w1, b1, w2, b2, pc1, pc2, fused_activation)
    from .legacy import matmul_ogs, routing
    rdata, gather, scatter = routing(logits, n_expts_act)
    h = matmul_ogs(x, w1, b1, rdata, gather_indx=gather, precision_config=pc1, fused_activation=fused_activation)
    return matmul_ogs(h, w2, b2, rdata, scatter_indx=scatter, precision_config=pc2, gammas=rdata.gate_scal)
