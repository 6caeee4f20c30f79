"""CPU oracle: ragged expert GEMM, swiglu, k-way combine and the whole MoE FFN layer.

Test infrastructure only.  Follows
  * `apply_precision` + `matmul_torch`   python/triton_kernels/triton_kernels/matmul.py:772-931
  * `swiglu_torch`                       .../swiglu.py:89-100   (evaluated in fp32 as the kernel does,
                                         .../swiglu_details/_swiglu.py:55-64)
  * `reduce_torch`                       .../reduce.py:1181-1214 (sum over `dim` in fp32, cast back)
  * layer composition                    python/triton_kernels/tests/test_distributed.py:203-220 and
                                         python/triton_kernels/bench/bench_mlp.py:60-96
"""
from __future__ import annotations

import torch

from . import mxfp as _mx
from . import routing as _rt


def dequant_weight(w: torch.Tensor, w_mx_scale: torch.Tensor | None, w_col_scale: torch.Tensor | None = None):
    """Weights as the GEMM oracle multiplies them.

    MX weights are dequantised to bf16 along K = dim -2 (matmul.py:799-811); plain weights are
    used as stored (matmul.py:776-779).  `w_col_scale [E, N]` is the per-output-channel fp32
    scale of the fp8 configuration, applied in fp32 (not pinned by the reference).
    """
    if w_mx_scale is not None:
        w = _mx.upcast_from_mxfp(w, w_mx_scale, torch.bfloat16, axis=w.ndim - 2)
    w = w.to("cpu")
    if w_col_scale is not None:
        w = w.to(torch.float32) * w_col_scale.to("cpu").to(torch.float32)[:, None, :]
    return w


def matmul(x, w, bias, slice_sizes=None, gather_indx=None, scatter_indx=None, gammas=None, betas=None,
           w_mx_scale=None, x_row_scale=None, w_col_scale=None, out_dtype=None, out_alpha=None, acc_in=None):
    """Y[dst(r)] = cast(((X[src(r)] @ W[e(r)]) + bias[e(r)]*beta_r) * out_alpha * gamma_r + acc_in[r])   (matmul.py:840-931).

    `out_alpha` and `acc_in` are not arguments of the reference's torch twin; they follow its kernel's epilogue
    (matmul_details/_matmul.py:547-559: `acc = acc + bias * betas; acc *= out_alpha; out = act(acc); out *= gammas`,
    and :581-591: `out += load(OutAcc)`), and are pinned against a float64 closed form in tests/test_oracle_moe.py.

    `x [M,K]`; `w [E,K,N]` (or `[K,N]`); `slice_sizes [E]` rows per expert in sorted order (None: one
    slice covering every row); accumulation in fp32 via `torch.matmul`; the result is rounded to
    `out_dtype` (default: x's dtype, matmul.py:913-917) before the scatter; rows not written by the
    scatter are zero (matmul.py:923-927).
    """
    x = x.detach().to("cpu")
    w = dequant_weight(w, w_mx_scale, w_col_scale)
    if w.ndim == 2:
        w = w[None]
    out_dtype = out_dtype or (x.dtype if x.dtype.itemsize > 1 else torch.bfloat16)
    xf = x.to(torch.float32)
    if x_row_scale is not None:
        xf = xf * x_row_scale.to("cpu").to(torch.float32)[:, None]
    n_rows = x.shape[0] if gather_indx is None else gather_indx.shape[0]
    if slice_sizes is None:
        bounds = [(0, n_rows)] * w.shape[0]
        assert w.shape[0] == 1
    else:
        sizes = slice_sizes.detach().to("cpu").to(torch.int64)
        off = torch.zeros(sizes.shape[0] + 1, dtype=torch.int64)
        off[1:] = torch.cumsum(sizes, 0)
        bounds = [(int(off[i]), int(off[i + 1])) for i in range(sizes.shape[0])]
    N = w.shape[-1]
    y = torch.zeros((n_rows, N), dtype=out_dtype)
    gi = None if gather_indx is None else gather_indx.detach().to("cpu").to(torch.int64)
    for e, (lo, hi) in enumerate(bounds):
        if hi <= lo:
            continue
        idx = torch.arange(lo, hi) if gi is None else gi[lo:hi]
        acc = torch.matmul(xf[idx, :], w[e].to(torch.float32))
        if bias is not None:
            b = bias.detach().to("cpu").to(torch.float32)
            b = b[e] if b.ndim == 2 else b
            acc += b if betas is None else b[None, :] * betas.to("cpu").to(torch.float32)[lo:hi, None]
        if out_alpha is not None:
            acc *= float(out_alpha)
        if gammas is not None:
            acc *= gammas.detach().to("cpu").to(torch.float32)[lo:hi, None]
        if acc_in is not None:
            assert scatter_indx is None  # matmul.py:531
            acc += acc_in.detach().to("cpu").to(torch.float32)[lo:hi, :]
        y[lo:hi, :] = acc.to(out_dtype)
    if scatter_indx is None:
        return y
    si = scatter_indx.detach().to("cpu").to(torch.int64)
    out = torch.zeros((si.shape[0], N), dtype=out_dtype)
    msk = si != -1
    out[si[msk], :] = y[msk, :]
    return out


def matmul_ragged_k(a, b, sizes, a_offs, b_offs, out_dtype=None):
    """out[e] = a[:, a_offs[e] : a_offs[e] + sizes[e]] @ b[b_offs[e] : b_offs[e] + sizes[e], :]   (matmul.py:852-875).

    The reduction dimension is the ragged one: `a [M, Ka]`, `b [Kb, N]`, one `[M, N]` result per slice, zero for an
    empty slice (matmul.py:860-861).  Each slice is an ordinary fp32-accumulated matmul (matmul.py:865-871 recurses
    into the dense case without bias or scales); the reference collects the slices in an fp32 tensor, the kernel's
    output type is `out_dtype` (default a's).
    """
    a = a.detach().to("cpu")
    b = b.detach().to("cpu")
    sizes = [int(v) for v in sizes.detach().to("cpu")]
    a_offs = [int(v) for v in a_offs.detach().to("cpu")]
    b_offs = [int(v) for v in b_offs.detach().to("cpu")]
    out_dtype = out_dtype or a.dtype
    out = torch.zeros((len(sizes), a.shape[0], b.shape[1]), dtype=out_dtype)
    for e, k in enumerate(sizes):
        if k == 0:
            continue
        xs = a[:, a_offs[e]:a_offs[e] + k].to(torch.float32)
        ws = b[b_offs[e]:b_offs[e] + k, :].to(torch.float32)
        out[e] = torch.matmul(xs, ws).to(out_dtype)
    return out


def swiglu(a: torch.Tensor, alpha: float, limit: float | None, out_dtype=None):
    """Interleaved (gate, linear) columns -> s*(linear+1), s = g*sigmoid(alpha*g)   (swiglu.py:89-100)."""
    a = a.detach().to("cpu")
    out_dtype = out_dtype or a.dtype
    af = a.to(torch.float32)
    g = af[..., ::2]
    l = af[..., 1::2]
    if limit is not None:
        g = g.clamp(max=limit)
        l = l.clamp(min=-limit, max=limit)
    s = g * torch.sigmoid(alpha * g)
    return (s * (l + 1)).to(out_dtype)


def reduce_k(y: torch.Tensor, k: int, mask: torch.Tensor | None = None):
    """`[T*k, d] -> [T, d]`: sum of each token's k rows in fp32, cast back (reduce.py:1196-1203)."""
    y = y.detach().to("cpu")
    v = y.view(y.shape[0] // k, k, y.shape[-1]).to(torch.float32)
    if mask is not None:
        v = torch.where(mask.to("cpu").to(torch.bool), v, torch.zeros_like(v))
    return v.sum(dim=1).to(y.dtype)


def quantize_fp8_rowwise(x: torch.Tensor):
    """Per-row dynamic e4m3 quantisation: `s = amax/448`, `q = sat_cast(x / s)`.

    PARITY UNPINNED by the reference (no reference function computes it); follows the
    saturating-cast note of mxfp.py:293-296.  An all-zero row gets scale 1 so it dequantises to 0.
    """
    xf = x.detach().to("cpu").to(torch.float32)
    amax = xf.abs().amax(dim=-1)
    s = amax / 448.0
    s = torch.where(s == 0, torch.ones_like(s), s)
    q = (xf / s[:, None]).clamp(-448.0, 448.0).to(torch.float8_e4m3fn)
    return q, s


def moe_layer(x, logits, k, w1, b1, w2, b2, swiglu_alpha=1.702, swiglu_limit=7.0, w1_mx_scale=None,
              w2_mx_scale=None, w1_col_scale=None, w2_col_scale=None, fp8_activations=False,
              return_intermediates=False):
    """router -> gather-GEMM(+bias) -> swiglu -> scatter-GEMM(+bias, *gate) -> k-way sum.

    Intermediates are rounded to bf16 exactly where the reference materialises them: `h` after the
    first GEMM's epilogue (before swiglu, tests/test_matmul.py:622-623), the swiglu output, the
    k-expanded `y`, and the combined output.
    """
    r = _rt.routing(logits, k, apply_softmax=True)
    sizes = r.meta.col_sum
    if fp8_activations:
        xq, sx = quantize_fp8_rowwise(x)
        h = matmul(xq, w1, b1, sizes, gather_indx=r.gather_indx, x_row_scale=sx, w_col_scale=w1_col_scale,
                   out_dtype=torch.bfloat16)
    else:
        h = matmul(x, w1, b1, sizes, gather_indx=r.gather_indx, w_mx_scale=w1_mx_scale, w_col_scale=w1_col_scale)
    a = swiglu(h, swiglu_alpha, swiglu_limit)
    if fp8_activations:
        aq, sa = quantize_fp8_rowwise(a)
        y = matmul(aq, w2, b2, sizes, scatter_indx=r.scatter_indx, gammas=r.gammas, x_row_scale=sa,
                   w_col_scale=w2_col_scale, out_dtype=torch.bfloat16)
    else:
        y = matmul(a, w2, b2, sizes, scatter_indx=r.scatter_indx, gammas=r.gammas, w_mx_scale=w2_mx_scale,
                   w_col_scale=w2_col_scale)
    out = reduce_k(y, k)
    if return_intermediates:
        return out, dict(routing=r, h=h, a=a, y=y)
    return out
