"""Seeded random problems through `matmul` with DEFAULT tile selection (the other GPU suites force `block_m`): random
slice counts and sizes (empty, tiny and large slices mixed), K and N that are not multiples of the tile, random
gather / scatter / gate weights / fused swiglu, outputs pre-filled with NaN so that a row nobody wrote cannot pass.
Tiled MXFP4 weights with bf16 activations (prefill and decode kernels, the fused top-k combine through `matmul_ogs`),
tiled e4m3 weights, strided bf16 weights.  Checked against the CPU oracle with the stated gate."""
import pytest
import torch

from oracle import moe as omoe
from oracle import mxfp as omx
from oracle.checks import assert_allclose_gate, assert_close

pytestmark = pytest.mark.gpu


def _random_sizes(g, n_slices, total):
    """Slice sizes summing to `total`: a few large slices, many small ones, some empty."""
    w = torch.rand(n_slices, generator=g) ** 3
    w[torch.rand(n_slices, generator=g) < 0.25] = 0
    if w.sum() == 0:
        w[0] = 1
    sizes = torch.floor(w / w.sum() * total).to(torch.int64)
    sizes[int(torch.argmax(w))] += total - int(sizes.sum())
    return sizes.to(torch.int32)


@pytest.mark.parametrize("seed", list(range(40)) + [100 + i for i in range(9)])
def test_random_ragged_problem(device, seed):
    import triton_amd.matmul as mm
    import triton_amd.tensor as tensor
    from triton_amd.swiglu import swiglu_fn
    from triton_amd.tensor import FP4, convert_layout, wrap_torch_tensor
    from triton_amd.tensor_details.layout import (make_default_matmul_fp8_w_layout, make_default_matmul_mxfp4_w_layout,
                                                 make_default_matmul_mxfp4_w_scale_layout)
    g = torch.Generator().manual_seed(1000 + seed)
    ri = lambda lo, hi: int(torch.randint(lo, hi + 1, (1, ), generator=g))
    kind = ("mxfp4_tiled", "fp8_tiled", "bf16")[seed % 3]
    E = ri(1, 12)
    m = (ri(1, 40), ri(41, 700), ri(701, 3000))[ri(0, 2)]
    k = 32 * ri(4, 24)                       # 128 .. 768, not always a multiple of the K-stage
    swiglu = bool(ri(0, 1))
    n = (16 if swiglu else 8) * ri(2, 80)    # up to 640 (1280 with swiglu), rarely a multiple of the tile width
    if seed >= 100:  # enough tiles for several rounds of the persistent grids (256 workgroups), around their multiples
        E, m, k = ri(8, 40), ri(12000, 40000), 32 * ri(4, 12)
        n = (16 if swiglu else 8) * ri(100, 200)
    do_gather, do_scatter, do_gamma = bool(ri(0, 1)), bool(ri(0, 1)), bool(ri(0, 1))
    sizes = _random_sizes(g, E, m)
    md = tensor.make_ragged_tensor_metadata(sizes.to(device), m)
    n_src = ri(1, m)
    gi = torch.randint(0, n_src, (m, ), generator=g).to(torch.int32) if do_gather else None
    sc = torch.randperm(m, generator=g).to(torch.int32) if do_scatter else None
    gam = (torch.rand((m, ), generator=g) + 0.5) if do_gamma else None
    bias = torch.randn((E, n), generator=g)
    act = mm.FusedActivation(mm.FnSpecs("swiglu", swiglu_fn, ("alpha", "limit"), reduction_n=2), (1.702, 7.0)) if swiglu else None
    dv = lambda t: None if t is None else t.to(device)
    rows_x = n_src if do_gather else m
    out = torch.full((m, n // 2 if swiglu else n), float("nan"), dtype=torch.bfloat16, device=device)
    if kind == "fp8_tiled":
        x = torch.randn((rows_x, k), generator=g)
        sx = x.abs().amax(dim=1).clamp_min(1e-6) / 448.0
        xq = (x / sx[:, None]).clamp(-448, 448).to(torch.float8_e4m3fn)
        w = torch.randn((E, k, n), generator=g) * 0.05
        sw = w.abs().amax(dim=1) / 448.0
        wq = (w / sw[:, None, :]).clamp(-448, 448).to(torch.float8_e4m3fn)
        wd = convert_layout(wrap_torch_tensor(wq.to(device).transpose(-1, -2).contiguous().transpose(-1, -2)), make_default_matmul_fp8_w_layout())
        pc = mm.PrecisionConfig(a_mx_tensor_scale=sx.to(device), b_mx_tensor_scale=sw.to(device), out_dtype=torch.bfloat16)
        y = mm.matmul(xq.to(device), wd, bias.to(device), md, gather_indx=dv(gi), scatter_indx=dv(sc), gammas=dv(gam), precision_config=pc,
                      fused_activation=act, c=out)
        oracle_args = dict(x=xq, w=wq, x_row_scale=sx, w_col_scale=sw)
    else:
        x = torch.randn((rows_x, k), generator=g).to(torch.bfloat16)
        w = (torch.randn((E, k, n), generator=g) * 0.1).to(torch.bfloat16)
        if kind == "mxfp4_tiled":
            q, s = omx.downcast_to_mxfp(w, torch.uint8, axis=1)
            qd = convert_layout(wrap_torch_tensor(q.to(device), dtype=FP4), make_default_matmul_mxfp4_w_layout(mx_axis=1))
            sd = convert_layout(wrap_torch_tensor(s.to(device)), make_default_matmul_mxfp4_w_scale_layout(mx_axis=1))
            y = mm.matmul(x.to(device), qd, bias.to(device), md, gather_indx=dv(gi), scatter_indx=dv(sc), gammas=dv(gam),
                          precision_config=mm.PrecisionConfig(b_mx_scale=sd), fused_activation=act, c=out)
            oracle_args = dict(x=x, w=q, w_mx_scale=s)
        else:
            y = mm.matmul(x.to(device), w.to(device), bias.to(device), md, gather_indx=dv(gi), scatter_indx=dv(sc), gammas=dv(gam),
                          fused_activation=act, c=out)
            oracle_args = dict(x=x, w=w)
    xo = oracle_args.pop("x")
    wo = oracle_args.pop("w")
    # the oracle applies the gate weight inside matmul; with swiglu the kernel applies it after the activation
    ref = omoe.matmul(xo, wo, bias, sizes, gather_indx=gi, scatter_indx=None if swiglu else sc, gammas=None if swiglu else gam,
                      out_dtype=torch.float32 if swiglu else torch.bfloat16, **oracle_args)
    if swiglu:
        ref = omoe.swiglu(ref, 1.702, 7.0).float()
        if gam is not None:
            ref = ref * gam[:, None]
        ref = ref.to(torch.bfloat16)
        if sc is not None:
            full = torch.zeros_like(ref)
            full[sc.long()] = ref
            ref = full
    what = f"{kind} E={E} m={m} k={k} n={n} sizes={sizes.tolist()} gather={do_gather} scatter={do_scatter} gamma={do_gamma} swiglu={swiglu}"
    assert y.data_ptr() == out.data_ptr()
    assert not torch.isnan(y).any(), "rows that nothing wrote: " + what
    assert_close(ref, y, maxtol=3e-2 if swiglu else 2e-2, what=what)
    if not swiglu:
        assert_allclose_gate(ref, y, what=what)


@pytest.mark.parametrize("seed", range(12))
def test_random_decode_layer_through_matmul_ogs(device, seed):
    """Decode-sized layers (1 .. 96 tokens) through `routing` + `matmul_ogs` (fused top-k combine inside GEMM2) against
    the oracle's layer, random expert counts, top-k and widths."""
    from triton_amd.legacy import matmul_ogs, routing
    from triton_amd.matmul import FnSpecs, FusedActivation, PrecisionConfig
    from triton_amd.swiglu import swiglu_fn
    from triton_amd.tensor import FP4, convert_layout, wrap_torch_tensor
    from triton_amd.tensor_details.layout import make_default_matmul_mxfp4_w_layout, make_default_matmul_mxfp4_w_scale_layout
    g = torch.Generator().manual_seed(7000 + seed)
    ri = lambda lo, hi: int(torch.randint(lo, hi + 1, (1, ), generator=g))
    T, E, k = ri(1, 96), (8, 16, 32, 64)[ri(0, 3)], (1, 2, 4)[ri(0, 2)]
    d, f2 = 32 * ri(4, 12), 64 * ri(2, 10)
    x = torch.randn((T, d), generator=g).to(torch.bfloat16)
    logits = torch.randn((T, E), generator=g)
    # model-like magnitudes (hidden values of order one): the fused swiglu works on fp32 accumulators while the oracle
    # rounds GEMM1's output to bf16 first, a one-ulp difference per hidden value that large weights would amplify
    w1 = (torch.randn((E, d, f2), generator=g) * 0.05).to(torch.bfloat16)
    w2 = (torch.randn((E, f2 // 2, d), generator=g) * 0.05).to(torch.bfloat16)
    b1, b2 = torch.randn((E, f2), generator=g) * 0.05, torch.randn((E, d), generator=g) * 0.05
    w1q, w1s = omx.downcast_to_mxfp(w1, torch.uint8, axis=1)
    w2q, w2s = omx.downcast_to_mxfp(w2, torch.uint8, axis=1)
    tile = lambda q, s: (convert_layout(wrap_torch_tensor(q.to(device), dtype=FP4), make_default_matmul_mxfp4_w_layout(mx_axis=1)),
                         convert_layout(wrap_torch_tensor(s.to(device)), make_default_matmul_mxfp4_w_scale_layout(mx_axis=1)))
    (w1d, s1d), (w2d, s2d) = tile(w1q, w1s), tile(w2q, w2s)
    act = FusedActivation(FnSpecs("swiglu", swiglu_fn, ("alpha", "limit"), reduction_n=2), (1.702, 7.0))
    rdata, gather, scatter = routing(logits.to(device), k)
    h = matmul_ogs(x.to(device), w1d, b1.to(device), rdata, gather_indx=gather, precision_config=PrecisionConfig(b_mx_scale=s1d),
                   fused_activation=act)
    out = matmul_ogs(h, w2d, b2.to(device), rdata, scatter_indx=scatter, precision_config=PrecisionConfig(b_mx_scale=s2d),
                     gammas=rdata.gate_scal)
    ref = omoe.moe_layer(x, logits, k, w1q, b1, w2q, b2, w1_mx_scale=w1s, w2_mx_scale=w2s)
    what = f"T={T} E={E} k={k} d={d} f2={f2}"
    assert out.shape == ref.shape, what
    assert not torch.isnan(out).any(), what
    # rms bound: the hidden activations pass through bf16 (relative rounding noise 2^-9 rms) on both sides, but the
    # kernel rounds swiglu(fp32) where the oracle rounds the GEMM output first; a handful of tokens does not average
    # that out to the 4e-3 the large layers meet
    assert_close(ref, out, maxtol=3e-2, rmstol=6e-3, what=what)
    assert_allclose_gate(ref, out, max_bad_frac=1e-4, what=what)
