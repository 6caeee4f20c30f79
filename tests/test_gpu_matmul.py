"""GPU parity of the ragged expert GEMM (through the C ABI) against the CPU oracle.

Mirrors the gfx950-relevant slice of python/triton_kernels/tests/test_matmul.py:116-301: bf16 x bf16 and
bf16 x mxfp4, plain and ragged (10 slices, one empty), x {none, gather, scatter, gather+scatter} x gammas,
block_m in {16, 128}, fused swiglu.  Tolerances are the reference's (testing.py:27-88, test_matmul.py:644-653)
and the rtol 2e-2 / atol 1e-2 gate."""
import pytest
import torch

from oracle import moe as omoe
from oracle import mxfp as omx
from oracle import routing as ort
from oracle.checks import assert_allclose_gate, assert_close

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def mods(device):
    import triton_amd.matmul as mm
    import triton_amd.swiglu as sw
    import triton_amd.tensor as tensor
    return mm, sw, tensor


def _slice_sizes(m, n_slices, g):
    cuts = torch.sort(torch.randint(0, m + 1, (n_slices - 1, ), generator=g)).values
    sizes = torch.diff(torch.cat([torch.tensor([0]), cuts, torch.tensor([m])]))
    if n_slices > 2:
        sizes[n_slices // 2 + 1] += sizes[n_slices // 2]  # one empty slice (testing.py:307-311)
        sizes[n_slices // 2] = 0
    return sizes.to(torch.int32)


_W_CACHE = {}


def _make_w(E, K, N, kind, g, device):
    """Expert weights of one (shape, kind), generated from their own seed and kept for the cases that share them
    (quantising them with the CPU oracle is the slow part of a case); `g` is left untouched."""
    key = (E, K, N, kind, str(device))
    if key not in _W_CACHE:
        if len(_W_CACHE) >= 6:
            _W_CACHE.pop(next(iter(_W_CACHE)))
        _W_CACHE[key] = _make_w_uncached(E, K, N, kind, torch.Generator().manual_seed(E * 1000003 + K * 1009 + N), device)
    return _W_CACHE[key]


def _make_w_uncached(E, K, N, kind, g, device):
    w = (torch.randn((E, K, N), generator=g) * 0.5 / K**0.5 * 4).to(torch.bfloat16)
    if kind in ("mxfp4", "mxfp4_tiled"):
        q, s = omx.downcast_to_mxfp(w, torch.uint8, axis=1)
        qd, sd = q.to(device), s.to(device)
        if kind == "mxfp4_tiled":  # the pre-tiled layouts, converted as the reference converts its weight layouts
            from triton_amd.tensor import FP4, convert_layout, wrap_torch_tensor
            from triton_amd.tensor_details.layout import make_default_matmul_mxfp4_w_layout, make_default_matmul_mxfp4_w_scale_layout
            qd = convert_layout(wrap_torch_tensor(qd, dtype=FP4), make_default_matmul_mxfp4_w_layout(mx_axis=1))
            sd = convert_layout(wrap_torch_tensor(sd), make_default_matmul_mxfp4_w_scale_layout(mx_axis=1))
        return dict(w_dev=qd, scale_dev=sd, w_cpu=q, scale_cpu=s)
    if kind == "bf16_kmajor":
        wd = w.to(device).transpose(-1, -2).contiguous().transpose(-1, -2)
        return dict(w_dev=wd, scale_dev=None, w_cpu=w, scale_cpu=None)
    return dict(w_dev=w.to(device), scale_dev=None, w_cpu=w, scale_cpu=None)


CASES = [
    # m, n, k, mode, wkind
    (16, 256, 256, "ragged", "bf16"),
    (300, 400, 400, "ragged", "bf16_kmajor"),
    (300, 400, 416, "ragged", "mxfp4"),
    (1000, 704, 832, "ragged", "bf16_kmajor"),
    (720, 576, 768, "ragged", "mxfp4"),
    (768, 512, 1024, "ragged", "mxfp4"),
    (720, 576, 768, "plain", "mxfp4"),
    (600, 400, 416, "plain", "bf16"),
    (5, 2880, 2880, "ragged", "mxfp4"),
    (300, 400, 416, "ragged", "mxfp4_tiled"),
    (720, 576, 768, "ragged", "mxfp4_tiled"),
    (1500, 512, 1024, "ragged", "mxfp4_tiled"),
    (720, 576, 768, "plain", "mxfp4_tiled"),
    (5, 2880, 2880, "ragged", "mxfp4_tiled"),
]


@pytest.mark.parametrize("m, n, k, mode, wkind", CASES)
@pytest.mark.parametrize("block_m", [16, 32, 64, 128, 256])
@pytest.mark.parametrize("do_gather, do_scatter", [(False, False), (True, False), (False, True), (True, True)])
@pytest.mark.parametrize("do_gamma", [False, True])
def test_matmul(mods, device, m, n, k, mode, wkind, block_m, do_gather, do_scatter, do_gamma):
    mm, _, tensor = mods
    g = torch.Generator().manual_seed(m * 7 + n * 3 + k + block_m)
    n_slices = 10 if mode == "ragged" else 1
    x = torch.randn((m, k), generator=g).to(torch.bfloat16)
    W = _make_w(n_slices, k, n, wkind, g, device)
    bias = torch.randn((n_slices, n), generator=g)
    sizes = _slice_sizes(m, n_slices, g) if mode == "ragged" else None
    gather = torch.randint(0, m, (m, ), generator=g, dtype=torch.int32) if do_gather else None
    scatter = torch.randperm(m, generator=g).to(torch.int32) if do_scatter else None
    if scatter is not None and m > 20:
        scatter[torch.rand(m, generator=g) < 0.05] = -1
    gammas = 2.0**torch.randint(-5, 0, (m, ), generator=g).float() if do_gamma else None
    md = tensor.make_ragged_tensor_metadata(sizes.to(device), m) if sizes is not None else None
    pc = mm.PrecisionConfig(b_mx_scale=W["scale_dev"])
    dev = lambda t: None if t is None else t.to(device)
    with mm.scoped_opt_flags_constraints({"block_m": block_m}):
        y = mm.matmul(x.to(device), W["w_dev"], dev(bias) if mode == "ragged" else dev(bias[0]), md, gather_indx=dev(gather),
                      scatter_indx=dev(scatter), precision_config=pc, gammas=dev(gammas))
    ref = omoe.matmul(x, W["w_cpu"], bias, sizes, gather_indx=gather, scatter_indx=scatter, gammas=gammas,
                      w_mx_scale=W["scale_cpu"])
    got = y.cpu()
    if scatter is not None:  # rows that no entry writes are undefined in the kernel path, zero in the oracle
        written = torch.zeros(m, dtype=torch.bool)
        written[scatter[scatter >= 0].long()] = True
        got = torch.where(written[:, None], got, torch.zeros_like(got))
    assert_close(ref, got, maxtol=3e-2 if wkind.startswith("mxfp4") else 2e-2, what="y")
    assert_allclose_gate(ref, got, what="y")


@pytest.mark.parametrize("wkind", ["bf16", "bf16_kmajor", "mxfp4", "mxfp4_tiled"])
@pytest.mark.parametrize("block_m", [16, 128])
@pytest.mark.parametrize("do_gather, swiglu", [(False, False), (True, False), (False, True)])
def test_betas_out_alpha_c_acc_in(mods, device, wkind, block_m, do_gather, swiglu):
    """`betas` (per-row multiplier of the bias), `out_alpha` and `c_acc_in` of the reference's signature
    (triton_kernels/matmul.py:251-258) in its epilogue order (matmul_details/_matmul.py:547-559,581-591):
    y = act((x @ w + bias * beta) * alpha) * gamma + c_acc_in."""
    mm, sw, tensor = mods
    g = torch.Generator().manual_seed(77 + block_m)
    m, n, k, n_slices = 300, 400, 416, 10
    x = torch.randn((m, k), generator=g).to(torch.bfloat16)
    W = _make_w(n_slices, k, n, wkind, g, device)
    bias = torch.randn((n_slices, n), generator=g)
    sizes = _slice_sizes(m, n_slices, g)
    gather = torch.randint(0, m, (m, ), generator=g, dtype=torch.int32) if do_gather else None
    betas = torch.rand((m, ), generator=g) + 0.5
    gammas = 2.0**torch.randint(-3, 0, (m, ), generator=g).float()
    n_out = n // 2 if swiglu else n
    acc_in = torch.randn((m, n_out), generator=g).to(torch.bfloat16)
    alpha = 0.75
    md = tensor.make_ragged_tensor_metadata(sizes.to(device), m)
    act = mm.FusedActivation(mm.FnSpecs("swiglu", sw.swiglu_fn, ("alpha", "limit"), reduction_n=2), (1.702, 7.0)) if swiglu else None
    dev = lambda t: None if t is None else t.to(device)
    with mm.scoped_opt_flags_constraints({"block_m": block_m}):
        y = mm.matmul(x.to(device), W["w_dev"], dev(bias), md, gather_indx=dev(gather), precision_config=mm.PrecisionConfig(b_mx_scale=W["scale_dev"]),
                      betas=dev(betas), gammas=dev(gammas), out_alpha=alpha, c_acc_in=dev(acc_in), fused_activation=act)
    if swiglu:  # the activation sits between out_alpha and the gate weight
        pre = omoe.matmul(x, W["w_cpu"], bias, sizes, gather_indx=gather, betas=betas, out_alpha=alpha, w_mx_scale=W["scale_cpu"], out_dtype=torch.float32)
        ref = (omoe.swiglu(pre, 1.702, 7.0, out_dtype=torch.float32) * gammas[:, None] + acc_in.float()).to(torch.bfloat16)
    else:
        ref = omoe.matmul(x, W["w_cpu"], bias, sizes, gather_indx=gather, gammas=gammas, betas=betas, out_alpha=alpha, acc_in=acc_in,
                          w_mx_scale=W["scale_cpu"])
    assert_close(ref, y.cpu(), maxtol=3e-2, what="y with betas / out_alpha / c_acc_in")
    assert_allclose_gate(ref, y.cpu(), what="y with betas / out_alpha / c_acc_in")


@pytest.mark.parametrize("block_m", [16, 128, 256])
@pytest.mark.parametrize("swiglu", [False, True])
def test_output_given_as_a_column_slice_keeps_its_neighbours(mods, device, block_m, swiglu):
    """`c` handed in as a column slice of a wider tensor, with a column count that is not a multiple of 8: the prefill
    kernels for tiled MXFP4 weights write whole 16-byte pieces, so the host must not let them run over the slice's
    last column into memory that belongs to the caller."""
    mm, sw, tensor = mods
    g = torch.Generator().manual_seed(11 + block_m)
    m, n, k, n_slices = 300, 396 if not swiglu else 792, 416, 10  # N_out = 396: 396 % 8 == 4
    x = torch.randn((m, k), generator=g).to(torch.bfloat16)
    W = _make_w(n_slices, k, n, "mxfp4_tiled", g, device)
    sizes = _slice_sizes(m, n_slices, g)
    md = tensor.make_ragged_tensor_metadata(sizes.to(device), m)
    n_out = n // 2 if swiglu else n
    wide = torch.full((m, n_out + 20), float("nan"), dtype=torch.bfloat16, device=device)
    c = wide[:, :n_out]
    act = mm.FusedActivation(mm.FnSpecs("swiglu", sw.swiglu_fn, ("alpha", "limit"), reduction_n=2), (1.702, 7.0)) if swiglu else None
    with mm.scoped_opt_flags_constraints({"block_m": block_m}):
        y = mm.matmul(x.to(device), W["w_dev"], None, md, precision_config=mm.PrecisionConfig(b_mx_scale=W["scale_dev"]), c=c,
                      fused_activation=act)
    assert y.data_ptr() == c.data_ptr()
    assert bool(torch.isnan(wide[:, n_out:]).all()), "columns next to the output slice were overwritten"
    assert not bool(torch.isnan(wide[:, :n_out]).any())
    ref = omoe.matmul(x, W["w_cpu"], None, sizes, w_mx_scale=W["scale_cpu"])
    if swiglu:
        ref = omoe.swiglu(ref, 1.702, 7.0)
    assert_close(ref, wide[:, :n_out].cpu(), maxtol=3e-2, what="y in a slice")


@pytest.mark.parametrize("m, n, k, mode", [(16, 256, 256, "ragged"), (300, 400, 416, "ragged"), (1000, 704, 832, "ragged"),
                                           (600, 400, 416, "plain"), (5, 2880, 2880, "ragged")])
@pytest.mark.parametrize("block_m", [16, 32, 64, 128])
@pytest.mark.parametrize("k_major", [False, True])
@pytest.mark.parametrize("do_gather, do_scatter, do_gamma, swiglu", [(False, False, False, False), (True, False, False, True),
                                                                     (False, True, True, False), (True, True, False, False)])
def test_matmul_fp16(mods, device, m, n, k, mode, block_m, k_major, do_gather, do_scatter, do_gamma, swiglu):
    """fp16 x fp16 -> fp16 (the reference's test_matmul.py float16 cases): the bf16 kernel with the fp16 MFMA and an
    fp16 epilogue."""
    mm, sw, tensor = mods
    g = torch.Generator().manual_seed(m * 7 + n * 3 + k + block_m + 17 * k_major)
    n_slices = 10 if mode == "ragged" else 1
    x = torch.randn((m, k), generator=g).to(torch.float16)
    w = (torch.randn((n_slices, k, n), generator=g) * 2 / k**0.5).to(torch.float16)
    wd = w.to(device)
    if k_major:
        wd = wd.transpose(-1, -2).contiguous().transpose(-1, -2)
    bias = torch.randn((n_slices, n), generator=g)
    sizes = _slice_sizes(m, n_slices, g) if mode == "ragged" else None
    gather = torch.randint(0, m, (m, ), generator=g, dtype=torch.int32) if do_gather else None
    scatter = torch.randperm(m, generator=g).to(torch.int32) if do_scatter else None
    gammas = 2.0**torch.randint(-5, 0, (m, ), generator=g).float() if do_gamma else None
    md = tensor.make_ragged_tensor_metadata(sizes.to(device), m) if sizes is not None else None
    dev = lambda t: None if t is None else t.to(device)
    act = mm.FusedActivation(mm.FnSpecs("swiglu", sw.swiglu_fn, ("alpha", "limit"), reduction_n=2), (1.702, 7.0)) if swiglu else None
    kw = dict(fused_activation=act) if swiglu else {}
    with mm.scoped_opt_flags_constraints({"block_m": block_m}):
        y = mm.matmul(x.to(device), wd, dev(bias) if mode == "ragged" else dev(bias[0]), md, gather_indx=dev(gather),
                      scatter_indx=dev(scatter), gammas=dev(gammas), **kw)
    assert y.dtype == torch.float16
    if swiglu:
        h = omoe.matmul(x, w, bias, sizes, gather_indx=gather, out_dtype=torch.float32)
        ref = omoe.swiglu(h, 1.702, 7.0, out_dtype=torch.float32)
        if gammas is not None:
            ref = ref * gammas[:, None]
        ref = ref.to(torch.float16)
    else:
        ref = omoe.matmul(x, w, bias, sizes, gather_indx=gather, scatter_indx=scatter, gammas=gammas)
    assert ref.dtype == torch.float16
    assert_close(ref, y.cpu(), maxtol=2e-2, what="y")
    assert_allclose_gate(ref, y.cpu(), what="y")


_NARROW = {"e4m3": torch.float8_e4m3fn, "e5m2": torch.float8_e5m2, "mxfp8_e4m3": torch.float8_e4m3fn,
           "mxfp8_e5m2": torch.float8_e5m2, "mxfp4": torch.uint8}


def _operand(t, kind, axis):
    """(values, scales or None, what the operand means as a 16-bit tensor) for an operand kind of the reference's test
    matrix (test_matmul.py:116-250)."""
    if kind in ("bf16", "fp16"):
        v = t.to(torch.bfloat16 if kind == "bf16" else torch.float16)
        return v, None, v
    if kind.startswith("mx"):
        q, sc = omx.downcast_to_mxfp(t.to(torch.bfloat16), _NARROW[kind], axis=axis)
        return q, sc, omx.upcast_from_mxfp(q, sc, torch.bfloat16, axis=axis)
    q = t.to(_NARROW[kind])
    return q, None, q.to(torch.bfloat16)


@pytest.mark.parametrize("m, n, k, mode, akind, wkind, tiled", [
    (300, 400, 416, "ragged", "bf16", "mxfp8_e4m3", False),
    (300, 400, 416, "ragged", "bf16", "mxfp8_e5m2", False),
    (300, 400, 832, "ragged", "e5m2", "mxfp4", False),
    (300, 400, 832, "ragged", "e5m2", "mxfp4", True),
    (16, 256, 256, "ragged", "e5m2", "mxfp4", True),
    (1024, 1024, 1024, "ragged", "e5m2", "mxfp4", True),
    (300, 400, 416, "ragged", "e5m2", "mxfp8_e4m3", False),
    (300, 400, 416, "ragged", "e5m2", "e5m2", False),
    (600, 400, 416, "plain", "e5m2", "e5m2", False),
    (300, 400, 416, "ragged", "e4m3", "mxfp4", False),
    (300, 400, 416, "ragged", "mxfp8_e4m3", "mxfp8_e4m3", False),
    (300, 400, 416, "ragged", "mxfp8_e5m2", "mxfp4", True),
    (300, 400, 416, "ragged", "mxfp8_e4m3", "mxfp4", False),
    (64, 128, 96, "ragged", "mxfp8_e4m3", "bf16", False),
    (64, 128, 96, "ragged", "mxfp8_e4m3", "fp16", False),
    (64, 128, 96, "ragged", "mxfp4", "bf16", False),
    (64, 128, 96, "ragged", "mxfp4", "fp16", False),
    (256, 256, 256, "plain", "mxfp4", "mxfp4", False),
    (256, 256, 256, "plain", "mxfp4", "mxfp4", True),
])
@pytest.mark.parametrize("block_m", [16, 128])
@pytest.mark.parametrize("do_gather, do_scatter, do_gamma", [(False, False, False), (True, True, True)])
def test_expanded_operand_pairs(mods, device, m, n, k, mode, akind, wkind, tiled, block_m, do_gather, do_scatter, do_gamma):
    """Operand pairs of the reference's matrix that run on the 16-bit kernels after the MX dequantiser has expanded the
    narrow side; the oracle multiplies the same dequantised operands."""
    mm, _, tensor = mods
    g = torch.Generator().manual_seed(m + 3 * n + 7 * k + len(akind) * 11 + len(wkind))
    n_slices = 10 if mode == "ragged" else 1
    xv, xs, x_ref = _operand(torch.randn((m, k), generator=g), akind, -1)
    wv, ws, w_ref = _operand(torch.randn((n_slices, k, n), generator=g) * 2 / k**0.5, wkind, 1)
    if akind == "fp16" or wkind == "fp16":
        x_ref, w_ref = x_ref.to(torch.float16), w_ref.to(torch.float16)
    bias = torch.randn((n_slices, n), generator=g)
    sizes = _slice_sizes(m, n_slices, g) if mode == "ragged" else None
    gather = torch.randint(0, m, (m, ), generator=g, dtype=torch.int32) if do_gather else None
    scatter = torch.randperm(m, generator=g).to(torch.int32) if do_scatter else None
    gammas = 2.0**torch.randint(-5, 0, (m, ), generator=g).float() if do_gamma else None
    md = tensor.make_ragged_tensor_metadata(sizes.to(device), m) if sizes is not None else None
    dev = lambda t: None if t is None else t.to(device)
    wd, wsd = dev(wv), dev(ws)
    if wkind == "mxfp4":
        wd = tensor.wrap_torch_tensor(wd, dtype=tensor.FP4)
        if tiled:
            from triton_amd.tensor_details.layout import make_default_matmul_mxfp4_w_layout, make_default_matmul_mxfp4_w_scale_layout
            wd = tensor.convert_layout(wd, make_default_matmul_mxfp4_w_layout(mx_axis=1))
            wsd = tensor.convert_layout(tensor.wrap_torch_tensor(wsd), make_default_matmul_mxfp4_w_scale_layout(mx_axis=1))
    xd = dev(xv)
    if akind == "mxfp4":
        xd = tensor.wrap_torch_tensor(xd, dtype=tensor.FP4)
    pc = mm.PrecisionConfig(a_mx_scale=dev(xs), b_mx_scale=wsd)
    with mm.scoped_opt_flags_constraints({"block_m": block_m}):
        y = mm.matmul(xd, wd, dev(bias) if mode == "ragged" else dev(bias[0]), md, gather_indx=dev(gather),
                      scatter_indx=dev(scatter), precision_config=pc, gammas=dev(gammas))
    assert y.dtype == x_ref.dtype
    ref = omoe.matmul(x_ref, w_ref, bias, sizes, gather_indx=gather, scatter_indx=scatter, gammas=gammas)
    assert_close(ref, y.cpu(), maxtol=3e-2 if wkind == "mxfp4" else 2e-2, what="y")
    assert_allclose_gate(ref, y.cpu(), what="y")


@pytest.mark.parametrize("m, n, k, wkind", [(300, 512, 416, "bf16_kmajor"), (720, 576, 768, "mxfp4"), (40, 5760, 2880, "mxfp4"),
                                            (720, 576, 768, "mxfp4_tiled"), (900, 5760, 2880, "mxfp4_tiled")])
@pytest.mark.parametrize("block_m", [16, 32, 64, 128])
@pytest.mark.parametrize("opts", [(1.1, 1.4), (1.702, 7.0), (0.5, None)])
def test_fused_swiglu(mods, device, m, n, k, wkind, block_m, opts):
    mm, sw, tensor = mods
    g = torch.Generator().manual_seed(m + n + k)
    n_slices = 6
    x = torch.randn((m, k), generator=g).to(torch.bfloat16)
    W = _make_w(n_slices, k, n, wkind, g, device)
    bias = torch.randn((n_slices, n), generator=g)
    sizes = _slice_sizes(m, n_slices, g)
    md = tensor.make_ragged_tensor_metadata(sizes.to(device), m)
    act = mm.FusedActivation(mm.FnSpecs("swiglu", sw.swiglu_fn, ("alpha", "limit"), reduction_n=2), opts)
    with mm.scoped_opt_flags_constraints({"block_m": block_m}):
        y = mm.matmul(x.to(device), W["w_dev"], bias.to(device), md, precision_config=mm.PrecisionConfig(b_mx_scale=W["scale_dev"]),
                      fused_activation=act)
    h = omoe.matmul(x, W["w_cpu"], bias, sizes, w_mx_scale=W["scale_cpu"])
    ref = omoe.swiglu(h, opts[0], opts[1])
    assert y.shape == (m, n // 2)
    assert_close(ref, y, maxtol=3e-2, what="swiglu(y)")
    # standalone swiglu kernel on the unfused GEMM output
    y2 = mm.matmul(x.to(device), W["w_dev"], bias.to(device), md, precision_config=mm.PrecisionConfig(b_mx_scale=W["scale_dev"]))
    s2 = sw.swiglu(y2, opts[0], sw.PrecisionConfig(opts[1]))
    assert_close(omoe.swiglu(y2.cpu(), opts[0], opts[1]), s2, maxtol=1e-2, what="standalone swiglu")


@pytest.mark.parametrize("kind", ["mxfp8_e4m3", "mxfp8_e5m2", "mxfp4"])
@pytest.mark.parametrize("wkind, swiglu, scatter", [("bf16", False, False), ("mxfp4_tiled", True, False), ("mxfp4", False, True)])
def test_mx_output_epilogue(mods, device, kind, wkind, swiglu, scatter):
    """`Epilogue(FnSpecs(QUANTIZE_MXFP8 | QUANTIZE_MXFP4))` + `c_mx_scale` (reference test: tests/test_matmul.py:560-573,
    checked at :627-643 by dequantising and comparing with maxtol 4e-1 / rmstol 4e-2 against the quantised reference).
    Strided weights run the bf16 GEMM followed by the MX quantiser kernel: (1) the values and scales are bit for bit the
    oracle's quantisation of the GEMM's own bf16 output; (2) dequantised, they meet the reference's tolerance against the
    oracle's GEMM -> quantise -> dequantise.  Tiled MXFP4 weights quantise the fp32 accumulator inside the GEMM and are
    checked against the oracle's fp32 GEMM -> oracle quantiser in `test_bf16_activations_with_fused_mx_output`."""
    mm, sw, tensor = mods
    from triton_amd.numerics_details.mxfp import quantize_mxfp4_fn, quantize_mxfp8_fn
    g = torch.Generator().manual_seed(17)
    m, n, k, n_slices = 300, 512, 416, 6
    x = torch.randn((m, k), generator=g).to(torch.bfloat16)
    W = _make_w(n_slices, k, n, wkind, g, device)
    bias = torch.randn((n_slices, n), generator=g)
    sizes = _slice_sizes(m, n_slices, g)
    md = tensor.make_ragged_tensor_metadata(sizes.to(device), m)
    act = mm.FusedActivation(mm.FnSpecs("swiglu", sw.swiglu_fn, ("alpha", "limit"), reduction_n=2), (1.702, 7.0)) if swiglu else None
    sc = torch.randperm(m, generator=g).to(torch.int32) if scatter else None
    n_out = n // 2 if swiglu else n
    out_dtype = {"mxfp8_e4m3": torch.float8_e4m3fn, "mxfp8_e5m2": torch.float8_e5m2, "mxfp4": torch.uint8}[kind]
    name, fn = (mm.FnName.QUANTIZE_MXFP4.name, quantize_mxfp4_fn) if kind == "mxfp4" else (mm.FnName.QUANTIZE_MXFP8.name, quantize_mxfp8_fn)
    epi = mm.Epilogue(mm.FnSpecs(name, fn, (), ()), tuple(), tuple(), effective_itemsize=6.0)
    c_scale = torch.full((m, n_out // 32), 0xFF, dtype=torch.uint8, device=device)
    kw = dict(fused_activation=act, scatter_indx=None if sc is None else sc.to(device))
    pc = mm.PrecisionConfig(b_mx_scale=W["scale_dev"], c_mx_scale=c_scale, out_dtype=out_dtype)
    yq = mm.matmul(x.to(device), W["w_dev"], bias.to(device), md, precision_config=pc, epilogue=epi, **kw)
    assert yq.dtype == out_dtype and yq.shape == (m, n_out // 2 if kind == "mxfp4" else n_out)
    # the caller's PrecisionConfig is left as it was given (the reference records the pack factor on it, matmul.py:364-369)
    assert pc.c_mx_scale is c_scale and pc.c_value_pack_factor == 1 and pc.c_microblock_size is None
    if wkind != "mxfp4_tiled":
        y = mm.matmul(x.to(device), W["w_dev"], bias.to(device), md, precision_config=mm.PrecisionConfig(b_mx_scale=W["scale_dev"]), **kw)
        q_ref, s_ref = omx.downcast_to_mxfp(y.cpu(), out_dtype, axis=-1)
        assert torch.equal(q_ref.view(torch.uint8), yq.cpu().view(torch.uint8)), "values are not the quantisation of the bf16 result"
        assert torch.equal(s_ref, c_scale.cpu()), "scales are not the quantisation of the bf16 result"
    h = omoe.matmul(x, W["w_cpu"], bias, sizes, w_mx_scale=W["scale_cpu"], scatter_indx=sc)
    if swiglu:
        h = omoe.swiglu(h, 1.702, 7.0)
    ref = omx.upcast_from_mxfp(*omx.downcast_to_mxfp(h, out_dtype, axis=-1), torch.bfloat16, axis=-1)
    got = omx.upcast_from_mxfp(yq.cpu(), c_scale.cpu(), torch.bfloat16, axis=-1)
    if kind == "mxfp4":
        # 3-bit magnitudes: an fp32-vs-bf16 rounding difference next to a decision threshold moves a value by a whole
        # e2m1 step (up to 100 % of a small value), so the max-error bound of the fp8 case does not apply; the
        # reference has no MXFP4-output test.  Bounded by how many elements differ and by the rms error.
        from oracle.checks import rel_errors
        differing = (ref.float() != got.float()).float().mean().item()
        _, rms = rel_errors(ref, got)
        assert differing <= 0.03 and rms <= 1e-1, f"mxfp4 output: {differing:.4f} of the elements differ, rms {rms:.4g}"
    else:
        assert_close(ref, got, maxtol=4e-1, rmstol=4e-2, what="dequantised MX output")


def _fp8_operands(m, n, k, n_slices, g):
    """e4m3 activations with one fp32 scale per row, e4m3 weights with one fp32 scale per (expert, column)."""
    x = torch.randn((m, k), generator=g)
    sx = x.abs().amax(dim=1).clamp_min(1e-6) / 448.0
    xq = (x / sx[:, None]).clamp(-448, 448).to(torch.float8_e4m3fn)
    w = torch.randn((n_slices, k, n), generator=g) * 0.05
    sw = w.abs().amax(dim=1) / 448.0  # [E, N]
    wq = (w / sw[:, None, :]).clamp(-448, 448).to(torch.float8_e4m3fn)
    return xq, sx, wq, sw


@pytest.mark.parametrize("m, n, k", [(300, 400, 416), (1000, 704, 832), (2100, 512, 1024), (64, 96, 16)])
@pytest.mark.parametrize("layout, block_m", [("strided", 16), ("strided", 128), ("tiled", 128), ("tiled", 256)])
@pytest.mark.parametrize("do_gather, do_scatter, do_gamma, swiglu", [(False, False, False, False), (True, False, True, True),
                                                                      (False, True, True, False), (True, True, False, True)])
def test_matmul_fp8(mods, device, m, n, k, layout, block_m, do_gather, do_scatter, do_gamma, swiglu):
    """e4m3 x e4m3 with per-row and per-column fp32 scales (config 5's operands; the reference's hooks:
    matmul.py:620-626, _matmul.py:363-382,507-517).  PARITY UNPINNED by the reference's tests; the oracle
    dequantises both operands and runs the pinned GEMM oracle.  Strided K-contiguous weights and the tiled FP8 layout."""
    mm, sw_mod, tensor = mods
    from triton_amd.tensor import convert_layout, wrap_torch_tensor
    from triton_amd.tensor_details.layout import make_default_matmul_fp8_w_layout
    g = torch.Generator().manual_seed(m * 7 + n + k)
    n_slices = 6
    xq, sx, wq, sw = _fp8_operands(m, n, k, n_slices, g)
    bias = torch.randn((n_slices, n), generator=g)
    sizes = _slice_sizes(m, n_slices, g)
    md = tensor.make_ragged_tensor_metadata(sizes.to(device), m)
    gi = torch.randint(0, m, (m, ), generator=g).to(torch.int32) if do_gather else None
    sc = torch.randperm(m, generator=g).to(torch.int32) if do_scatter else None
    gam = (torch.rand((m, ), generator=g) + 0.5) if do_gamma else None
    wd = wq.to(device).transpose(-1, -2).contiguous().transpose(-1, -2)  # stride 1 along K
    if layout == "tiled":
        wd = convert_layout(wrap_torch_tensor(wd), make_default_matmul_fp8_w_layout())
    act = mm.FusedActivation(mm.FnSpecs("swiglu", sw_mod.swiglu_fn, ("alpha", "limit"), reduction_n=2), (1.702, 7.0)) if swiglu else None
    pc = mm.PrecisionConfig(a_mx_tensor_scale=sx.to(device), b_mx_tensor_scale=sw.to(device), out_dtype=torch.bfloat16)
    dv = lambda t: None if t is None else t.to(device)
    with mm.scoped_opt_flags_constraints({"block_m": block_m}):
        y = mm.matmul(xq.to(device), wd, bias.to(device), md, gather_indx=dv(gi), scatter_indx=dv(sc), gammas=dv(gam),
                      precision_config=pc, fused_activation=act)
    # the oracle applies the gate weight inside matmul; with swiglu the kernel applies it after the activation
    ref = omoe.matmul(xq, wq, bias, sizes, gather_indx=gi, scatter_indx=None if swiglu else sc, gammas=None if swiglu else gam,
                      x_row_scale=sx, w_col_scale=sw, out_dtype=torch.float32 if swiglu else torch.bfloat16)
    if swiglu:
        ref = omoe.swiglu(ref, 1.702, 7.0).float()
        if gam is not None:
            ref = ref * gam[:, None]
        ref = ref.to(torch.bfloat16)
        if sc is not None:
            out = torch.zeros_like(ref)
            out[sc.long()] = ref
            ref = out
    assert y.shape == ref.shape
    assert_close(ref, y, maxtol=3e-2 if swiglu else 2e-2, what="fp8 y")
    assert_allclose_gate(ref, y, what="fp8 y")


@pytest.mark.parametrize("do_gather, do_scatter", [(True, False), (False, True)])
def test_matmul_fp8_long_k_takes_the_wide_tiles(mods, device, monkeypatch, do_gather, do_scatter):
    """With at least 512 rows per slice and K >= 8192 `matmul` picks row blocks of 256 for tiled e4m3 weights (256 x 256
    tiles, every row fragment multiplied): two slices of 700 and 900 rows (partly filled last blocks), K = 8192, against
    the oracle; the descriptor is checked to ask for block_m 256."""
    mm, _, tensor = mods
    from triton_amd import _native as nt
    from triton_amd.tensor import convert_layout, wrap_torch_tensor
    from triton_amd.tensor_details.layout import make_default_matmul_fp8_w_layout
    g = torch.Generator().manual_seed(97)
    m, n, k, n_slices = 1600, 320, 8192, 2
    xq, sx, wq, sw = _fp8_operands(m, n, k, n_slices, g)
    bias = torch.randn((n_slices, n), generator=g)
    sizes = torch.tensor([700, 900], dtype=torch.int32)
    md = tensor.make_ragged_tensor_metadata(sizes.to(device), m)
    gi = torch.randint(0, m, (m, ), generator=g).to(torch.int32) if do_gather else None
    sc = torch.randperm(m, generator=g).to(torch.int32) if do_scatter else None
    wd = convert_layout(wrap_torch_tensor(wq.to(device).transpose(-1, -2).contiguous().transpose(-1, -2)), make_default_matmul_fp8_w_layout())
    pc = mm.PrecisionConfig(a_mx_tensor_scale=sx.to(device), b_mx_tensor_scale=sw.to(device), out_dtype=torch.bfloat16)
    seen = []
    real_lib = nt.lib()

    class Spy:
        def tk_moe_gemm(self, d, stream):
            seen.append(int(d.block_m))
            return real_lib.tk_moe_gemm(d, stream)

        def __getattr__(self, name):
            return getattr(real_lib, name)

    spy = Spy()
    monkeypatch.setattr(mm.nt, "lib", lambda: spy)
    dv = lambda t: None if t is None else t.to(device)
    y = mm.matmul(xq.to(device), wd, bias.to(device), md, gather_indx=dv(gi), scatter_indx=dv(sc), precision_config=pc)
    assert seen == [256], f"block_m asked of tk_moe_gemm: {seen}"
    ref = omoe.matmul(xq, wq, bias, sizes, gather_indx=gi, scatter_indx=sc, x_row_scale=sx, w_col_scale=sw)
    assert_close(ref, y, maxtol=2e-2, what="fp8 y, 256-row tiles")
    assert_allclose_gate(ref, y, what="fp8 y, 256-row tiles")


@pytest.mark.parametrize("per_expert", [False, True])
def test_flexpoint_input_scales(mods, device, per_expert):
    """`FlexCtx(lhs_data=InFlexData(scale=...), rhs_data=InFlexData(scale=...))`: fp8 operands with one-element device
    scales (per expert for the weights when the scale tensor has one entry per expert), `acc *= x_scale * w_scale`
    before the bias (matmul_details/_matmul.py:540-547).  Oracle: dequantise with the scales, pinned GEMM oracle."""
    mm, _, tensor = mods
    from triton_amd.numerics import InFlexData
    g = torch.Generator().manual_seed(31)
    m, n, k, n_slices = 200, 256, 320, 4
    xq = (torch.randn((m, k), generator=g) * 2).to(torch.float8_e4m3fn)
    wq = (torch.randn((n_slices, k, n), generator=g) * 2).to(torch.float8_e4m3fn)
    bias = torch.randn((n_slices, n), generator=g)
    sx = torch.tensor([0.37])
    sw = torch.tensor([0.11, 0.25, 0.5, 0.07]) if per_expert else torch.tensor([0.19])
    sizes = _slice_sizes(m, n_slices, g)
    md = tensor.make_ragged_tensor_metadata(sizes.to(device), m)
    flex = mm.FlexCtx(lhs_data=InFlexData(scale=sx.to(device)), rhs_data=InFlexData(scale=sw.to(device)))
    wd = wq.to(device).transpose(-1, -2).contiguous().transpose(-1, -2)
    y = mm.matmul(xq.to(device), wd, bias.to(device), md, precision_config=mm.PrecisionConfig(flex_ctx=flex, out_dtype=torch.bfloat16))
    ref = omoe.matmul(xq, wq, bias, sizes, x_row_scale=sx.expand(m), w_col_scale=sw.reshape(-1, 1).expand(n_slices, n), out_dtype=torch.bfloat16)
    assert_close(ref, y, what="flexpoint-scaled y")
    assert_allclose_gate(ref, y, what="flexpoint-scaled y")
    with pytest.raises(NotImplementedError):  # output-side flexpoint needs fp8 outputs
        from triton_amd.numerics import OutFlexData
        mm.matmul(xq.to(device), wd, None, md, precision_config=mm.PrecisionConfig(
            flex_ctx=mm.FlexCtx(out_data=OutFlexData(expected_scale=sx.to(device))), out_dtype=torch.bfloat16))


@pytest.mark.parametrize("wkind", ["mxfp4", "mxfp4_tiled"])
def test_cdna4_scale_layout_accepted(mods, device, wkind):
    """Scales pre-shuffled with the reference's `CDNA4MXScaleLayout` (what its default helper returns on this GPU,
    tensor_details/layout.py:43-54) give the same result, bit for bit, as the same scales in the kernel's own order."""
    mm, _, tensor = mods
    from triton_amd.tensor import convert_layout, wrap_torch_tensor
    from triton_amd.tensor_details.layout import CDNA4MXScaleLayout
    g = torch.Generator().manual_seed(23)
    m, n, k, n_slices = 300, 416, 576, 5
    x = torch.randn((m, k), generator=g).to(torch.bfloat16).to(device)
    W = _make_w(n_slices, k, n, wkind, g, device)
    sizes = _slice_sizes(m, n_slices, g)
    md = tensor.make_ragged_tensor_metadata(sizes.to(device), m)
    cd = convert_layout(wrap_torch_tensor(W["scale_cpu"].to(device)), CDNA4MXScaleLayout())
    y_ref = mm.matmul(x, W["w_dev"], None, md, precision_config=mm.PrecisionConfig(b_mx_scale=W["scale_dev"]))
    for _ in range(2):  # the second call takes the cached conversion
        y = mm.matmul(x, W["w_dev"], None, md, precision_config=mm.PrecisionConfig(b_mx_scale=cd))
        assert torch.equal(y, y_ref)


def test_zero_sized(mods, device):
    mm, _, tensor = mods
    for m, n, k in [(0, 5, 7), (5, 0, 7)]:
        x = torch.zeros((m, k), dtype=torch.bfloat16, device=device)
        w = torch.zeros((1, k, n), dtype=torch.bfloat16, device=device)
        assert mm.matmul(x, w, None).shape == (m, n)


def test_rejected_options(mods, device):
    mm, _, _ = mods
    x = torch.zeros((4, 32), dtype=torch.bfloat16, device=device)
    w = torch.zeros((1, 32, 16), dtype=torch.bfloat16, device=device)
    with pytest.raises(AssertionError):  # c_acc_in + scatter (triton_kernels/matmul.py:531)
        mm.matmul(x, w, None, c_acc_in=torch.zeros((4, 16), dtype=torch.bfloat16, device=device),
                  scatter_indx=torch.arange(4, dtype=torch.int32, device=device))
    with pytest.raises(NotImplementedError):  # c_acc_in of another type than the output
        mm.matmul(x, w, None, c_acc_in=torch.zeros((4, 16), device=device))
    with pytest.raises(NotImplementedError):  # NVFP4 output (float8 block scales) is a Blackwell format
        mm.matmul(x, w, None, epilogue=mm.Epilogue(mm.FnSpecs(mm.FnName.QUANTIZE_NVFP4.name, object(), (), ()), (), (), 2.0))
    with pytest.raises(ValueError):  # an MX epilogue without a scale tensor to fill
        mm.matmul(x, w, None, precision_config=mm.PrecisionConfig(out_dtype=torch.float8_e4m3fn),
                  epilogue=mm.Epilogue(mm.FnSpecs(mm.FnName.QUANTIZE_MXFP8.name, object(), (), ()), (), (), 6.0))
    with pytest.raises(mm.InapplicableConstraint):
        with mm.scoped_opt_flags_constraints({"split_k": 2}):
            mm.matmul(x, w, None)
    with pytest.raises(mm.InapplicableConstraint):
        with mm.scoped_opt_flags_constraints({"is_persistent": True}):
            mm.matmul(x, w, None)


def test_n_contiguous_weights_are_relaid_once(mods, device):
    """A plain torch [E, K, N] bf16 weight (N-contiguous) is transposed to the K-contiguous form the kernels read on
    the first call only: later calls reuse the copy kept on the tensor (same object, no new device memory), and an
    in-place update of the weight makes a new copy."""
    mm, _, tensor = mods
    g = torch.Generator().manual_seed(5)
    E, K, N, m = 4, 256, 384, 200
    x = torch.randn((m, K), generator=g).to(torch.bfloat16)
    w = (torch.randn((E, K, N), generator=g) * 0.1).to(torch.bfloat16)
    sizes = torch.tensor([50, 0, 100, 50], dtype=torch.int32)
    md = tensor.make_ragged_tensor_metadata(sizes.to(device), m)
    wd, xd = w.to(device), x.to(device)
    y1 = mm.matmul(xd, wd, None, md)
    cached = wd._tk_k_contiguous[1]
    assert cached.stride(-2) == 1
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    y2 = mm.matmul(xd, wd, None, md)
    torch.cuda.synchronize()
    assert wd._tk_k_contiguous[1] is cached, "second call converted the weights again"
    assert torch.cuda.memory_allocated() - before <= y2.numel() * 2 + 4096, "second call allocated more than its output"
    assert torch.equal(y1, y2)
    assert_close(omoe.matmul(x, w, None, sizes), y2, what="y")
    wd.mul_(2.0)  # in-place update: the cached copy is stale and must be rebuilt
    y3 = mm.matmul(xd, wd, None, md)
    assert wd._tk_k_contiguous[1] is not cached
    assert_close(omoe.matmul(x, (w.float() * 2).to(torch.bfloat16), None, sizes), y3, what="y after update")


@pytest.mark.parametrize("idle", [0, 7, 250, 1000])
def test_idle_sms_keeps_results(mods, device, idle):
    """`idle_sms` (constraint or `set_idle_sms`) shrinks the persistent grid of the tiled kernels; results do not change
    (with every compute unit "idle" one workgroup still runs)."""
    mm, _, tensor = mods
    g = torch.Generator().manual_seed(6)
    m, n, k = 1500, 512, 1024
    W = _make_w(10, k, n, "mxfp4_tiled", g, device)
    x = torch.randn((m, k), generator=g).to(torch.bfloat16)
    sizes = _slice_sizes(m, 10, g)
    md = tensor.make_ragged_tensor_metadata(sizes.to(device), m)
    pc = mm.PrecisionConfig(b_mx_scale=W["scale_dev"])
    base = mm.matmul(x.to(device), W["w_dev"], None, md, precision_config=pc)
    with mm.scoped_opt_flags_constraints({"idle_sms": idle}):
        y = mm.matmul(x.to(device), W["w_dev"], None, md, precision_config=pc)
    assert torch.equal(base, y)


def test_standalone_swiglu_with_routing_data(mods, device):
    """`swiglu(a, alpha, pc, routing_data=rdata)` bounds the rows by the routed row count read on the device
    (swiglu.py:53-55 of the reference): rows past it are left unwritten, the rest match the oracle."""
    _, sw, _ = mods
    from triton_amd.legacy import routing
    g = torch.Generator().manual_seed(9)
    T, E, k, n = 40, 8, 2, 96
    logits = torch.randn((T, E), generator=g)
    rdata, _, _ = routing(logits.to(device), k, n_rows=25)  # 25 of the 40 tokens are routed: 50 rows
    a = torch.randn((T * k, 2 * n), generator=g).to(torch.bfloat16)
    out = sw.swiglu(a.to(device), 1.702, sw.PrecisionConfig(limit=7.0), routing_data=rdata)
    ref = omoe.swiglu(a, 1.702, 7.0)
    assert int(rdata.expt_data.slice_offs[E]) == 50
    assert_close(ref[:50], out[:50], what="swiglu rows")


def _mx_activations(x):
    """MXFP8 (e4m3 + e8m0 per 32 along K) quantisation of x with the oracle, and what it dequantises to."""
    xq, xs = omx.downcast_to_mxfp(x, torch.float8_e4m3fn, axis=-1)
    return xq, xs, omx.upcast_from_mxfp(xq, xs, torch.bfloat16, axis=-1)


@pytest.mark.parametrize("m, n, k", [(16, 256, 256), (300, 400, 416), (1000, 704, 800), (256, 1024, 512), (1500, 512, 1024)])
@pytest.mark.parametrize("block_m", [128, 256])
@pytest.mark.parametrize("do_gather, do_scatter, do_gamma, swiglu", [(False, False, False, False), (True, False, False, True),
                                                                      (False, True, True, False), (True, True, True, False)])
def test_matmul_mxfp8_activations(mods, device, m, n, k, block_m, do_gather, do_scatter, do_gamma, swiglu):
    """MXFP8 activations x MXFP4 weights (`PrecisionConfig.a_mx_scale`; the reference's cases:
    tests/test_matmul.py:207-216) on the scaled MFMA.  The oracle is fed the SAME quantised activations, dequantised
    to bf16 as the reference's `apply_precision` does (matmul.py:783-795): both operands are then exact in bf16 and only
    the accumulation order differs, so the bf16 GEMM tolerance applies."""
    mm, sw_mod, tensor = mods
    g = torch.Generator().manual_seed(m * 5 + n + k + block_m)
    n_slices = 10
    x = torch.randn((m, k), generator=g).to(torch.bfloat16)
    xq, xs, x_deq = _mx_activations(x)
    W = _make_w(n_slices, k, n, "mxfp4_tiled", g, device)
    bias = torch.randn((n_slices, n), generator=g)
    sizes = _slice_sizes(m, n_slices, g)
    md = tensor.make_ragged_tensor_metadata(sizes.to(device), m)
    gi = torch.randint(0, m, (m, ), generator=g, dtype=torch.int32) if do_gather else None
    sc = torch.randperm(m, generator=g).to(torch.int32) if do_scatter else None
    if sc is not None and m > 20:
        sc[torch.rand(m, generator=g) < 0.05] = -1
    gam = 2.0**torch.randint(-5, 0, (m, ), generator=g).float() if do_gamma else None
    act = mm.FusedActivation(mm.FnSpecs("swiglu", sw_mod.swiglu_fn, ("alpha", "limit"), reduction_n=2), (1.702, 7.0)) if swiglu else None
    pc = mm.PrecisionConfig(a_mx_scale=xs.to(device), b_mx_scale=W["scale_dev"], out_dtype=torch.bfloat16)
    dv = lambda t: None if t is None else t.to(device)
    with mm.scoped_opt_flags_constraints({"block_m": block_m}):
        y = mm.matmul(xq.to(device), W["w_dev"], bias.to(device), md, gather_indx=dv(gi), scatter_indx=dv(sc), gammas=dv(gam),
                      precision_config=pc, fused_activation=act)
    ref = omoe.matmul(x_deq, W["w_cpu"], bias, sizes, gather_indx=gi, scatter_indx=sc, gammas=gam, w_mx_scale=W["scale_cpu"],
                      out_dtype=torch.float32 if swiglu else torch.bfloat16)
    if swiglu:
        ref = omoe.swiglu(ref, 1.702, 7.0).to(torch.bfloat16)
    got = y.cpu()
    if sc is not None:  # rows that no entry writes are undefined in the kernel path, zero in the oracle
        written = torch.zeros(m, dtype=torch.bool)
        written[sc[sc >= 0].long()] = True
        got = torch.where(written[:, None], got, torch.zeros_like(got))
    assert y.dtype == torch.bfloat16 and got.shape == ref.shape
    assert_close(ref, got, maxtol=3e-2, what="y")
    assert_allclose_gate(ref, got, what="y")


@pytest.mark.parametrize("swiglu, scatter", [(True, False), (False, True), (False, False)])
@pytest.mark.parametrize("block_m", [128, 256])
def test_mxfp8_activations_with_fused_mx_output(mods, device, swiglu, scatter, block_m):
    """With MXFP8 activations the `QUANTIZE_MXFP8` epilogue runs inside the GEMM, on the fp32 accumulator
    (matmul_details/_matmul.py:593-637).  Against the oracle's GEMM (fp32 result) -> MX quantisation: (1) block scales
    equal except where the two fp32 sums put a block's maximum on different sides of a power-of-two boundary (a handful
    of blocks at most), (2) dequantised values within the reference's tolerance for this epilogue (maxtol 4e-1 /
    rmstol 4e-2, tests/test_matmul.py:627-643), (3) nearly all codes bit-equal."""
    mm, sw_mod, tensor = mods
    from triton_amd.numerics_details.mxfp import quantize_mxfp8_fn
    g = torch.Generator().manual_seed(23 + block_m)
    m, n, k, n_slices = 600, 512, 416, 6
    x = torch.randn((m, k), generator=g).to(torch.bfloat16)
    xq, xs, x_deq = _mx_activations(x)
    W = _make_w(n_slices, k, n, "mxfp4_tiled", g, device)
    bias = torch.randn((n_slices, n), generator=g)
    sizes = _slice_sizes(m, n_slices, g)
    md = tensor.make_ragged_tensor_metadata(sizes.to(device), m)
    sc = torch.randperm(m, generator=g).to(torch.int32) if scatter else None
    act = mm.FusedActivation(mm.FnSpecs("swiglu", sw_mod.swiglu_fn, ("alpha", "limit"), reduction_n=2), (1.702, 7.0)) if swiglu else None
    n_out = n // 2 if swiglu else n
    epi = mm.Epilogue(mm.FnSpecs(mm.FnName.QUANTIZE_MXFP8.name, quantize_mxfp8_fn, (), ()), tuple(), tuple(), effective_itemsize=6.0)
    c_scale = torch.full((m, n_out // 32), 0xFF, dtype=torch.uint8, device=device)
    pc = mm.PrecisionConfig(a_mx_scale=xs.to(device), b_mx_scale=W["scale_dev"], c_mx_scale=c_scale, out_dtype=torch.float8_e4m3fn)
    with mm.scoped_opt_flags_constraints({"block_m": block_m}):
        yq = mm.matmul(xq.to(device), W["w_dev"], bias.to(device), md, precision_config=pc, epilogue=epi, fused_activation=act,
                       scatter_indx=None if sc is None else sc.to(device))
    assert yq.dtype == torch.float8_e4m3fn and yq.shape == (m, n_out) and pc.c_mx_scale is c_scale
    h = omoe.matmul(x_deq, W["w_cpu"], bias, sizes, w_mx_scale=W["scale_cpu"], scatter_indx=sc, out_dtype=torch.float32)
    if swiglu:
        h = omoe.swiglu(h, 1.702, 7.0)
    q_ref, s_ref = omx.downcast_to_mxfp(h, torch.float8_e4m3fn, axis=-1)
    s_got, q_got = c_scale.cpu(), yq.cpu()
    scale_diff = (s_ref != s_got).float().mean().item()
    assert scale_diff <= 2e-3, f"{scale_diff:.4g} of the block scales differ from the oracle's"
    code_diff = (q_ref.view(torch.uint8) != q_got.view(torch.uint8)).float().mean().item()
    assert code_diff <= 0.02, f"{code_diff:.4g} of the e4m3 codes differ from the oracle's"
    ref = omx.upcast_from_mxfp(q_ref, s_ref, torch.bfloat16, axis=-1)
    got = omx.upcast_from_mxfp(q_got, s_got, torch.bfloat16, axis=-1)
    assert_close(ref, got, maxtol=4e-1, rmstol=4e-2, what="dequantised MX output")
    # the quantised result is close to the unquantised GEMM (e4m3 has 3 mantissa bits: half a step is 2^-4 relative)
    assert_close(h, got, maxtol=1.0, rmstol=4e-2, what="MX output against the unquantised result")


@pytest.mark.parametrize("kind", ["mxfp8_e4m3", "mxfp8_e5m2", "mxfp4"])
@pytest.mark.parametrize("swiglu, scatter, gamma", [(True, False, False), (False, True, True), (False, False, False)])
@pytest.mark.parametrize("block_m", [128, 256])
def test_bf16_activations_with_fused_mx_output(mods, device, monkeypatch, kind, swiglu, scatter, gamma, block_m):
    """bf16 activations x tiled MXFP4 weights with `Epilogue(QUANTIZE_MXFP8 | QUANTIZE_MXFP4)`: the prefill kernel's epilogue
    quantises the fp32 accumulator (matmul_details/_matmul.py:593-637) to e4m3, e5m2 or packed e2m1.  Against the oracle's
    GEMM (fp32 result, bias, swiglu, gate weight) -> oracle MX quantiser: block scales equal except where the two fp32
    sums put a block's maximum on different sides of a power-of-two boundary, nearly all codes bit-equal, and the
    dequantised values within the reference's tolerance for this epilogue (tests/test_matmul.py:627-643)."""
    mm, sw_mod, tensor = mods
    from triton_amd.numerics_details.mxfp import quantize_mxfp4_fn, quantize_mxfp8_fn
    g = torch.Generator().manual_seed(29 + block_m)
    m, n, k, n_slices = 700, 640, 416, 6
    x = torch.randn((m, k), generator=g).to(torch.bfloat16)
    W = _make_w(n_slices, k, n, "mxfp4_tiled", g, device)
    bias = torch.randn((n_slices, n), generator=g)
    sizes = _slice_sizes(m, n_slices, g)
    md = tensor.make_ragged_tensor_metadata(sizes.to(device), m)
    sc = torch.randperm(m, generator=g).to(torch.int32) if scatter else None
    gammas = 2.0**torch.randint(-5, 0, (m, ), generator=g).float() if gamma else None
    act = mm.FusedActivation(mm.FnSpecs("swiglu", sw_mod.swiglu_fn, ("alpha", "limit"), reduction_n=2), (1.702, 7.0)) if swiglu else None
    n_out = n // 2 if swiglu else n
    out_dtype = {"mxfp8_e4m3": torch.float8_e4m3fn, "mxfp8_e5m2": torch.float8_e5m2, "mxfp4": torch.uint8}[kind]
    name, fn = (mm.FnName.QUANTIZE_MXFP4.name, quantize_mxfp4_fn) if kind == "mxfp4" else (mm.FnName.QUANTIZE_MXFP8.name, quantize_mxfp8_fn)
    epi = mm.Epilogue(mm.FnSpecs(name, fn, (), ()), tuple(), tuple(), effective_itemsize=6.0)
    c_scale = torch.full((m, n_out // 32), 0xFF, dtype=torch.uint8, device=device)
    pc = mm.PrecisionConfig(b_mx_scale=W["scale_dev"], c_mx_scale=c_scale, out_dtype=out_dtype)
    def two_step(*args, **kwargs):
        raise AssertionError("the GEMM + quantiser path ran instead of the fused epilogue")

    monkeypatch.setattr(mm, "_matmul_mx_out", two_step)
    with mm.scoped_opt_flags_constraints({"block_m": block_m}):
        yq = mm.matmul(x.to(device), W["w_dev"], bias.to(device), md, precision_config=pc, epilogue=epi, fused_activation=act,
                       scatter_indx=None if sc is None else sc.to(device), gammas=None if gammas is None else gammas.to(device))
    assert yq.dtype == out_dtype and yq.shape == (m, n_out // 2 if kind == "mxfp4" else n_out)
    h = omoe.matmul(x, W["w_cpu"], bias, sizes, w_mx_scale=W["scale_cpu"], scatter_indx=sc, gammas=None if swiglu else gammas, out_dtype=torch.float32)
    if swiglu:
        h = omoe.swiglu(h, 1.702, 7.0)
    q_ref, s_ref = omx.downcast_to_mxfp(h, out_dtype, axis=-1)
    s_got, q_got = c_scale.cpu(), yq.cpu()
    scale_diff = (s_ref != s_got).float().mean().item()
    assert scale_diff <= 2e-3, f"{scale_diff:.4g} of the block scales differ from the oracle's"
    if kind == "mxfp4":
        lo_diff = ((q_ref & 0xF) != (q_got & 0xF)).float().mean().item()
        hi_diff = ((q_ref >> 4) != (q_got >> 4)).float().mean().item()
        code_diff = 0.5 * (lo_diff + hi_diff)
    else:
        code_diff = (q_ref.view(torch.uint8) != q_got.view(torch.uint8)).float().mean().item()
    assert code_diff <= 0.02, f"{code_diff:.4g} of the {kind} codes differ from the oracle's"
    ref = omx.upcast_from_mxfp(q_ref, s_ref, torch.bfloat16, axis=-1)
    got = omx.upcast_from_mxfp(q_got, s_got, torch.bfloat16, axis=-1)
    if kind == "mxfp4":
        # 3-bit magnitudes: a code that differs moves a value by a whole e2m1 step, so the bound is on how many differ (above)
        # and on the rms error
        from oracle.checks import rel_errors
        _, rms = rel_errors(ref, got)
        assert rms <= 3e-2, f"mxfp4 output: rms {rms:.4g}"
    else:
        assert_close(ref, got, maxtol=4e-1, rmstol=4e-2, what="dequantised MX output")


@pytest.mark.parametrize("kind", ["bf16", "mxfp4", "mxfp4_tiled"])
@pytest.mark.parametrize("B, m, n, k", [(3, 200, 256, 256), (10, 72, 576, 768), (4, 1, 64, 128)])
@pytest.mark.parametrize("swiglu", [False, True])
def test_batched_matmul(mods, device, kind, B, m, n, k, swiglu):
    """Batched mode (python/triton_kernels/tests/test_matmul.py:116-127,144-176 "batched"): a [B, m, k] x b [B, k, n] with a
    bias per batch; against the oracle's ragged GEMM with B slices of m rows (what batched mode is), output [B, m, n_out]."""
    mm, _, _ = mods
    from triton_amd.swiglu import swiglu_fn
    g = torch.Generator().manual_seed(B * 1000 + m + n + k)
    a = torch.randn((B, m, k), generator=g).to(torch.bfloat16)
    bias = torch.randn((B, n), generator=g)
    w = _make_w(B, k, n, kind, g, device)
    sizes = torch.full((B, ), m, dtype=torch.int32)
    ref = omoe.matmul(a.reshape(B * m, k), w["w_cpu"], bias, sizes, w_mx_scale=w.get("scale_cpu"))
    act = None
    if swiglu:
        act = mm.FusedActivation(mm.FnSpecs("swiglu", swiglu_fn, ("alpha", "limit"), reduction_n=2), (1.702, 7.0))
        ref = omoe.swiglu(ref, 1.702, 7.0)
    pc = mm.PrecisionConfig(b_mx_scale=w.get("scale_dev"))
    out = mm.matmul(a.to(device), w["w_dev"], bias.to(device), precision_config=pc, fused_activation=act)
    assert out.shape == (B, m, n // (2 if swiglu else 1)) and out.dtype == torch.bfloat16
    if swiglu:  # computed on the fp32 accumulators, the oracle rounds the GEMM output to bf16 first (see test_fused_swiglu)
        assert_close(ref.reshape(out.shape), out, maxtol=3e-2, what="batched swiglu(y)")
    else:
        assert_allclose_gate(ref.reshape(out.shape), out, what="batched matmul")


@pytest.mark.parametrize("kind", ["mxfp4_tiled", "fp8_tiled"])
@pytest.mark.parametrize("sizes", [[200], [200, 200, 200], [130, 0, 300], [1, 1, 1, 1, 1, 1, 1]])
def test_persistent_kernels_with_a_handful_of_tiles(mods, device, kind, sizes):
    """The persistent prefill kernels launch one workgroup per tile when there are fewer tiles than compute units; with
    fewer than 8 workgroups some XCD queue of the tile claimer has no workgroup of its own, and its tiles must still be
    computed.  The output buffer is pre-filled with NaN so that a tile nobody wrote cannot pass."""
    mm, _, tensor = mods
    from triton_amd.tensor import convert_layout, wrap_torch_tensor
    from triton_amd.tensor_details.layout import make_default_matmul_fp8_w_layout
    g = torch.Generator().manual_seed(len(sizes) * 100 + sizes[0])
    E, m, k, n = len(sizes), sum(sizes), 256, 256
    st = torch.tensor(sizes, dtype=torch.int32)
    md = tensor.make_ragged_tensor_metadata(st.to(device), m)
    bias = torch.randn((E, n), generator=g)
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=device)
    if kind == "mxfp4_tiled":
        x = torch.randn((m, k), generator=g).to(torch.bfloat16)
        w = _make_w(E, k, n, kind, g, device)
        y = mm.matmul(x.to(device), w["w_dev"], bias.to(device), md, precision_config=mm.PrecisionConfig(b_mx_scale=w["scale_dev"]), c=out)
        ref = omoe.matmul(x, w["w_cpu"], bias, st, w_mx_scale=w["scale_cpu"])
    else:
        xq, sx, wq, sw = _fp8_operands(m, n, k, E, g)
        wd = convert_layout(wrap_torch_tensor(wq.to(device).transpose(-1, -2).contiguous().transpose(-1, -2)), make_default_matmul_fp8_w_layout())
        pc = mm.PrecisionConfig(a_mx_tensor_scale=sx.to(device), b_mx_tensor_scale=sw.to(device), out_dtype=torch.bfloat16)
        y = mm.matmul(xq.to(device), wd, bias.to(device), md, precision_config=pc, c=out)
        ref = omoe.matmul(xq, wq, bias, st, x_row_scale=sx, w_col_scale=sw, out_dtype=torch.bfloat16)
    assert y.data_ptr() == out.data_ptr()
    assert not torch.isnan(y).any(), "rows that no tile wrote"
    assert_allclose_gate(ref, y, what="few tiles")
