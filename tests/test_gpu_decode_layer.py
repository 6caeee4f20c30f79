"""The decode-sized MoE layer in one launch (`tk_moe_decode_layer` behind `moe_mlp`) against the CPU oracle and against
the three-call sequence it stands for (routing -> gather-GEMM + swiglu -> scatter-GEMM * gate -> combine).

Routing decisions must be bit-equal to the oracle's (and the gate values close); the layer output is held to the same
gates as the three-call layer tests.  Covers benchmark config 4 at its real shape (128 experts, top-4, skewed router,
T in {1, 4, 16, 64}), repeated launches on one workspace (the counters are left clean), heavy skew (one expert with
many row blocks), odd shapes (K not a multiple of 128, the largest dimensions, more than 128 experts), and a HIP graph replayed with eager
work in between."""
import pytest
import torch

from oracle import moe as omoe
from oracle import mxfp as omx
from oracle import routing as ort
from oracle.checks import assert_allclose_gate, assert_close, assert_equal

pytestmark = pytest.mark.gpu

LAYER_GATE_SLACK = 1e-4  # see tests/test_gpu_moe_layer.py


@pytest.fixture(scope="module")
def api(device):
    from triton_kernels import moe_decode
    from triton_kernels.legacy import matmul_ogs, routing
    from triton_kernels.matmul import FnSpecs, FusedActivation, PrecisionConfig
    from triton_kernels.swiglu import swiglu_fn

    class A:
        pass

    a = A()
    a.md, a.routing, a.matmul_ogs, a.PrecisionConfig = moe_decode, routing, matmul_ogs, PrecisionConfig
    a.act = lambda alpha, limit: FusedActivation(FnSpecs("swiglu", swiglu_fn, ("alpha", "limit"), reduction_n=2), (alpha, limit))
    return a


@pytest.fixture(scope="module")
def gptoss_weights(device):
    from bench import make_moe_weights, to_matmul_layout
    W0 = make_moe_weights(128, 2880, 5760, seed=2, device=device)[0]
    return {"strided": W0, "tiled": to_matmul_layout(W0)}


def _oracle_layer(x, logits, k, W0, alpha=1.702, limit=7.0):
    r = ort.routing(logits, k)
    sizes = r.meta.col_sum
    act = torch.nonzero(sizes > 0).flatten()
    pick = lambda name: None if W0[name] is None else W0[name][act.to(W0[name].device)].cpu()
    h = omoe.matmul(x, pick("w1"), pick("b1"), sizes[act], gather_indx=r.gather_indx, w_mx_scale=pick("w1s"))
    a = omoe.swiglu(h, alpha, limit)
    y = omoe.matmul(a, pick("w2"), pick("b2"), sizes[act], scatter_indx=r.scatter_indx, gammas=r.gammas, w_mx_scale=pick("w2s"))
    return omoe.reduce_k(y, k), r


def _run(api, W, x, logits, k, act, **kw):
    pc1, pc2 = api.PrecisionConfig(b_mx_scale=W["w1s"]), api.PrecisionConfig(b_mx_scale=W["w2s"])
    assert api.md.one_launch_reason(x, logits, k, W["w1"], W["b1"], W["w2"], W["b2"], pc1, pc2, act) is None
    return api.md.moe_decode_layer(x, logits, k, W["w1"], W["b1"], W["w2"], W["b2"], pc1, pc2, act, **kw)


@pytest.mark.parametrize("T", [1, 4, 16, 64])
def test_config4_full_shape_one_launch(api, device, gptoss_weights, T):
    g = torch.Generator().manual_seed(3)
    E, k, d = 128, 4, 2880
    ebias = torch.randn((E, ), generator=g) * 1.5
    x = torch.randn((T, d), generator=g).to(torch.bfloat16)
    logits = torch.randn((T, E), generator=g) + ebias
    W = gptoss_weights["tiled"]
    act = api.act(1.702, 7.0)
    xd, ld = x.to(device), logits.to(device)
    ref, r = _oracle_layer(x, logits, k, gptoss_weights["strided"])
    for rep in range(3):  # the same workspace three times in a row
        out, indx, vals = _run(api, W, xd, ld, k, act, return_routing=True)
        torch.cuda.synchronize()
        assert api.md.workspace_error_word(xd, ld, k, W["w1"]) == 0
        assert_equal(r.indx, indx.to(torch.int32), f"indx (launch {rep})")
        assert_close(r.vals, vals, what="gate values")
        assert_close(ref, out, maxtol=3e-2, what=f"one-launch decode layer T={T} (launch {rep})")
        assert_allclose_gate(ref, out, what=f"one-launch decode layer T={T}", max_bad_frac=LAYER_GATE_SLACK)
    # the three-call sequence on the same inputs agrees to the same gates (it rounds at the same places)
    rdata, gather, scatter = api.routing(ld, k)
    pc1, pc2 = api.PrecisionConfig(b_mx_scale=W["w1s"]), api.PrecisionConfig(b_mx_scale=W["w2s"])
    h = api.matmul_ogs(xd, W["w1"], W["b1"], rdata, gather_indx=gather, precision_config=pc1, fused_activation=act)
    three = api.matmul_ogs(h, W["w2"], W["b2"], rdata, scatter_indx=scatter, precision_config=pc2, gammas=rdata.gate_scal)
    assert torch.equal(rdata.expt_indx, indx)
    assert_close(rdata.gate_vals, vals, what="gate values against tk_route")
    assert_close(three.cpu(), out, maxtol=3e-2, what="one launch against three calls")
    # moe_mlp picks the single launch from 8 routed rows on, the three calls below
    again = api.md.moe_mlp(xd, ld, k, W["w1"], W["b1"], W["w2"], W["b2"], pc1, pc2, act)
    if T * k >= api.md.MIN_ROWS:
        assert torch.equal(again, out), "two launches on the same inputs differ"
    else:
        assert torch.equal(again, three), "moe_mlp below its row threshold is the three-call sequence"


def test_heavy_skew_many_row_blocks_on_one_expert(api, device, gptoss_weights):
    """64 tokens that all pick expert 5 first (64 rows = 4 row blocks of one expert) and spread their other three
    choices: three launches in a row against the oracle."""
    g = torch.Generator().manual_seed(21)
    T, E, k, d = 64, 128, 4, 2880
    x = torch.randn((T, d), generator=g).to(torch.bfloat16)
    logits = torch.randn((T, E), generator=g)
    logits[:, 5] += 20.0
    logits[:, 77] += torch.where(torch.arange(T) % 2 == 0, 10.0, 0.0)  # a second popular expert with 32 rows
    W = gptoss_weights["tiled"]
    act = api.act(1.702, 7.0)
    xd, ld = x.to(device), logits.to(device)
    ref, r = _oracle_layer(x, logits, k, gptoss_weights["strided"])
    assert int(r.meta.col_sum[5]) == 64 and int(r.meta.col_sum[77]) >= 32
    # With one gate near 1 the output is a single expert row, values up to 5: the share of elements outside the
    # rtol 2e-2 / atol 1e-2 gate is a property of the input (the three-call sequence leaves the same elements outside),
    # so the bound here is what that sequence shows plus the usual slack.
    rdata, gather, scatter = api.routing(ld, k)
    pc1, pc2 = api.PrecisionConfig(b_mx_scale=W["w1s"]), api.PrecisionConfig(b_mx_scale=W["w2s"])
    h = api.matmul_ogs(xd, W["w1"], W["b1"], rdata, gather_indx=gather, precision_config=pc1, fused_activation=act)
    three = api.matmul_ogs(h, W["w2"], W["b2"], rdata, scatter_indx=scatter, precision_config=pc2, gammas=rdata.gate_scal).cpu().float()
    reff = ref.float()
    outside = lambda got: int(((got - reff).abs() > 0.01 + 0.02 * reff.abs()).sum())
    allowed = outside(three) + LAYER_GATE_SLACK * ref.numel()
    for rep in range(3):
        out, indx, _ = _run(api, W, xd, ld, k, act, return_routing=True)
        torch.cuda.synchronize()
        assert api.md.workspace_error_word(xd, ld, k, W["w1"]) == 0
        assert_equal(r.indx, indx.to(torch.int32), "indx")
        assert_close(ref, out, maxtol=3e-2, what=f"skewed decode layer (launch {rep})")
        assert outside(out.cpu().float()) <= allowed, f"launch {rep}: {outside(out.cpu().float())} elements outside the gate, the three-call sequence has {outside(three)}"
        assert_close(three, out, maxtol=3e-2, what="one launch against three calls")


@pytest.mark.parametrize("T, E, k, d_model, d_ff, bias_dtype, limit", [
    (7, 8, 2, 224, 160, torch.float32, None),       # K not a multiple of 128 in either GEMM, fp32 biases, no limit
    (33, 12, 4, 256, 3072, torch.bfloat16, 7.0),    # the largest d_ff (every K-slice of GEMM 2 in use), ragged row blocks
    (16, 130, 1, 384, 192, None, 7.0),              # E > 128 (the wide-router variant), top-1, no biases
    (64, 4, 4, 3072, 512, torch.bfloat16, 5.0),     # the largest d_model, every token on every expert (4 blocks each)
    (256, 16, 1, 128, 64, None, None),              # 256 tokens: every word of the token masks in use, top-1
    (32, 512, 8, 128, 128, torch.float32, 7.0),     # the most experts (the wide router, eight experts per lane), top-8
    (100, 64, 2, 2880, 64, torch.bfloat16, None),   # 200 routed rows over four mask words, gpt-oss d_model, a thin FFN
])
def test_odd_shapes(api, device, T, E, k, d_model, d_ff, bias_dtype, limit):
    from bench import to_matmul_layout
    g = torch.Generator().manual_seed(T * 131 + E)
    x = torch.randn((T, d_model), generator=g).to(torch.bfloat16)
    logits = torch.randn((T, E), generator=g)
    w1 = (torch.randn((E, d_model, 2 * d_ff), generator=g) / d_model**0.5).to(torch.bfloat16)
    w2 = (torch.randn((E, d_ff, d_model), generator=g) / d_ff**0.5).to(torch.bfloat16)
    w1q, w1s = omx.downcast_to_mxfp(w1, torch.uint8, axis=1)
    w2q, w2s = omx.downcast_to_mxfp(w2, torch.uint8, axis=1)
    b1 = b2 = None
    if bias_dtype is not None:
        b1 = (torch.randn((E, 2 * d_ff), generator=g) * 0.1).to(bias_dtype)
        b2 = (torch.randn((E, d_model), generator=g) * 0.1).to(bias_dtype)
    W0 = dict(w1=w1q, w1s=w1s, w2=w2q, w2s=w2s, b1=b1, b2=b2)
    dev = lambda t: None if t is None else t.to(device)
    W = to_matmul_layout({n: dev(t) for n, t in W0.items()})
    act = api.act(1.702, limit)
    xd, ld = x.to(device), logits.to(device)
    ref, r = _oracle_layer(x, logits, k, W0, limit=limit)
    # the three-call sequence on the same inputs bounds the share of elements outside the rtol 2e-2 / atol 1e-2 gate
    # (where the k partial rows cancel, a bf16 ulp of a partial row exceeds the gate whichever path computes it)
    rdata, gather, scatter = api.routing(ld, k)
    pc1, pc2 = api.PrecisionConfig(b_mx_scale=W["w1s"]), api.PrecisionConfig(b_mx_scale=W["w2s"])
    h = api.matmul_ogs(xd, W["w1"], W["b1"], rdata, gather_indx=gather, precision_config=pc1, fused_activation=act)
    three = api.matmul_ogs(h, W["w2"], W["b2"], rdata, scatter_indx=scatter, precision_config=pc2, gammas=rdata.gate_scal).cpu().float()
    reff = ref.float()
    outside = lambda got: int(((got - reff).abs() > 0.01 + 0.02 * reff.abs()).sum())
    allowed = outside(three) + LAYER_GATE_SLACK * ref.numel()
    for rep in range(2):
        out, indx, vals = _run(api, W, xd, ld, k, act, return_routing=True)
        torch.cuda.synchronize()
        assert api.md.workspace_error_word(xd, ld, k, W["w1"]) == 0
        assert_equal(r.indx, indx.to(torch.int32), "indx")
        assert_close(r.vals, vals, what="gate values")
        assert_close(ref, out, maxtol=3e-2, what=f"decode layer {T}x{E} top-{k} d={d_model} f={d_ff} (launch {rep})")
        assert outside(out.cpu().float()) <= allowed, f"launch {rep}: {outside(out.cpu().float())} elements outside the gate, the three-call sequence has {outside(three)}"
        assert_close(three, out, maxtol=3e-2, what="one launch against three calls")


def test_one_launch_layer_in_a_hip_graph(api, device, gptoss_weights):
    """Captured once, replayed three times with new inputs and eager launches in between; every replay must equal the
    eager launch on the same inputs bit for bit."""
    g = torch.Generator().manual_seed(31)
    T, E, k, d = 16, 128, 4, 2880
    W = gptoss_weights["tiled"]
    act = api.act(1.702, 7.0)
    x = torch.randn((T, d), generator=g).to(torch.bfloat16).to(device)
    logits = (torch.randn((T, E), generator=g) + torch.randn((E, ), generator=g) * 1.5).to(device)
    _run(api, W, x, logits, k, act)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        _run(api, W, x, logits, k, act)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        got = _run(api, W, x, logits, k, act)
    for rep in range(3):
        x.copy_(torch.randn((T, d), generator=g).to(torch.bfloat16))
        logits.copy_(torch.randn((T, E), generator=g) + torch.randn((E, ), generator=g) * 1.5)
        graph.replay()
        torch.cuda.synchronize()
        want = _run(api, W, x, logits, k, act)
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"graph replay {rep} differs from the eager launch"


def test_fallback_and_refusals(api, device, gptoss_weights):
    W = gptoss_weights["tiled"]
    act = api.act(1.702, 7.0)
    pc1, pc2 = api.PrecisionConfig(b_mx_scale=W["w1s"]), api.PrecisionConfig(b_mx_scale=W["w2s"])
    x = torch.randn((128, 2880), device=device).to(torch.bfloat16)  # 512 routed rows: too many for the single launch
    logits = torch.randn((128, 128), device=device)
    assert api.md.one_launch_reason(x, logits, 4, W["w1"], W["b1"], W["w2"], W["b2"], pc1, pc2, act) is not None
    with pytest.raises(NotImplementedError):
        api.md.moe_decode_layer(x, logits, 4, W["w1"], W["b1"], W["w2"], W["b2"], pc1, pc2, act)
    out = api.md.moe_mlp(x, logits, 4, W["w1"], W["b1"], W["w2"], W["b2"], pc1, pc2, act)  # three calls
    rdata, gather, scatter = api.routing(logits, 4)
    h = api.matmul_ogs(x, W["w1"], W["b1"], rdata, gather_indx=gather, precision_config=pc1, fused_activation=act)
    want = api.matmul_ogs(h, W["w2"], W["b2"], rdata, scatter_indx=scatter, precision_config=pc2, gammas=rdata.gate_scal)
    assert torch.equal(out, want)
    # activations whose rows are not contiguous take the three calls as well (the single launch reads rows of x 16 bytes
    # at a time through a buffer resource), and give what the contiguous copy gives
    xt = torch.randn((2880, 16), device=device).to(torch.bfloat16).t()  # [16, 2880] with unit stride along the tokens
    lg = torch.randn((16, 128), device=device)
    assert api.md.one_launch_reason(xt, lg, 4, W["w1"], W["b1"], W["w2"], W["b2"], pc1, pc2, act) is not None
    assert api.md.one_launch_reason(xt.contiguous(), lg, 4, W["w1"], W["b1"], W["w2"], W["b2"], pc1, pc2, act) is None
    a = api.md.moe_mlp(xt, lg, 4, W["w1"], W["b1"], W["w2"], W["b2"], pc1, pc2, act)
    rdata, gather, scatter = api.routing(lg, 4)
    h = api.matmul_ogs(xt.contiguous(), W["w1"], W["b1"], rdata, gather_indx=gather, precision_config=pc1, fused_activation=act)
    b = api.matmul_ogs(h, W["w2"], W["b2"], rdata, scatter_indx=scatter, precision_config=pc2, gammas=rdata.gate_scal)
    assert torch.equal(a, b)
    one = api.md.moe_mlp(xt.contiguous(), lg, 4, W["w1"], W["b1"], W["w2"], W["b2"], pc1, pc2, act)  # (one launch: other K-split)
    torch.testing.assert_close(one.float(), b.float(), atol=3e-2, rtol=3e-2)


def test_padded_activation_rows_give_what_contiguous_rows_give(api, device, gptoss_weights):
    """Rows of x with a pitch (a slice of a wider buffer): the single launch reads them through the row stride."""
    W = gptoss_weights["tiled"]
    act = api.act(1.702, 7.0)
    pc1, pc2 = api.PrecisionConfig(b_mx_scale=W["w1s"]), api.PrecisionConfig(b_mx_scale=W["w2s"])
    g = torch.Generator().manual_seed(11)
    wide = torch.randn((24, 2880 + 64), generator=g).to(torch.bfloat16).to(device)
    x = wide[:, 8:8 + 2880]  # pitch 2944 elements, first element 16 bytes into the buffer
    logits = torch.randn((24, 128), generator=g).to(device)
    assert x.stride(0) == 2944 and api.md.one_launch_reason(x, logits, 4, W["w1"], W["b1"], W["w2"], W["b2"], pc1, pc2, act) is None
    a = api.md.moe_decode_layer(x, logits, 4, W["w1"], W["b1"], W["w2"], W["b2"], pc1, pc2, act)
    b = api.md.moe_decode_layer(x.contiguous(), logits, 4, W["w1"], W["b1"], W["w2"], W["b2"], pc1, pc2, act)
    torch.cuda.synchronize()
    assert api.md.workspace_error_word(x, logits, 4, W["w1"]) == 0
    assert torch.equal(a, b)
