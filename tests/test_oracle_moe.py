"""Pins the GEMM / swiglu / combine oracle (oracle/moe.py) by what the mathematics fixes: reduction to a
dense library GEMM, permutation equivariance, linearity, closed forms at hand-computable points and a
pure-Python brute force on a tiny case.  CPU only."""
import math

import numpy as np
import pytest
import torch

from oracle import moe as omoe
from oracle import mxfp as omx
from oracle import routing as ort


def _case(seed, T=24, K=32, N=20, E=5, k=2, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((T, K), generator=g).to(dtype)
    w = (torch.randn((E, K, N), generator=g) * 0.25).to(dtype)
    b = torch.randn((E, N), generator=g).to(dtype)
    r = ort.routing(torch.randn((T, E), generator=g), k)
    return x, w, b, r


def test_single_expert_is_a_dense_gemm():
    x, w, b, _ = _case(0, E=1, k=1)
    y = omoe.matmul(x, w, b, torch.tensor([x.shape[0]]))
    ref = (x.double() @ w[0].double() + b[0].double())
    assert torch.allclose(y.double(), ref, rtol=1e-2, atol=1e-2)
    assert torch.equal(y, omoe.matmul(x, w[0], b[0]))  # 2-D weight path


def test_brute_force_tiny():
    # every output element recomputed with Python floats, including gather, bias, gate and scatter
    x, w, b, r = _case(1, T=6, K=8, N=4, E=3, k=2, dtype=torch.float32)
    y = omoe.matmul(x, w, b, r.meta.col_sum, gather_indx=r.gather_indx, scatter_indx=r.scatter_indx, gammas=r.gammas)
    flat_e = r.indx.reshape(-1).tolist()
    for pos in range(12):  # flat position t*k+j is the destination row
        t, e = pos // 2, flat_e[pos]
        gate = float(r.vals.reshape(-1)[pos])
        for n in range(4):
            acc = sum(float(x[t, kk]) * float(w[e, kk, n]) for kk in range(8)) + float(b[e, n])
            assert abs(float(y[pos, n]) - acc * gate) < 1e-5


def test_token_permutation_equivariance():
    x, w, b, _ = _case(2)
    g = torch.Generator().manual_seed(5)
    logits = torch.randn((x.shape[0], w.shape[0]), generator=g)
    perm = torch.randperm(x.shape[0], generator=g)
    w2 = (torch.randn((w.shape[0], w.shape[2] // 2, 16), generator=g) * 0.3).to(torch.bfloat16)
    out = omoe.moe_layer(x, logits, 2, w, b, w2, None)
    out_p = omoe.moe_layer(x[perm], logits[perm], 2, w, b, w2, None)
    assert torch.equal(out[perm], out_p)


def test_unit_gammas_zero_bias_is_plain_grouped_gemm():
    x, w, _, r = _case(3)
    ones = torch.ones_like(r.gammas)
    a = omoe.matmul(x, w, None, r.meta.col_sum, gather_indx=r.gather_indx)
    c = omoe.matmul(x, w, torch.zeros((w.shape[0], w.shape[2])), r.meta.col_sum, gather_indx=r.gather_indx, gammas=ones)
    assert torch.equal(a, c)
    # power-of-two gate weights commute with the bf16 rounding
    two = omoe.matmul(x, w, None, r.meta.col_sum, gather_indx=r.gather_indx, gammas=ones * 2)
    assert torch.equal(two.float(), a.float() * 2)


def test_scatter_is_the_inverse_of_the_sort():
    x, w, _, r = _case(4)
    y_sorted = omoe.matmul(x, w, None, r.meta.col_sum, gather_indx=r.gather_indx)
    y_tok = omoe.matmul(x, w, None, r.meta.col_sum, gather_indx=r.gather_indx, scatter_indx=r.scatter_indx)
    assert torch.equal(y_tok[r.scatter_indx.long()], y_sorted)
    assert torch.equal(y_tok, y_sorted[r.meta.row_sorted_indx.long()])


def test_mx_weights_equal_dense_weights_after_dequant():
    g = torch.Generator().manual_seed(6)
    x = torch.randn((16, 64), generator=g).to(torch.bfloat16)
    w = (torch.randn((2, 64, 8), generator=g) * 0.1).to(torch.bfloat16)
    q, s = omx.downcast_to_mxfp(w, torch.uint8, axis=1)
    wd = omx.upcast_from_mxfp(q, s, torch.bfloat16, axis=1)
    sizes = torch.tensor([10, 6])
    assert torch.equal(omoe.matmul(x, q, None, sizes, w_mx_scale=s), omoe.matmul(x, wd, None, sizes))


def test_row_and_column_scales_are_a_dequantisation():
    g = torch.Generator().manual_seed(7)
    x = torch.randn((12, 32), generator=g).to(torch.bfloat16)
    xq, sx = omoe.quantize_fp8_rowwise(x)
    # the scale maps the row maximum to +-448 and the round trip stays within half an e4m3 step (2^-4 relative)
    assert torch.all(xq.float().abs().amax(dim=1) == 448.0)
    assert torch.allclose(xq.float() * sx[:, None], x.float(), rtol=2**-4, atol=float(sx.max()) * 2**-9)
    w = torch.randn((1, 32, 8), generator=g)
    sw = torch.rand((1, 8), generator=g) + 0.5
    y = omoe.matmul(xq, w, None, torch.tensor([12]), x_row_scale=sx, w_col_scale=sw, out_dtype=torch.float32)
    ref = (xq.float() * sx[:, None]) @ (w[0] * sw[0][None, :])
    assert torch.allclose(y, ref, rtol=1e-5, atol=1e-6)
    z, sz = omoe.quantize_fp8_rowwise(torch.zeros((1, 32), dtype=torch.bfloat16))
    assert sz.item() == 1.0 and not z.float().any()


def test_swiglu_hand_values():
    # swiglu.py:89-100 with alpha = 1, limit = 2 on points computed by hand: s = g*sigmoid(g), out = s*(l+1)
    a = torch.tensor([[0.0, 5.0, 1.0, 1.0, 3.0, -4.0, -1.0, 0.5]], dtype=torch.float32)
    out = omoe.swiglu(a, 1.0, 2.0)
    sig = lambda v: 1.0 / (1.0 + math.exp(-v))
    want = [0.0, 1.0 * sig(1.0) * 2.0, 2.0 * sig(2.0) * (-2.0 + 1.0), -1.0 * sig(-1.0) * 1.5]
    assert np.allclose(out[0].tolist(), want, rtol=1e-6, atol=1e-7)
    # no limit: nothing is clamped
    out = omoe.swiglu(a, 1.0, None)
    assert np.isclose(out[0, 2].item(), 3.0 * sig(3.0) * (-3.0))
    # the gate is clamped from above only (a very negative gate keeps its value)
    out = omoe.swiglu(torch.tensor([[-30.0, 1.0]]), 1.702, 7.0)
    assert abs(out.item()) < 1e-18


def test_swiglu_reference_test_shape():
    # tests/test_swiglu.py:25-32 shape and parameters; checked against a float64 evaluation
    g = torch.Generator().manual_seed(8)
    a = torch.randn((1311, 4352), generator=g)
    for limit in (1e-2, 10.0):
        out = omoe.swiglu(a, 0.5, limit)
        gg = a[:, ::2].double().clamp(max=limit)
        ll = a[:, 1::2].double().clamp(-limit, limit)
        ref = gg / (1 + torch.exp(-0.5 * gg)) * (ll + 1)
        assert out.shape == (1311, 2176) and torch.allclose(out.double(), ref, rtol=1e-5, atol=1e-7)


def test_reduce_k_closed_form():
    y = torch.arange(24, dtype=torch.float32).reshape(6, 4).to(torch.bfloat16)
    out = omoe.reduce_k(y, 3)
    assert out.tolist() == [[12.0, 15.0, 18.0, 21.0], [48.0, 51.0, 54.0, 57.0]]
    mask = torch.tensor([[[1], [0], [1]], [[0], [0], [0]]])
    out = omoe.reduce_k(y, 3, mask=mask.expand(2, 3, 4))
    assert out.tolist() == [[8.0, 10.0, 12.0, 14.0], [0.0] * 4]


def test_layer_equals_dense_sum_over_selected_experts():
    # the routed layer equals, token by token, sum_j gate_j * FFN_{e_j}(x_t) evaluated densely in float64
    x, w1, b1, _ = _case(10, T=10, K=16, N=12, E=4, k=2, dtype=torch.float32)
    g = torch.Generator().manual_seed(11)
    w2 = torch.randn((4, 6, 16), generator=g) * 0.3
    b2 = torch.randn((4, 16), generator=g)
    logits = torch.randn((10, 4), generator=g)
    out = omoe.moe_layer(x, logits, 2, w1, b1, w2, b2, swiglu_alpha=1.3, swiglu_limit=5.0)
    vals, indx, _ = ort.topk(logits, 2)
    for t in range(10):
        acc = torch.zeros(16, dtype=torch.float64)
        for j in range(2):
            e = int(indx[t, j])
            h = x[t].double() @ w1[e].double() + b1[e].double()
            gg, ll = h[::2].clamp(max=5.0), h[1::2].clamp(-5.0, 5.0)
            a = gg * torch.sigmoid(1.3 * gg) * (ll + 1)
            acc += float(vals[t, j]) * (a @ w2[e].double() + b2[e].double())
        assert torch.allclose(out[t].double(), acc, rtol=1e-4, atol=1e-5)


def test_layer_gate_against_float64():
    """How strict the rtol 2e-2 / atol 1e-2 gate is at the LAYER level: the oracle (bf16-rounded intermediates, as the
    reference materialises them) against an exact float64 evaluation of the same layer on gpt-oss-shaped experts
    (d 2880, W1 [E, 2880, 5760], W2 [E, 2880, 2880], top-4).  Almost every element is far inside the gate, but not
    all: the k partial rows are rounded to bf16 before they are summed, so where they cancel the sum carries an
    absolute error of a partial row's ulp.  This is why the layer-level GPU tests allow a small share of elements
    outside the gate (LAYER_GATE_SLACK in tests/test_gpu_moe_layer.py) while single GEMMs get none."""
    g = torch.Generator().manual_seed(2)
    E, k, d, f2, T = 8, 4, 2880, 5760, 256
    x = torch.randn((T, d), generator=g).to(torch.bfloat16)
    logits = torch.randn((T, E), generator=g)
    # synthetic MXFP4 weights: uniform e2m1 codes with scale 2^-7 have rms 0.023, like N(0, 0.02) weights
    w1q = torch.randint(0, 256, (E, f2, d // 2), generator=g, dtype=torch.uint8).transpose(1, 2)
    w2q = torch.randint(0, 256, (E, d, f2 // 4), generator=g, dtype=torch.uint8).transpose(1, 2)
    w1s = torch.full((E, f2, d // 32), 120, dtype=torch.uint8).transpose(1, 2)
    w2s = torch.full((E, d, f2 // 64), 120, dtype=torch.uint8).transpose(1, 2)
    b1 = (torch.randn((E, f2), generator=g) * 0.01).to(torch.bfloat16)
    b2 = (torch.randn((E, d), generator=g) * 0.01).to(torch.bfloat16)
    out = omoe.moe_layer(x, logits, k, w1q, b1, w2q, b2, w1_mx_scale=w1s, w2_mx_scale=w2s)
    W1 = omoe.dequant_weight(w1q, w1s).double()
    W2 = omoe.dequant_weight(w2q, w2s).double()
    vals, indx, _ = ort.topk(logits, k)
    exact = torch.zeros((T, d), dtype=torch.float64)
    for e in range(E):
        tj = (indx == e).nonzero()
        t, j = tj[:, 0], tj[:, 1]
        h = x[t].double() @ W1[e] + b1[e].double()
        gg, ll = h[:, ::2].clamp(max=7.0), h[:, 1::2].clamp(-7.0, 7.0)
        a = gg * torch.sigmoid(1.702 * gg) * (ll + 1)
        exact.index_add_(0, t, (a @ W2[e] + b2[e].double()) * vals[t, j].double()[:, None])
    err = (out.double() - exact).abs()
    outside = err > (1e-2 + 2e-2 * exact.abs())
    frac = float(outside.double().mean())
    print(f"oracle vs float64: worst |err| {float(err.max()):.4g}, median {float(err.median()):.4g}, output rms "
          f"{float(exact.pow(2).mean().sqrt()):.4g}, outside the gate {int(outside.sum())} of {outside.numel()}")
    # the worst element sits at the gate (an ulp of a partial row) while the typical one is far inside it
    assert float(err.max()) > 5e-3, f"worst error {float(err.max()):.3g}: the gate would be loose here"
    assert float(err.median()) < 0.2 * float(err.max())
    # the oracle itself is outside the gate for about two elements in 100 000 here: a zero-tolerance gate at layer
    # level would reject the oracle; the GPU tests allow 1e-4
    assert int(outside.sum()) > 0 and frac <= 1e-4, f"{frac:.3g} of the oracle's own elements are outside the gate"
    # rounding the exact result once to bf16 is always inside the gate: the slack comes from the partial rows
    once = (exact.to(torch.bfloat16).double() - exact).abs() > (1e-2 + 2e-2 * exact.abs())
    assert int(once.sum()) == 0


def test_ragged_k_is_a_masked_dense_product():
    """Pins `matmul_ragged_k` by mathematics: with both operands' slices laid end to end at their offsets,
    out[e][m][n] = sum_k a[m, ao_e + k] b[bo_e + k, n] is a float64 einsum over a 0/1 selector per slice; the offsets
    of the two operands differ (one side padded), one slice is empty, and out[e] summed over e with equal offsets is
    the plain product a @ b."""
    g = torch.Generator().manual_seed(5)
    sizes = torch.tensor([5, 0, 17, 32, 1], dtype=torch.int32)
    a_offs = torch.tensor([0, 8, 8, 32, 64], dtype=torch.int32)   # padded to multiples of 8
    b_offs = torch.tensor([0, 5, 5, 22, 54], dtype=torch.int32)   # dense
    M, N = 9, 13
    a = torch.randn((M, 72), generator=g).to(torch.bfloat16)
    b = torch.randn((55, N), generator=g).to(torch.bfloat16)
    got = omoe.matmul_ragged_k(a, b, sizes, a_offs, b_offs, out_dtype=torch.float32)
    for e in range(5):
        want = torch.zeros((M, N), dtype=torch.float64)
        for kk in range(int(sizes[e])):
            want += torch.outer(a[:, int(a_offs[e]) + kk].double(), b[int(b_offs[e]) + kk, :].double())
        torch.testing.assert_close(got[e].double(), want, rtol=1e-5, atol=1e-5)
    assert got[1].abs().max() == 0
    # equal dense offsets: the slices partition K, so the outputs sum to the full product
    got2 = omoe.matmul_ragged_k(a[:, :55], b, sizes, b_offs, b_offs, out_dtype=torch.float32)
    torch.testing.assert_close(got2.sum(0).double(), a[:, :55].double() @ b.double(), rtol=1e-5, atol=1e-4)
    # a transposed (strided) operand is the same problem
    got3 = omoe.matmul_ragged_k(a.t().contiguous().t(), b, sizes, a_offs, b_offs, out_dtype=torch.float32)
    assert torch.equal(got3, got)


def test_matmul_betas_out_alpha_acc_in_against_float64():
    """The less common epilogue options in the kernel's order (matmul_details/_matmul.py:547-559,581-591):
    y = ((x @ w + bias * beta) * alpha) * gamma + acc_in, checked element-wise against float64 on a small ragged case;
    a swapped order (alpha applied to the accumulated input, beta applied to the product) would miss by far more."""
    g = torch.Generator().manual_seed(5)
    M, K, N, E = 37, 24, 20, 3
    sizes = torch.tensor([10, 0, 27], dtype=torch.int32)
    x = torch.randn((M, K), generator=g)
    w = torch.randn((E, K, N), generator=g)
    bias = torch.randn((E, N), generator=g)
    betas, gammas = torch.rand((M, ), generator=g) + 0.5, torch.rand((M, ), generator=g) + 0.5
    acc_in = torch.randn((M, N), generator=g)
    alpha = 0.37
    got = omoe.matmul(x, w, bias, sizes, gammas=gammas, betas=betas, out_alpha=alpha, acc_in=acc_in, out_dtype=torch.float32)
    ref = torch.zeros((M, N), dtype=torch.float64)
    lo = 0
    for e, n in enumerate(sizes.tolist()):
        hi = lo + n
        t = x[lo:hi].double() @ w[e].double() + bias[e].double()[None, :] * betas[lo:hi].double()[:, None]
        ref[lo:hi] = t * alpha * gammas[lo:hi].double()[:, None] + acc_in[lo:hi].double()
        lo = hi
    assert float((got.double() - ref).abs().max()) < 1e-4
    wrong = omoe.matmul(x, w, bias, sizes, gammas=gammas, betas=betas, out_dtype=torch.float32) + alpha * acc_in
    assert float((wrong.double() - ref).abs().max()) > 1e-2
