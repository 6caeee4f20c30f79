"""Benchmark of the quantized MoE hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-extra]

A "step" is one forward pass of the gpt-oss-120b-shaped MXFP4 MoE FFN (config 3 of the benchmark set: 4096 tokens,
d_model 2880, 128 experts, top-4, W1 [128, 2880, 5760] and W2 [128, 2880, 2880] in MXFP4 with bf16 biases):
router -> gather-GEMM (+bias, swiglu) -> scatter-GEMM (+bias, gate weight) -> top-k combine, on synthetic
seeded inputs resident in HBM.  Prints ONE JSON line; `value` is the layer's TFLOP/s (2*R*K*N over both
GEMMs, R = routed rows).  `roofline` covers the dominant kernel (the first expert GEMM), timed live with
HIP events on the launch stream; `cpu_baseline` is the CPU oracle on a bounded sample of the same
workload; `extra` carries the FP8 (config 5), decode (config 4) and MX round-trip (config 2) figures.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_HBM_GBPS = 8000.0  # MI355X HBM3E
# HBM bytes one launch of the first expert GEMM moves at this workload, from two counter runs over this script
# (FETCH_SIZE x 2.000 + WRITE_SIZE x 1.000 KiB, factors from the 1 GiB copy of --calibrate-copy): 1368.4 MB read
# + 95.7 MB written, against 1318.3 MB of algorithmic bytes.
GEMM1_TRAFFIC_BYTES = 1.4641e9


def make_moe_weights(E, d_model, d_ff2, seed, device, n_copies=1):
    """MXFP4 expert weights (+ bf16 biases) of a gpt-oss-shaped FFN, quantised along K on the GPU."""
    from triton_amd.numerics_details.mxfp import downcast_to_mxfp
    g = torch.Generator(device="cpu").manual_seed(seed)
    out = []
    for _ in range(n_copies):
        w1q, w1s, w2q, w2s = [], [], [], []
        for _e in range(E):
            w1 = (torch.randn((d_model, d_ff2), generator=g) * 0.02).to(torch.bfloat16).to(device)
            q, s = downcast_to_mxfp(w1[None], torch.uint8, axis=1)
            w1q.append(q)
            w1s.append(s)
            w2 = (torch.randn((d_ff2 // 2, d_model), generator=g) * 0.02).to(torch.bfloat16).to(device)
            q, s = downcast_to_mxfp(w2[None], torch.uint8, axis=1)
            w2q.append(q)
            w2s.append(s)

        def cat(parts):
            # keep the K-contiguous layout the quantiser produces ([E, N, K/2] in memory)
            return torch.cat([p.transpose(1, 2) for p in parts], dim=0).contiguous().transpose(1, 2)

        b1 = (torch.randn((E, d_ff2), generator=g) * 0.01).to(torch.bfloat16).to(device)
        b2 = (torch.randn((E, d_model), generator=g) * 0.01).to(torch.bfloat16).to(device)
        out.append(dict(w1=cat(w1q), w1s=cat(w1s), w2=cat(w2q), w2s=cat(w2s), b1=b1, b2=b2))
    return out


def to_matmul_layout(weights):
    """Expert weights in the layouts `matmul` prefers on this GPU, converted once as a model loader would (the
    reference's benchmark does the same with its `make_default_matmul_mxfp4_w_layout`, bench/bench_mlp.py:40-58)."""
    from triton_kernels.tensor import FP4, convert_layout, wrap_torch_tensor
    from triton_kernels.tensor_details.layout import make_default_matmul_mxfp4_w_layout, make_default_matmul_mxfp4_w_scale_layout
    out = dict(weights)
    for name in ("w1", "w2"):
        out[name] = convert_layout(wrap_torch_tensor(weights[name], dtype=FP4), make_default_matmul_mxfp4_w_layout(mx_axis=1))
        out[name + "s"] = convert_layout(wrap_torch_tensor(weights[name + "s"]), make_default_matmul_mxfp4_w_scale_layout(mx_axis=1))
    return out


class MoeLayer:
    """The hot path composed from the drop-in API (triton_kernels names)."""

    def __init__(self, weights, k, alpha=1.702, limit=7.0):
        from triton_kernels.legacy import matmul_ogs, routing
        from triton_kernels.matmul import FnSpecs, FusedActivation, PrecisionConfig, matmul
        from triton_kernels.reduce import reduce
        from triton_kernels.swiglu import swiglu_fn
        self.routing, self.matmul, self.reduce, self.matmul_ogs = routing, matmul, reduce, matmul_ogs
        self.W = weights
        self.k = k
        self.act = FusedActivation(FnSpecs("swiglu", swiglu_fn, ("alpha", "limit"), reduction_n=2), (alpha, limit))
        self.pc1 = PrecisionConfig(b_mx_scale=weights["w1s"])
        self.pc2 = PrecisionConfig(b_mx_scale=weights["w2s"])

    def set_weights(self, weights):
        from triton_kernels.matmul import PrecisionConfig
        self.W = weights
        self.pc1 = PrecisionConfig(b_mx_scale=weights["w1s"])
        self.pc2 = PrecisionConfig(b_mx_scale=weights["w2s"])

    def __call__(self, x, logits):
        W, k = self.W, self.k
        rdata, gather, scatter = self.routing(logits, k)
        md = rdata.expt_data
        h = self.matmul(x, W["w1"], W["b1"], md, gather_indx=rdata.token_indx, precision_config=self.pc1,
                        fused_activation=self.act)
        # scatter-GEMM and top-k combine through the legacy entry point: one launch at decode shapes, GEMM + reduce otherwise
        out = self.matmul_ogs(h, W["w2"], W["b2"], rdata, scatter_indx=scatter, precision_config=self.pc2, gammas=rdata.gate_scal)
        return out, rdata


def spin_up(fn, seconds=0.15):
    """Runs `fn` for about `seconds` before any warm-up step so that the GPU's clocks have left their idle state:
    the first ~30 ms of work after an idle period run up to 20 % slower, which would otherwise be charged to
    whichever figure happens to be measured first."""
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(4):
            fn()
        torch.cuda.synchronize()


def board_state_under(fn, seconds=2.5):
    """Socket power and engine clocks as `amd-smi` reports them while `fn` keeps the GPU busy (launched in a loop from
    this thread while a second thread asks amd-smi once, a second into the load).  The published peaks assume 2.4 GHz;
    what the board sustains under a kernel at its power cap is part of reading a roofline fraction.  None when amd-smi
    is missing, fails, or a profiler is attached (its preloaded library would follow into the child process)."""
    import re
    import shutil
    import subprocess
    import threading
    if shutil.which("amd-smi") is None or "rocprof" in os.environ.get("LD_PRELOAD", ""):
        return None
    out = {}

    def ask():
        time.sleep(1.0)
        try:
            r = subprocess.run(["amd-smi", "metric", "--clock", "--power", "--json"], capture_output=True, text=True, timeout=20)
            pw = re.search(r'"socket_power":\s*\{\s*"value":\s*(\d+)', r.stdout)
            clks = re.findall(r'"gfx_\d+":\s*\{\s*"clk":\s*\{\s*"value":\s*(\d+)', r.stdout)
            if pw and clks:
                out["socket_power_w"] = int(pw.group(1))
                out["gfx_mhz_min"] = min(int(c) for c in clks)
                out["gfx_mhz_max"] = max(int(c) for c in clks)
        except Exception:  # noqa: BLE001  (a figure for the report, never a reason to fail the bench)
            pass

    th = threading.Thread(target=ask)
    th.start()
    t0 = time.perf_counter()
    while th.is_alive() and time.perf_counter() - t0 < 30.0:
        for _ in range(50):
            fn()
        torch.cuda.synchronize()
    th.join()
    return out or None


def mfma_sustained_probe(device, kind=0):
    """MFMA rate the board sustains under its power cap: a kernel of nothing but MFMA instructions on register operands
    (tk_probe_mfma; kind 0 = v_mfma_f32_32x32x16_bf16, 1 = v_mfma_f32_32x32x64_f8f6f4 on e4m3, 2 =
    v_mfma_f32_16x16x32_bf16), timed with events, with amd-smi's power and clocks under it.  The published peaks
    assume 2.4 GHz; this is the ceiling a GEMM of that class can be held against on this machine."""
    from triton_amd import _native as nt
    n_wg = 2 * torch.cuda.get_device_properties(device).multi_processor_count
    iters = 2000 if kind == 1 else 4000
    per_iter = {0: 8 * 32768.0, 1: 8 * 131072.0, 2: 16 * 16384.0}[kind]
    out = torch.zeros(n_wg * 256, dtype=torch.float32, device=device)

    def fn():
        with nt.on_device(device):
            nt.check(nt.lib().tk_probe_mfma(out.data_ptr(), n_wg, iters, kind, nt.stream_ptr(device)))

    spin_up(fn, 0.5)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(20):
        fn()
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / 20
    flops = n_wg * 4 * iters * per_iter
    peak = 5000.0 if kind == 1 else PEAK_BF16_TFLOPS
    return dict(TFLOPs=round(flops / ms / 1e9, 1), frac_of_published_peak=round(flops / ms / 1e9 / peak, 4),
                board=board_state_under(fn))


def time_steps(fn, steps, warmup):
    spin_up(fn)
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


def time_graph_steps(fn, steps, warmup):
    """`fn()` (returns a tensor) captured twice in HIP graphs; a step is one replay, the two captures in turn (a graph
    cannot overlap with its own previous launch, so replays of ONE graph would charge an idle gap to every step).
    Every capture's replay is compared with the eager result first.  Returns (ms per replayed step, ms per eager step)."""
    eager = fn().clone()
    graphs = [capture(fn) for _ in range(2)]
    for _ in range(2):  # replays with eager work in between
        for graph, out in graphs:
            graph.replay()
            torch.cuda.synchronize()
            if not torch.equal(out, eager):
                raise RuntimeError("graph replay differs from the eager result")
        fn()
    ms = time_steps(lambda i=[0]: (graphs[i[0] % 2][0].replay(), i.__setitem__(0, i[0] + 1)), steps, warmup)
    return ms, time_steps(fn, steps, warmup)


def cpu_baseline(seed=2, min_seconds=10.0):
    """CPU oracle on a bounded sample of config 3: 32 of the 128 experts and 1024 tokens (top-4), which keeps
    the ~128 routed rows per expert of the full workload; passes are repeated until `min_seconds` of CPU work."""
    from oracle import moe as omoe
    from oracle import mxfp as omx
    E, T, k, d, f2 = 32, 1024, 4, 2880, 5760
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((T, d), generator=g).to(torch.bfloat16)
    logits = torch.randn((T, E), generator=g)
    w1 = (torch.randn((E, d, f2), generator=g) * 0.02).to(torch.bfloat16)
    w2 = (torch.randn((E, f2 // 2, d), generator=g) * 0.02).to(torch.bfloat16)
    b1 = (torch.randn((E, f2), generator=g) * 0.01).to(torch.bfloat16)
    b2 = (torch.randn((E, d), generator=g) * 0.01).to(torch.bfloat16)
    w1q, w1s = omx.downcast_to_mxfp(w1, torch.uint8, axis=1)
    w2q, w2s = omx.downcast_to_mxfp(w2, torch.uint8, axis=1)
    del w1, w2
    torch.set_num_threads(min(os.cpu_count() or 1, 16))
    passes, t0 = 0, time.perf_counter()
    while True:
        omoe.moe_layer(x, logits, k, w1q, b1, w2q, b2, w1_mx_scale=w1s, w2_mx_scale=w2s)
        passes += 1
        dt = time.perf_counter() - t0
        if dt >= min_seconds or passes >= 20:
            break
    flops = 2.0 * T * k * d * (f2 + d) * passes
    return dict(value=round(flops / dt / 1e12, 4), unit="TFLOP/s", cores=torch.get_num_threads(), kind="port",
                sample=f"CPU oracle (oracle/moe.py: dequantise MXFP4, fp32 torch.matmul per expert) on {E} of 128 experts x {T} "
                f"tokens, top-{k}, same per-expert shapes; {passes} passes in {dt:.1f} s wall")


def calibration_copy(device, reps=3):
    """A copy of known size (1 GiB read + 1 GiB written per launch) so that a counter run over this script
    holds a kernel whose FETCH_SIZE / WRITE_SIZE readings can be compared with its true bytes."""
    src = torch.empty(1 << 28, dtype=torch.float32, device=device).normal_()
    dst = torch.empty_like(src)
    for _ in range(reps):
        dst.copy_(src)
    torch.cuda.synchronize()


def capture(fn):
    """Captures `fn()` (which returns a tensor) in a HIP graph after a warm-up on a side stream; returns
    (graph, output tensor that every replay overwrites)."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = fn()
    return graph, out


def bench_decode(device, steps, warmup, n_layers=10):
    """Config 4: T in {1, 4, 16, 64}, skewed router; GB/s on the expert weights actually touched.  `n_layers` layers
    with their own weight copies are captured in ONE HIP graph, as a serving loop captures a decode step over all its
    layers (gpt-oss-120b has 36); the time of a layer is the replay time / n_layers.  Ten copies rotate at least
    530 MB of touched weights at every T (the last-level cache holds 256 MB), so no layer finds its weights cached.
    Two paths are timed on the same inputs: `moe_mlp` (one launch per layer from 8 routed rows on) and the three-call
    sequence routing -> matmul_ogs -> matmul_ogs.  Every layer's output of every checked replay is compared with the
    eager result before timing."""
    from triton_kernels.moe_decode import MIN_ROWS, moe_mlp
    E, k, d, f2 = 128, 4, 2880, 5760
    copies = [to_matmul_layout(w) for w in make_moe_weights(E, d, f2, seed=3, device=device, n_copies=n_layers)]
    per_expert = d * f2 // 2 + d * f2 // 32 + (f2 // 2) * d // 2 + (f2 // 2) * d // 32
    res = {}
    g = torch.Generator().manual_seed(3)
    ebias = torch.randn((E, ), generator=g) * 1.5
    layers = [MoeLayer(w, k) for w in copies]
    for T in (1, 4, 16, 64):
        x = torch.randn((T, d), generator=g).to(torch.bfloat16).to(device)
        logits = (torch.randn((T, E), generator=g) + ebias).to(device)
        active = int((layers[0](x, logits)[1].expt_hist > 0).sum())
        gbytes = active * per_expert / 1e9

        def three_call():
            return [layer(x, logits)[0] for layer in layers]

        def one_call():
            return [moe_mlp(x, logits, k, l.W["w1"], l.W["b1"], l.W["w2"], l.W["b2"], l.pc1, l.pc2, l.act) for l in layers]

        timed = {}
        for name, fn in (("three_calls", three_call), ("moe_mlp", one_call)):
            eager = fn()
            ms_eager = time_steps(fn, steps, warmup) / n_layers
            graph, outs = capture(fn)
            for rep in range(2):  # replays with eager work in between, each compared with the eager outputs
                graph.replay()
                torch.cuda.synchronize()
                for out, ref in zip(outs, eager):
                    if not torch.equal(out, ref):
                        raise RuntimeError(f"decode T={T} ({name}): graph replay {rep} differs from the eager result")
                fn()
            ms = time_steps(graph.replay, steps, warmup) / n_layers
            timed[name] = dict(ms=round(ms, 4), ms_eager=round(ms_eager, 4), GBps=round(gbytes / (ms * 1e-3), 1),
                               frac_hbm=round(gbytes / (ms * 1e-3) / PEAK_HBM_GBPS, 4))
            if T == 16 and name == "moe_mlp":
                timed[name]["board_under_replay"] = board_state_under(graph.replay)
            del graph
        best = min(timed, key=lambda n: timed[n]["ms"])
        res[f"T{T}"] = dict(ms=timed[best]["ms"], path=best, launches_per_layer=1 if (best == "moe_mlp" and T * k >= MIN_ROWS) else 3,
                            active_experts=active, weight_GB=round(gbytes, 4), GBps=timed[best]["GBps"], frac_hbm=timed[best]["frac_hbm"],
                            layers_per_graph=n_layers, rotated_weight_GB=round(gbytes * n_layers, 3), **{n: timed[n] for n in timed})
    return res


def bench_mx(device, steps, warmup):
    """Config 2: MX quantise / dequantise of [32, 2880, 5760] bf16 along axis 1 (2.53125 B per element each way)."""
    from triton_kernels.numerics_details.mxfp import downcast_to_mxfp, upcast_from_mxfp
    w = (torch.randn((32, 2880, 5760), device=device) * 0.02).to(torch.bfloat16)
    nbytes = w.numel() * 2.53125
    ms_q = time_steps(lambda: downcast_to_mxfp(w, torch.uint8, axis=1), steps, warmup)
    q, s = downcast_to_mxfp(w, torch.uint8, axis=1)
    ms_d = time_steps(lambda: upcast_from_mxfp(q, s, torch.bfloat16, axis=1), steps, warmup)
    board = board_state_under(lambda: downcast_to_mxfp(w, torch.uint8, axis=1))
    return dict(quant_ms=round(ms_q, 4), quant_GBps=round(nbytes / ms_q / 1e6, 1), dequant_ms=round(ms_d, 4),
                dequant_GBps=round(nbytes / ms_d / 1e6, 1), frac_hbm_quant=round(nbytes / ms_q / 1e6 / PEAK_HBM_GBPS, 4),
                frac_hbm_dequant=round(nbytes / ms_d / 1e6 / PEAK_HBM_GBPS, 4), board_under_quant=board)


def bench_ragged_k(device, steps, warmup):
    """Expert weight gradient of config 3's first GEMM: dW1[e] = x_e^T @ dh_e for 128 experts, 16384 routed rows,
    [2880, 5760] per expert in bf16 (bound by writing the 4.2 GB of gradients)."""
    from triton_kernels.matmul import matmul
    from triton_kernels.tensor import make_ragged_tensor_metadata
    E, R, d, f2 = 128, 16384, 2880, 5760
    g = torch.Generator().manual_seed(6)
    cuts = torch.sort(torch.randint(0, R + 1, (E - 1, ), generator=g)).values
    sizes = torch.diff(torch.cat([torch.tensor([0]), cuts, torch.tensor([R])])).to(torch.int32).to(device)
    md = make_ragged_tensor_metadata(sizes, R)
    x = torch.randn((R, d), device=device).to(torch.bfloat16)
    dh = torch.randn((R, f2), device=device).to(torch.bfloat16)
    out = torch.empty((E, d, f2), dtype=torch.bfloat16, device=device)
    ms = time_steps(lambda: matmul(x.t(), dh, None, a_ragged_metadata=md, b_ragged_metadata=md, c=out), steps, warmup)
    nbytes = out.numel() * 2 + x.numel() * 2 + dh.numel() * 2
    flops = 2.0 * R * d * f2
    return dict(ms=round(ms, 4), GBps=round(nbytes / ms / 1e6, 1), frac_hbm=round(nbytes / ms / 1e6 / PEAK_HBM_GBPS, 4),
                TFLOPs=round(flops / ms / 1e9, 1))


def bench_fp8(device, steps, warmup):
    """Config 5 (Mixtral-style FP8) at full size: 8192 tokens, top-2 of 8 experts, W1 [8, 4096, 28672] and
    W2 [8, 14336, 4096] in e4m3 with per-output-channel fp32 scales, activations quantised per token to e4m3
    before each GEMM.  One step = router, quantise, GEMM1 + swiglu, quantise, GEMM2 * gate, combine."""
    from triton_kernels.legacy import routing
    from triton_kernels.matmul import FnSpecs, FusedActivation, PrecisionConfig, matmul
    from triton_kernels.numerics_details.rowwise_fp8 import quantize_fp8_rowwise
    from triton_kernels.reduce import reduce
    from triton_kernels.swiglu import swiglu_fn
    T, d, E, k, f2 = 8192, 4096, 8, 2, 28672
    torch.manual_seed(4)
    x = torch.randn((T, d), device=device).to(torch.bfloat16)
    logits = torch.randn((T, E), device=device)

    def qw(kdim, ndim):  # K-major e4m3 weights [E, K, N] (stride 1 along K) and their column scales [E, N]
        q = torch.empty((E, ndim, kdim), dtype=torch.float8_e4m3fn, device=device)
        s = torch.empty((E, ndim), dtype=torch.float32, device=device)
        for e in range(E):
            w = torch.randn((ndim, kdim), device=device) * 0.02
            s[e] = w.abs().amax(dim=1) / 448.0
            q[e] = (w / s[e][:, None]).clamp(-448, 448).to(torch.float8_e4m3fn)
        return q.transpose(1, 2), s

    from triton_kernels.tensor import convert_layout, wrap_torch_tensor
    from triton_kernels.tensor_details.layout import make_default_matmul_fp8_w_layout
    w1, s1 = qw(d, f2)
    w2, s2 = qw(f2 // 2, d)
    # converted once, as a model loader would, to the layout `matmul` prefers for e4m3 weights on this GPU
    w1 = convert_layout(wrap_torch_tensor(w1), make_default_matmul_fp8_w_layout())
    w2 = convert_layout(wrap_torch_tensor(w2), make_default_matmul_fp8_w_layout())
    act = FusedActivation(FnSpecs("swiglu", swiglu_fn, ("alpha", "limit"), reduction_n=2), (1.702, 7.0))

    def step():
        rdata, _, scatter = routing(logits, k)
        xq, sx = quantize_fp8_rowwise(x)
        h = matmul(xq, w1, None, rdata.expt_data, gather_indx=rdata.token_indx, fused_activation=act,
                   precision_config=PrecisionConfig(a_mx_tensor_scale=sx, b_mx_tensor_scale=s1, out_dtype=torch.bfloat16))
        hq, sh = quantize_fp8_rowwise(h)
        y = matmul(hq, w2, None, rdata.expt_data, scatter_indx=scatter.dst_indx, gammas=rdata.gate_scal,
                   precision_config=PrecisionConfig(a_mx_tensor_scale=sh, b_mx_tensor_scale=s2, out_dtype=torch.bfloat16))
        return reduce(y.view(T, k, -1), dim=1)[0]

    ms, ms_eager = time_graph_steps(step, steps, warmup)
    board = board_state_under(step)
    flops = 2.0 * T * k * (d * f2 + (f2 // 2) * d)
    return dict(ms_per_step=round(ms, 4), ms_per_step_eager=round(ms_eager, 4), step_mode="hip_graph_replay",
                TFLOPs=round(flops / ms / 1e9, 1), mfma_class="fp8",
                frac_mfma_fp8=round(flops / ms / 1e9 / 5000.0, 4), board_under_step=board,
                mfma_sustained_probe=mfma_sustained_probe(device, kind=1))


def bench_scaled_mfma(device, weights, x, logits, k, steps, warmup):
    """Config 3's shapes on the scaled-MFMA path: the activations are MX-quantised (e4m3 + one e8m0 scale per 32 along
    K) and multiplied with the MXFP4 weights by v_mfma_scale_f32_32x32x64_f8f6f4, both operands in their storage
    formats; the first GEMM's epilogue quantises its fp32 accumulator to MXFP8 for the second.  Not the headline:
    config 3 states bf16 activations, and this path is checked against an oracle fed the same quantised activations.
    One step = router, quantise x, GEMM1 (+bias, swiglu, MX output), GEMM2 (+bias, gate weight, top-k combine)."""
    from triton_kernels.legacy import matmul_ogs, routing
    from triton_kernels.matmul import Epilogue, FnName, FnSpecs, FusedActivation, PrecisionConfig, matmul
    from triton_kernels.numerics_details.mxfp import downcast_to_mxfp, quantize_mxfp8_fn
    from triton_kernels.swiglu import swiglu_fn
    T, d = x.shape
    W = weights
    f2 = W["b1"].shape[-1]
    act = FusedActivation(FnSpecs("swiglu", swiglu_fn, ("alpha", "limit"), reduction_n=2), (1.702, 7.0))
    epi = Epilogue(FnSpecs(FnName.QUANTIZE_MXFP8.name, quantize_mxfp8_fn, (), ()), tuple(), tuple(), effective_itemsize=1.0)
    h_scale = torch.empty((T * k, (f2 // 2) // 32), dtype=torch.uint8, device=device)

    def step():
        rdata, _, scatter = routing(logits, k)
        xq, xs = downcast_to_mxfp(x, torch.float8_e4m3fn, axis=-1)
        h = matmul(xq, W["w1"], W["b1"], rdata.expt_data, gather_indx=rdata.token_indx, fused_activation=act, epilogue=epi,
                   precision_config=PrecisionConfig(a_mx_scale=xs, b_mx_scale=W["w1s"], c_mx_scale=h_scale, out_dtype=torch.float8_e4m3fn))
        # (the legacy entry point sums the k rows of a token at the end of the scatter-GEMM's launch, as in the headline step)
        return matmul_ogs(h, W["w2"], W["b2"], rdata, scatter_indx=scatter, gammas=rdata.gate_scal,
                          precision_config=PrecisionConfig(a_mx_scale=h_scale, b_mx_scale=W["w2s"], out_dtype=torch.bfloat16))

    ms, ms_eager = time_graph_steps(step, steps, warmup)
    board = board_state_under(step)
    flops = 2.0 * T * k * (d * f2 + (f2 // 2) * d)
    # algorithmic bytes with one-byte activations: x_q + scales, W1, h_q twice, W2, y twice, out
    R = T * k
    E = W["b1"].shape[0]
    nbytes = (R * d * 33 / 32 + E * (d * f2 * 17 / 32 + f2 * 2) + 2 * R * (f2 // 2) * 33 / 32 + E * ((f2 // 2) * d * 17 / 32 + d * 2) + 2 * R * d * 2 + T * d * 2)
    t_roof_ms = max(flops / 5.0e15, nbytes / (PEAK_HBM_GBPS * 1e9)) * 1e3
    return dict(ms_per_step=round(ms, 4), ms_per_step_eager=round(ms_eager, 4), step_mode="hip_graph_replay", TFLOPs=round(flops / ms / 1e9, 1),
                mfma_class="fp8 (MXFP8 x MXFP4, scaled MFMA)",
                frac_mfma_fp8=round(flops / ms / 1e9 / 5000.0, 4), t_roof_ms=round(t_roof_ms, 4), frac=round(t_roof_ms / ms, 4),
                bound="hbm" if nbytes / (PEAK_HBM_GBPS * 1e9) > flops / 5.0e15 else "mfma", board_under_step=board)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU oracle baseline")
    ap.add_argument("--no-extra", action="store_true", help="skip the decode and MX round-trip figures")
    ap.add_argument("--no-board-state", action="store_true", help="do not sample amd-smi (power, clocks) under the dominant kernel")
    ap.add_argument("--calibrate-copy", action="store_true", help="also run a 1 GiB device copy (reference kernel for counter runs)")
    ap.add_argument("--only", choices=["mx", "decode", "fp8", "ragged_k"],
                    help="run one of the side workloads alone and print its figures (for profiler runs)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus must be 1 (with more GPUs the layer shards by expert, which is not built)",
              file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: needs a GPU", file=sys.stderr)
        sys.exit(2)
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    if args.only:
        if args.calibrate_copy:
            calibration_copy(device)
        fn = {"mx": bench_mx, "decode": bench_decode, "fp8": bench_fp8, "ragged_k": bench_ragged_k}[args.only]
        print(json.dumps({args.only: fn(device, args.steps, args.warmup)}))
        return
    T, E, k, d, f2 = 4096, 128, 4, 2880, 5760
    g = torch.Generator().manual_seed(2)
    x = torch.randn((T, d), generator=g).to(torch.bfloat16).to(device)
    logits = torch.randn((T, E), generator=g).to(device)
    weights = to_matmul_layout(make_moe_weights(E, d, f2, seed=2, device=device)[0])
    layer = MoeLayer(weights, k)
    if args.calibrate_copy:
        calibration_copy(device)

    # The whole layer (router, two GEMMs, combine) is captured in a HIP graph and a step is one replay, as a serving
    # loop would run it: the eager Python path costs about as much host time per step as the GPU needs.  Two
    # captures are replayed in turn: a graph cannot overlap with its own previous launch, so back-to-back replays
    # of ONE graph would add an idle gap per step that a model, which runs other layers in between, never sees.
    eager_out, rdata = layer(x, logits)
    graphs = [capture(lambda: layer(x, logits)[0]) for _ in range(2)]
    for _ in range(2):  # replays with eager work in between, each compared with the eager output
        for graph, graph_out in graphs:
            graph.replay()
            torch.cuda.synchronize()
            if not torch.equal(graph_out, eager_out):
                raise RuntimeError("graph replay differs from the eager result")
        layer(x, logits)
    spin_up(lambda: (graphs[0][0].replay(), graphs[1][0].replay()))
    for i in range(args.warmup):
        graphs[i % 2][0].replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        graphs[i % 2][0].replay()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    # the dominant kernel alone, same inputs, HIP events on the launch stream around args.steps launches
    md = rdata.expt_data

    def gemm1():
        return layer.matmul(x, layer.W["w1"], layer.W["b1"], md, gather_indx=rdata.token_indx, precision_config=layer.pc1,
                            fused_activation=layer.act)

    spin_up(gemm1)
    for _ in range(args.warmup):
        gemm1()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(args.steps):
        gemm1()
    e1.record()
    torch.cuda.synchronize()
    gemm1_ms = e0.elapsed_time(e1) / args.steps
    board = None if args.no_board_state else board_state_under(gemm1)
    ms_eager = time_steps(lambda: layer(x, logits), args.steps, args.warmup)
    R = T * k
    flops1 = 2.0 * R * d * f2
    flops = flops1 + 2.0 * R * (f2 // 2) * d
    achieved = flops1 / (gemm1_ms * 1e-3) / 1e12
    rec = {
        "metric": "MoE layer TFLOP/s + HBM GB/s (% roofline), gpt-oss-120b shape, 1 MI355X",
        "value": round(flops / (ms * 1e-3) / 1e12, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms, 4),
        "ms_per_step_eager": round(ms_eager, 4),
        "step_mode": "hip_graph_replay",
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16 MFMA, fp32 accumulate (mxfp4 weights dequantised in registers)",
        "data": "synthetic",
        "config": {"workload": "gpt-oss-120b-shaped MXFP4 MoE FFN prefill (BASELINE config 3)", "tokens": T, "d_model": d,
                   "experts": E, "top_k": k, "w1": [E, d, f2], "w2": [E, f2 // 2, d]},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK_BF16_TFLOPS, 4), "traffic": GEMM1_TRAFFIC_BYTES,
                     "kernel": "moe_gemm_mxn_kernel (gather-GEMM, tiled MXFP4 W1, bias, swiglu)", "kernel_ms": round(gemm1_ms, 4),
                     "board_under_kernel": board,
                     "mfma_sustained_probe": None if args.no_board_state else mfma_sustained_probe(device),
                     "mfma_sustained_probe_16x16x32": None if args.no_board_state else mfma_sustained_probe(device, kind=2)},
    }
    # layer-level roofline: t_roof = max(flops / bf16 peak, algorithmic bytes / HBM peak)
    layer_bytes = 2.19e9
    t_roof_ms = max(flops / (PEAK_BF16_TFLOPS * 1e12), layer_bytes / (PEAK_HBM_GBPS * 1e9)) * 1e3
    rec["layer_roofline"] = {"t_roof_ms": round(t_roof_ms, 4), "frac": round(t_roof_ms / ms, 4),
                             "GBps": round(layer_bytes / (ms * 1e-3) / 1e9, 1)}
    if not args.no_extra:
        rec["extra"] = {"scaled_mfma_config3": bench_scaled_mfma(device, weights, x, logits, k, args.steps, args.warmup),
                        "fp8_config5": bench_fp8(device, max(5, args.steps // 2), 2),
                        "decode_config4": bench_decode(device, max(5, args.steps), args.warmup),
                        "mx_round_trip_config2": bench_mx(device, max(5, args.steps), args.warmup)}
    if not args.no_cpu:
        rec["cpu_baseline"] = cpu_baseline()
    print(json.dumps(rec))


if __name__ == "__main__":
    main()
