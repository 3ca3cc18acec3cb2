#!/usr/bin/env python3
"""Benchmark of the ConvBlock hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-sweep] [--no-kernels] [--no-configs]
                    [--no-torch-gpu]

A step is one ConvBlock forward + backward on the headline workload
(ConvBlock(128, kernel_size=13), bf16, x [32,56,56,128], seeded synthetic data, inputs resident in HBM),
replayed as one HIP graph.  Consecutive steps run on different sets of buffers (inputs, saved activations,
gradients) that together exceed the 256 MB Infinity Cache, so that a step finds its inputs in HBM and not in
the cache: that is the headline `value` ("rotated").  The same step replayed on one set of buffers (inputs
cache-warm) is reported beside it as `warm_ms_per_step`.

Prints ONE JSON line: ms per step, the forward-only times, the k = 9/13/17 sweep, rows for the other
workloads (stand-alone depthwise conv at C = 128; the fp16 high-resolution block; the ragged block in fp32 and
bf16), the per-kernel timings (HIP events on the launch stream) with the roofline record of the longest launch
of the step, the same op set through torch's own GPU operators, and the PyTorch-CPU baseline.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

# How the HIP runtime submits a graph replay (a host-side setting of ROCm's runtime, read when it loads; it changes no
# kernel and no result): with this image's default, every replay of a captured step costs about 4 us more on the GPU
# than with the kernels submitted as ordinary dispatches.  Set before torch loads the runtime; a value given in the
# environment wins.  The line reports the setting, and the step's time under the runtime's default beside `value`.
GRAPH_SUBMIT_ENV = "DEBUG_CLR_GRAPH_PACKET_CAPTURE"
os.environ.setdefault(GRAPH_SUBMIT_ENV, "0")

import torch  # noqa: E402

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12     # B/s, MI355X published
MFMA_PEAK = 2.5e15    # dense bf16/fp16 matrix FLOP/s, MI355X published
FP32_PEAK = 157.3e12  # fp32 vector FLOP/s, MI355X published
MALL_BYTES = 256e6    # Infinity Cache

WORKLOAD = dict(B=32, H=56, W=56, D=128, k=13, dtype="bf16")
DTYPES = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}


# ------------------------------------------------------------------------------------------------
# Algorithmic bytes and flops

def block_alg_bytes(B, H, W, D, k, esize, scales=(1.0, 0.5)):
    """Compulsory HBM traffic of the unfused op graph (each op reads each input once and writes
    each output once), forward and forward+backward, in bytes."""
    I, G = D // 2, D // 4
    N = B * H * W
    n = B * int(H * scales[1]) * int(W * scales[1])
    fwd = (N * D + N * I) + 2 * N * I + 1.5 * N * I + (N * I + n * I) + 2 * n * I + 1.5 * n * I + (n * G + N * G) \
        + 4 * N * G + (2 * N * G + N * D) + N * D + 2 * N * D
    bwd = N * D + 2 * (N * D + 2 * N * G) + (N * G + n * G) + 2.5 * n * I + 2 * n * I + 2 * n * I + (n * I + N * I) \
        + 2.5 * N * I + 2 * N * I + 2 * N * I + 3 * N * I + 2 * (N * I + N * D) + 2 * N * D
    params = D * I + 2 * k * k * I + 2 * G * D + D + D * D + D
    return esize * (fwd + params), esize * (fwd + bwd + 3 * params)


def conv_issue(k):
    """Multiply-adds the matrix-core depthwise kernels issue per output (forward / input gradient: a 4 x 4 patch
    against its (k+3)^2 window, 32 window positions per instruction) and per position (weight gradient: 16 x 16
    taps per instruction), against the k*k that fall on a real tap."""
    ic = k + 3
    icb = (ic + 7) // 8
    nm = (ic * icb + 3) // 4
    return dict(fwd=nm * 32, wgrad=256 if k <= 14 else None, useful=k * k)


# ------------------------------------------------------------------------------------------------
# Timing

def time_gpu(fn, steps, warmup):
    """Wall time per call of fn over `steps` calls, bracketed by device synchronisation."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def rotate(replayers):
    """One callable that replays the next of `replayers` on every call."""
    state = {"i": 0}

    def fn():
        replayers[state["i"] % len(replayers)]()
        state["i"] += 1

    return fn


def time_kernel_events(launch, nbuf, iters=24, reps=4):
    """Average duration of one launch.  `iters` launches (launch(i) uses buffer set i % nbuf, so that
    consecutive launches do not hit in the Infinity Cache) are captured into a HIP graph, and the
    replays are bracketed by HIP events recorded on the stream the graph runs on, so the figure is GPU
    time per launch, free of the host's per-call overhead."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for i in range(min(nbuf, 3)):
            launch(i)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for i in range(iters):
            launch(i % nbuf)
    graph.replay()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(reps):
        graph.replay()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) * 1e-3 / (iters * reps)


# ------------------------------------------------------------------------------------------------
# Block workloads

def make_block(D, k, dtype, seed=0):
    import pyramid_dwconv

    torch.manual_seed(seed)
    return pyramid_dwconv.ConvBlock(dim=D, kernel_size=k).to(dtype).cuda()


def make_inputs(shape, dtype, dist, seed):
    gen = torch.Generator().manual_seed(seed)
    if dist == "uniform":   # U(-2, 2)
        x = (torch.rand(*shape, generator=gen) * 4 - 2)
    else:
        x = torch.randn(*shape, generator=gen)
    g = torch.randn(*shape, generator=gen)
    return x.to(dtype).cuda(), g.to(dtype).cuda()


def n_sets(B, H, W, D, k, esize):
    """Buffer sets to rotate over: their inputs and saved activations (about half of the forward+backward
    algorithmic bytes each) together exceed twice the Infinity Cache; between 3 and 24."""
    per_set = 0.5 * block_alg_bytes(B, H, W, D, k, esize)[1]
    return int(min(24, max(3, math.ceil(2 * MALL_BYTES / per_set))))


def measure_block(m, shape, dtype, dist, steps, warmup, with_forward=True):
    """ms per forward+backward step (rotated over buffer sets / one warm set) and per inference forward."""
    from pyramidconvblock_amd.graphs import GraphedForward, GraphedStep

    B, H, W, D = shape
    k = m.gates[0].conv_spatial.weight.shape[0]
    es = torch.empty((), dtype=dtype).element_size()
    ns = n_sets(B, H, W, D, k, es)
    steps_g, fwds_g = [], []
    for i in range(ns):
        x, g = make_inputs(shape, dtype, dist, seed=i)
        steps_g.append(GraphedStep(m, x, g))
        if with_forward:
            fwds_g.append(GraphedForward(m, x))
        for p in m.parameters():
            p.grad = None
    out = {"buffer_sets": ns}
    out["fwd_bwd_ms"] = time_gpu(rotate([s.replay for s in steps_g]), steps, warmup) * 1e3
    out["fwd_bwd_ms_warm"] = time_gpu(steps_g[0].replay, steps, warmup) * 1e3
    if with_forward:
        out["fwd_ms"] = time_gpu(rotate([f.replay for f in fwds_g]), steps, warmup) * 1e3
        out["fwd_ms_warm"] = time_gpu(fwds_g[0].replay, steps, warmup) * 1e3
    bf, bfb = block_alg_bytes(B, H, W, D, k, es)
    out["hbm_frac_fwd_bwd"] = bfb / (out["fwd_bwd_ms"] * 1e-3 * HBM_PEAK)
    if with_forward:
        out["hbm_frac_fwd"] = bf / (out["fwd_ms"] * 1e-3 * HBM_PEAK)
    return out


def measure_block_in_one_graph(m, shape, dtype, steps, warmup):
    """ms per forward+backward step when one HIP graph holds a step on each buffer set (n_sets steps per replay):
    the block as one of several layers of a captured model, where the idle time between two graph replays is
    shared by the layers instead of falling on a single block."""
    B, H, W, D = shape
    k = m.gates[0].conv_spatial.weight.shape[0]
    ns = n_sets(B, H, W, D, k, torch.empty((), dtype=dtype).element_size())
    sets = [make_inputs(shape, dtype, "normal", seed=i) for i in range(ns)]
    xs = [x.detach().clone().requires_grad_() for x, _ in sets]
    keep = []

    def steps_once():
        for x, (_, g) in zip(xs, sets):
            x.grad = None
            for p in m.parameters():
                p.grad = None
            y = m(x)
            torch.autograd.backward(y, g)
            keep.append([y, x.grad] + [p.grad for p in m.parameters()])   # graph-owned results stay referenced

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        steps_once()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    keep.clear()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        steps_once()
    t = time_gpu(graph.replay, max(1, steps // ns), max(1, warmup // ns)) / ns * 1e3
    for p in m.parameters():
        p.grad = None
    return t, ns


def torch_gpu_block(shape, D, k, dtype, steps, warmup):
    """The same block through torch's own GPU operators, as the reference's benchmark times its all-torch twin on
    the same device (pyramid_dwconv/conv_block.py:52-97, :99-158): NCHW, 1x1 and grouped F.conv2d,
    adaptive_avg_pool2d, interpolate; forward + backward, eager launches, cache-warm."""
    import torch.nn.functional as F

    B, H, W, _ = shape
    I, G = D // 2, D // 4
    torch.manual_seed(0)
    P = {
        "up": torch.randn(I, D, 1, 1) / D ** 0.5, "w0": torch.randn(I, 1, k, k) / k, "w1": torch.randn(I, 1, k, k) / k,
        "out": torch.randn(D, 2 * G, 1, 1) / (2 * G) ** 0.5, "out_b": torch.zeros(D),
        "pool": torch.randn(D, D, 1, 1) / D ** 0.5, "pool_b": torch.zeros(D),
    }
    P = {n: v.to(dtype).cuda().requires_grad_() for n, v in P.items()}
    x = torch.randn(B, D, H, W).to(dtype).cuda().requires_grad_()
    g = torch.randn(B, D, H, W).to(dtype).cuda()
    scale = (I / 2) ** -0.5

    def gate(a, w, s):
        if s != 1.0:
            a = F.adaptive_avg_pool2d(a, (int(H * s), int(W * s)))
        c = F.conv2d(a, w, None, 1, k // 2, 1, I)
        c1, c2 = c.chunk(2, dim=1)
        y = c1 * (c2 / scale)
        if s != 1.0:
            y = F.interpolate(y, size=(H, W), mode="bilinear", align_corners=False)
        return y

    def step():
        a = F.conv2d(x, P["up"])
        cat = torch.cat([gate(a, P["w0"], 1.0), gate(a, P["w1"], 0.5)], dim=1)
        y = F.conv2d(cat, P["out"], P["out_b"]) + F.conv2d(F.adaptive_avg_pool2d(x, 1), P["pool"], P["pool_b"])
        torch.autograd.backward(y, g)
        x.grad = None
        for v in P.values():
            v.grad = None

    return time_gpu(step, steps, warmup) * 1e3


# ------------------------------------------------------------------------------------------------
# Per-kernel timings

def load_traffic():
    """HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (scaled by a plain copy of known
    size), as recorded in profiles/hbm_traffic_by_kernel.txt: lines `key = bytes`."""
    out = {}
    try:
        with open(os.path.join(ROOT, "profiles", "hbm_traffic_by_kernel.txt")) as f:
            for line in f:
                line = line.split("#", 1)[0]
                if "=" in line:
                    key, _, val = line.rpartition("=")   # keys carry "k=13" themselves
                    out[key.strip()] = float(val.split()[0])
    except OSError:
        pass
    return out


def kernel_rooflines(B, H, W, D, k, dtype):
    """Times each hot kernel of the block alone at its real shapes; returns a list of dicts."""
    from pyramidconvblock_amd import avgpool, dwconv, ops, up

    I, G = D // 2, D // 4
    es = torch.empty((), dtype=dtype).element_size()
    out = []
    geo = ((1, 1), (k // 2, k // 2), (1, 1))
    iss = conv_issue(k)
    for tag, (h, w) in (("full", (H, W)), ("half", (H // 2, W // 2))):
        n_el = B * h * w * I
        nbuf = max(2, int(600e6 // (2 * n_el * es)) + 1)
        xs = [torch.randn(B, h, w, I, device="cuda").to(dtype) for _ in range(nbuf)]
        gs = [torch.randn(B, h, w, I, device="cuda").to(dtype) for _ in range(nbuf)]
        wt = (torch.randn(k, k, I, device="cuda") / k).to(dtype)
        conv_bytes = es * (2 * n_el + k * k * I)
        flops = 2.0 * k * k * n_el
        for name, fn, issued in (
            ("dwconv_fwd", lambda i: dwconv.dwconv_forward(xs[i], wt, *geo), iss["fwd"]),
            ("dwconv_dgrad", lambda i: dwconv.dwconv_dgrad(gs[i], wt, xs[i].shape, *geo), iss["fwd"]),
            ("dwconv_wgrad", lambda i: dwconv.dwconv_wgrad(xs[i], gs[i], wt.shape, *geo), iss["wgrad"]),
        ):
            t = time_kernel_events(fn, nbuf)
            out.append(dict(kernel=f"{name}[{B}x{h}x{w}x{I},k={k}]", seconds=t, alg_bytes=conv_bytes, flops=flops,
                            issued_flops=2.0 * issued * n_el if issued else None, pipe="mfma"))
        del xs, gs
    h, w = H // 2, W // 2
    nF, nH = B * H * W * I, B * h * w * I
    # the forward convolutions of both scales as one launch
    nbuf = max(2, int(600e6 // (2.5 * nF * es)) + 1)
    xf = [torch.randn(B, H, W, I, device="cuda").to(dtype) for _ in range(nbuf)]
    xh = [torch.randn(B, h, w, I, device="cuda").to(dtype) for _ in range(nbuf)]
    wt, wt1 = ((torch.randn(k, k, I, device="cuda") / k).to(dtype) for _ in range(2))
    if dwconv.dwconv_forward2(xf[0], wt, xh[0], wt1) is not None:
        t = time_kernel_events(lambda i: dwconv.dwconv_forward2(xf[i], wt, xh[i], wt1), nbuf)
        out.append(dict(kernel=f"dwconv_fwd2[{B}x{H}x{W}x{I},k={k}]", seconds=t, alg_bytes=es * (2 * nF + 2 * nH + 2 * k * k * I),
                        flops=2.0 * k * k * (nF + nH), issued_flops=2.0 * iss["fwd"] * (nF + nH), pipe="mfma"))
    del xf, xh
    # the backward's largest launch: full-scale input gradient (adds the pooled branch's) + both weight gradients
    nbuf = max(2, int(600e6 // (4 * nF * es)) + 1)
    gf = [torch.randn(B, H, W, I, device="cuda").to(dtype) for _ in range(nbuf)]
    xf = [torch.randn(B, H, W, I, device="cuda").to(dtype) for _ in range(nbuf)]
    gp = [torch.randn(B, h, w, I, device="cuda").to(dtype) for _ in range(nbuf)]
    xh = [torch.randn(B, h, w, I, device="cuda").to(dtype) for _ in range(nbuf)]
    gh = [torch.randn(B, h, w, I, device="cuda").to(dtype) for _ in range(nbuf)]
    wt = (torch.randn(k, k, I, device="cuda") / k).to(dtype)
    if dwconv.dwconv_bwd3(gf[0], wt, gp[0], xf[0], xh[0], gh[0]) is not None:
        from pyramidconvblock_amd import _lib

        def four(i):   # as in the block, the summations of the weight-gradient partials are deferred: one small
            with _lib.deferred_reductions(gf[0].device):   # launch per 4 calls here, one per backward pass there
                for j in range(4 * i, 4 * i + 4):
                    dwconv.dwconv_bwd3(gf[j % nbuf], wt, gp[j % nbuf], xf[j % nbuf], xh[j % nbuf], gh[j % nbuf])

        t_call = time_kernel_events(four, nbuf, iters=6) / 4
        # the launch alone: a graph of `group` calls whose summations are recorded inside the capture and run after
        # it (the deferral is closed outside the graph), replayed between two HIP events
        group = min(nbuf, 4)
        four(0)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        ctx = _lib.deferred_reductions(gf[0].device)
        with torch.cuda.graph(graph):
            ctx.__enter__()
            for j in range(group):
                dwconv.dwconv_bwd3(gf[j], wt, gp[j], xf[j], xh[j], gh[j])
        ctx.__exit__(None, None, None)
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        graph.replay()
        torch.cuda.synchronize()
        start.record()
        for _ in range(24):
            graph.replay()
        stop.record()
        torch.cuda.synchronize()
        t = start.elapsed_time(stop) * 1e-3 / (24 * group)
        del graph
        out.append(dict(kernel=f"dwconv_bwd3[{B}x{H}x{W}x{I},k={k}]", seconds=t, call_seconds=t_call,
                        alg_bytes=es * (3 * nF + 3 * nH + 3 * k * k * I), flops=2.0 * k * k * (2 * nF + nH),
                        issued_flops=(2.0 * (iss["fwd"] * nF + iss["wgrad"] * (nF + nH)) if iss["wgrad"] else None),
                        pipe="mfma"))
    del gf, xf, gp, xh, gh
    # resampling kernels of the half-resolution gate
    nbuf = 8
    a = [torch.randn(B, H, W, I, device="cuda").to(dtype) for _ in range(nbuf)]
    p = [torch.randn(B, h, w, I, device="cuda").to(dtype) for _ in range(nbuf)]
    gsm = [torch.randn(B, h, w, G, device="cuda").to(dtype) for _ in range(nbuf)]
    gbig = [torch.randn(B, H, W, G, device="cuda").to(dtype) for _ in range(nbuf)]
    for name, fn, nbytes in (
        ("avgpool_fwd", lambda i: avgpool.avgpool_forward(a[i], (h, w)), es * (B * H * W * I + B * h * w * I)),
        ("avgpool_bwd", lambda i: avgpool.avgpool_backward(p[i], (H, W)), es * (B * H * W * I + B * h * w * I)),
        ("bilinear_fwd", lambda i: up.bilinear_forward(gsm[i], (H, W)), es * (B * H * W * G + B * h * w * G)),
        ("bilinear_bwd", lambda i: up.bilinear_backward(gbig[i], (h, w)), es * (B * H * W * G + B * h * w * G)),
    ):
        t = time_kernel_events(fn, nbuf)
        out.append(dict(kernel=name, seconds=t, alg_bytes=nbytes, flops=0.0, issued_flops=None, pipe="valu"))
    # the same four at four times the batch: at the block's own size their tensors are 8-16 MB, which at 8 TB/s is
    # 1-2 us of traffic under the ~2.8 us that any launch costs here, so the fraction there measures the launch
    B4, nb4 = 4 * B, 4
    a4 = [torch.randn(B4, H, W, I, device="cuda").to(dtype) for _ in range(nb4)]
    p4 = [torch.randn(B4, h, w, I, device="cuda").to(dtype) for _ in range(nb4)]
    gsm4 = [t_[..., :G].contiguous() for t_ in p4]
    gbig4 = [t_[..., :G].contiguous() for t_ in a4]
    for name, fn, nbytes in (
        (f"avgpool_fwd[{B4}x{H}x{W}x{I}]", lambda i: avgpool.avgpool_forward(a4[i], (h, w)), es * B4 * (H * W + h * w) * I),
        (f"avgpool_bwd[{B4}x{H}x{W}x{I}]", lambda i: avgpool.avgpool_backward(p4[i], (H, W)), es * B4 * (H * W + h * w) * I),
        (f"bilinear_fwd[{B4}x{H}x{W}x{G}]", lambda i: up.bilinear_forward(gsm4[i], (H, W)), es * B4 * (H * W + h * w) * G),
        (f"bilinear_bwd[{B4}x{H}x{W}x{G}]", lambda i: up.bilinear_backward(gbig4[i], (h, w)), es * B4 * (H * W + h * w) * G),
    ):
        t = time_kernel_events(fn, nb4, iters=12)
        out.append(dict(kernel=name, seconds=t, alg_bytes=nbytes, flops=0.0, issued_flops=None, pipe="valu"))
    del a4, p4, gsm4, gbig4
    # gate and the dense conv_up layer ([N,D] <-> [N,I])
    c = [torch.randn(B, H, W, I, device="cuda").to(dtype) for _ in range(nbuf)]
    xin = [torch.randn(B, H, W, D, device="cuda").to(dtype) for _ in range(4)]
    wup = (torch.randn(I, D, device="cuda") / D ** 0.5).to(dtype)
    wout = (torch.randn(D, I, device="cuda") / I ** 0.5).to(dtype)
    rbias = torch.randn(B, D, device="cuda")
    cats = [torch.empty(B, H, W, I, device="cuda", dtype=dtype) for _ in range(4)]
    N = B * H * W
    for name, fn, nb_, nbytes, fl, pipe in (
        ("gate_fwd", lambda i: ops.gate_forward(c[i]), nbuf, es * 1.5 * N * I, 0.0, "valu"),
        ("gate_bwd", lambda i: ops.gate_backward(c[i], gbig[i]), nbuf, es * 2.5 * N * I, 0.0, "valu"),
        ("dense_fwd", lambda i: ops.dense_forward(xin[i], wup), 4, es * (N * D + N * I + D * I), 2.0 * N * D * I, "mfma"),
        # conv_up as the block runs it: with the tile sums of x and the 2x2 average pool of its result
        ("dense_fwd_pool", lambda i: ops.dense_forward_pool(xin[i], wup), 4, es * (N * D + N * I + N * I // 4 + D * I),
         2.0 * N * D * I, "mfma"),
        ("dense_dgrad", lambda i: ops.dense_forward(a[i], wup, w_kmajor=True), 4, es * (N * D + N * I + D * I),
         2.0 * N * D * I, "mfma"),
        ("dense_wgrad", lambda i: ops.dense_wgrad(a[i % 4], xin[i % 4]), 4, es * (N * D + N * I + D * I),
         2.0 * N * D * I, "mfma"),
        # both gradients of conv_up as the block's backward runs them: one launch, gy read once
        ("dense_bwd_pair", lambda i: ops.dense_backward_pair(a[i % 4], wup, xin[i % 4]), 4,
         es * (2 * N * D + N * I + 2 * D * I), 4.0 * N * D * I, "mfma"),
        # conv_out as the block's forward runs it: on rows it makes from the convolution outputs of both scales (gates,
        # resize), which it also writes out for the backward
        ("dense_mid", lambda i: ops.dense_forward_gated(c[i % 4], p[i % 4], wout, rowbias=rbias, cat=cats[i % 4]), 4,
         es * (N * I + N * I // 4 + N * I + N * D + D * I), 2.0 * N * D * I, "mfma"),
    ):
        t = time_kernel_events(fn, nb_)
        out.append(dict(kernel=name, seconds=t, alg_bytes=nbytes, flops=fl, issued_flops=fl if pipe == "mfma" else None,
                        pipe=pipe))
    return out


def conv_rows(B, H, W, C, dtype, ks=(9, 13, 17)):
    """Stand-alone depthwise-conv forward, x [B,H,W,C], weight ~ N(0, 1/k^2), 'same' padding, stride 1."""
    from pyramidconvblock_amd import dwconv

    es = torch.empty((), dtype=dtype).element_size()
    n_el = B * H * W * C
    nbuf = max(2, int(600e6 // (2 * n_el * es)) + 1)
    xs = [torch.randn(B, H, W, C, device="cuda").to(dtype) for _ in range(nbuf)]
    rows = {}
    for k in ks:
        wt = (torch.randn(k, k, C, device="cuda") / k).to(dtype)
        geo = ((1, 1), (k // 2, k // 2), (1, 1))
        t = time_kernel_events(lambda i: dwconv.dwconv_forward(xs[i], wt, *geo), nbuf)
        nbytes = es * (2 * n_el + k * k * C)
        iss = conv_issue(k)
        rows[f"k{k}"] = {"us": round(t * 1e6, 2), "hbm_frac": round(nbytes / t / HBM_PEAK, 4),
                         "mfma_issue_frac": round(2.0 * iss["fwd"] * n_el / t / MFMA_PEAK, 4),
                         "useful_tap_frac": round(iss["useful"] / iss["fwd"], 3)}
    return rows


def run_single_kernel(name, iters, B, H, W, D, k, dtype):
    """Launches one hot kernel `iters` times at its shape inside the headline block (for rocprofv3 runs).
    name: {fwd,dgrad,wgrad}_{full,half} | fwd2 (the forward convolutions of both scales, one launch) |
    bwd3 (full-scale input gradient + both weight gradients, one launch) |
    conv128 (stand-alone forward at C = D) | avgpool_fwd | avgpool_bwd |
    bilinear_fwd | bilinear_bwd | dense_{fwd,pool,dgrad,wgrad,pair} (the conv_up layer: [N,D] <-> [N,D/2]; pool = forward with tile sums and the
    2x2 pool of the result; pair = both
    gradients in one launch) | step (whole forward+backward steps, eager) | copy"""
    from pyramidconvblock_amd import avgpool, dwconv, up

    I, G = D // 2, D // 4
    h, w = H // 2, W // 2
    geo = ((1, 1), (k // 2, k // 2), (1, 1))
    op, _, res = name.partition("_")
    if name == "copy":  # a plain copy of known size: the yardstick for the FETCH_SIZE / WRITE_SIZE counters
        src = torch.randn(B, H, W, I, device="cuda").to(dtype)
        dst = torch.empty_like(src)
        fn = lambda: dst.copy_(src)
    elif name == "step":
        m = make_block(D, k, dtype)
        x, g = make_inputs((B, H, W, D), dtype, "normal", 0)
        x.requires_grad_()

        def fn():
            torch.autograd.backward(m(x), g)
            x.grad = None
            for p in m.parameters():
                p.grad = None
    elif name == "conv128":
        x = torch.randn(B, H, W, D, device="cuda").to(dtype)
        wt = (torch.randn(k, k, D, device="cuda") / k).to(dtype)
        fn = lambda: dwconv.dwconv_forward(x, wt, *geo)
    elif name == "fwd2":
        xf = torch.randn(B, H, W, I, device="cuda").to(dtype)
        xh = torch.randn(B, h, w, I, device="cuda").to(dtype)
        wt, wt1 = ((torch.randn(k, k, I, device="cuda") / k).to(dtype) for _ in range(2))
        fn = lambda: dwconv.dwconv_forward2(xf, wt, xh, wt1)
    elif name == "dense_mid":   # conv_out on rows made from the two scales' convolution outputs, writing them to cat
        from pyramidconvblock_amd import ops

        cf = torch.randn(B, H, W, I, device="cuda").to(dtype)
        chh = torch.randn(B, h, w, I, device="cuda").to(dtype)
        cat = torch.empty_like(cf)
        wout = (torch.randn(D, I, device="cuda") / I ** 0.5).to(dtype)
        rb = torch.randn(B, D, device="cuda")
        fn = lambda: ops.dense_forward_gated(cf, chh, wout, rowbias=rb, cat=cat)
    elif name == "bwd3":
        gf, xf = (torch.randn(B, H, W, I, device="cuda").to(dtype) for _ in range(2))
        gp, xh, gh = (torch.randn(B, h, w, I, device="cuda").to(dtype) for _ in range(3))
        wt = (torch.randn(k, k, I, device="cuda") / k).to(dtype)
        fn = lambda: dwconv.dwconv_bwd3(gf, wt, gp, xf, xh, gh)
    elif op in ("fwd", "dgrad", "wgrad"):
        hh, ww = (H, W) if res == "full" else (h, w)
        x = torch.randn(B, hh, ww, I, device="cuda").to(dtype)
        g = torch.randn(B, hh, ww, I, device="cuda").to(dtype)
        wt = (torch.randn(k, k, I, device="cuda") / k).to(dtype)
        fn = {"fwd": lambda: dwconv.dwconv_forward(x, wt, *geo),
              "dgrad": lambda: dwconv.dwconv_dgrad(g, wt, x.shape, *geo),
              "wgrad": lambda: dwconv.dwconv_wgrad(x, g, wt.shape, *geo)}[op]
    elif op == "dense":
        from pyramidconvblock_amd import ops

        xin = torch.randn(B, H, W, D, device="cuda").to(dtype)
        ain = torch.randn(B, H, W, I, device="cuda").to(dtype)
        wup = (torch.randn(I, D, device="cuda") / D ** 0.5).to(dtype)
        rb = torch.randn(B, D, device="cuda")
        fn = {"fwd": lambda: ops.dense_forward(xin, wup),
              "pool": lambda: ops.dense_forward_pool(xin, wup),
              "dgrad": lambda: ops.dense_forward(ain, wup, w_kmajor=True, rowbias=rb, rows_per_image=H * W),
              "wgrad": lambda: ops.dense_wgrad(ain, xin),
              "pair": lambda: ops.dense_backward_pair(ain, wup, xin, rowbias=rb, rows_per_image=H * W)}[res]
    else:
        a = torch.randn(B, H, W, I, device="cuda").to(dtype)
        p = torch.randn(B, h, w, I, device="cuda").to(dtype)
        gs = torch.randn(B, h, w, G, device="cuda").to(dtype)
        gb = torch.randn(B, H, W, G, device="cuda").to(dtype)
        fn = {"avgpool_fwd": lambda: avgpool.avgpool_forward(a, (h, w)),
              "avgpool_bwd": lambda: avgpool.avgpool_backward(p, (H, W)),
              "bilinear_fwd": lambda: up.bilinear_forward(gs, (H, W)),
              "bilinear_bwd": lambda: up.bilinear_backward(gb, (h, w))}[name]
    for _ in range(iters):
        fn()
    torch.cuda.synchronize()


# ------------------------------------------------------------------------------------------------
# CPU baseline

def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_threads():
    """Threads for the CPU baseline: the host's processors, capped by the share the job was given
    (OMP_NUM_THREADS where the environment sets one)."""
    n = os.cpu_count() or 1
    try:
        n = min(n, int(os.environ["OMP_NUM_THREADS"]))
    except (KeyError, ValueError):
        pass
    return max(1, n)


def cpu_baseline(B, H, W, D, k, dtype, threads, iters=3):
    """The reference's PyTorch path (F.conv2d groups=C, adaptive_avg_pool2d, interpolate, linear) on
    the host cores: forward+backward of the same block on the same seeded inputs."""
    from oracle import torch_path

    torch.set_num_threads(threads)
    torch.manual_seed(0)
    P = {n: v.to(dtype).requires_grad_() for n, v in torch_path.default_params(D, k).items()}
    gen = torch.Generator().manual_seed(0)
    x = torch.randn(B, H, W, D, generator=gen).to(dtype).requires_grad_()
    g = torch.randn(B, H, W, D, generator=gen).to(dtype)

    def step():
        y = torch_path.convblock(x, P)
        torch.autograd.backward(y, g)
        x.grad = None
        for v in P.values():
            v.grad = None

    step()
    ts = []
    for _ in range(iters):
        t0 = time.perf_counter()
        step()
        ts.append(time.perf_counter() - t0)
    ts.sort()
    return ts[len(ts) // 2]


# ------------------------------------------------------------------------------------------------

def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=60)
    ap.add_argument("--warmup", type=int, default=12)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-sweep", action="store_true", help="skip the k=9/17 sweep and the batch-size sweep")
    ap.add_argument("--no-kernels", action="store_true", help="skip the per-kernel event timings")
    ap.add_argument("--no-configs", action="store_true", help="skip the rows of the other workloads")
    ap.add_argument("--no-torch-gpu", action="store_true", help="skip the torch-operator comparator on the GPU")
    ap.add_argument("--kernel", default=None, help="only launch this kernel --steps times and exit (for rocprofv3): "
                    "{fwd,dgrad,wgrad}_{full,half}, fwd2, bwd3, conv128, avgpool_{fwd,bwd}, bilinear_{fwd,bwd}, "
                    "dense_{fwd,pool,dgrad,wgrad,pair,mid}, step, copy")
    ap.add_argument("--torch-gpu-only", action="store_true", help="(internal) time the torch-operator comparator and exit")
    ap.add_argument("--headline-only", action="store_true", help="(internal) time the headline step only and exit")
    ap.add_argument("--k", type=int, default=WORKLOAD["k"], help="kernel size for --kernel runs")
    ap.add_argument("--dtype", default="bf16", choices=sorted(DTYPES), help="element type for --kernel runs")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py measures one GPU: this path has no multi-GPU part (pure data parallel over B; "
                 "only the k*k*C weight-gradient all-reduce would cross GPUs). Run with --gpus 1.")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU (the kernels have no CPU path)")

    from pyramidconvblock_amd import _lib

    _lib.lib()
    dtype = torch.bfloat16
    B, H, W, D, k = (WORKLOAD[n] for n in ("B", "H", "W", "D", "k"))
    if args.kernel:
        run_single_kernel(args.kernel, args.steps, B, H, W, D, args.k, DTYPES[args.dtype])
        return
    if args.torch_gpu_only:
        print(json.dumps({"fwd_bwd_ms": torch_gpu_block((B, H, W, D), D, k, dtype, steps=10, warmup=3)}))
        return

    m = make_block(D, k, dtype)
    if args.headline_only:
        head = measure_block(m, (B, H, W, D), dtype, "normal", args.steps, args.warmup, with_forward=False)
        print(json.dumps({"fwd_bwd_ms": head["fwd_bwd_ms"], "fwd_bwd_ms_warm": head["fwd_bwd_ms_warm"]}))
        return
    head = measure_block(m, (B, H, W, D), dtype, "normal", args.steps, args.warmup)
    t_chain, n_chain = measure_block_in_one_graph(m, (B, H, W, D), dtype, args.steps, args.warmup)
    # eager launches of the same step (host-bound), for reference
    x0, g0 = make_inputs((B, H, W, D), dtype, "normal", 0)
    x0.requires_grad_()

    def eager():
        torch.autograd.backward(m(x0), g0)
        x0.grad = None
        for p in m.parameters():
            p.grad = None

    t_eager = time_gpu(eager, args.steps, args.warmup)
    for p in m.parameters():
        p.grad = None
    del x0, g0
    bytes_f, bytes_fb = block_alg_bytes(B, H, W, D, k, 2)
    t_step = head["fwd_bwd_ms"] * 1e-3

    result = {
        "metric": "convblock_fwd_bwd_ms",
        "value": head["fwd_bwd_ms"],
        "unit": "ms",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": head["fwd_bwd_ms"],
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "ConvBlock(dim=128,kernel_size=13) fwd+bwd, bf16, x[32,56,56,128] N(0,1), "
                               "default-init weights, grad_out N(0,1)"},
        "cache_state": f"rotated: consecutive steps use {head['buffer_sets']} different sets of inputs, activations and "
                       "gradients (more than twice the 256 MB Infinity Cache in total), so a step's inputs come from HBM",
        "warm_ms_per_step": head["fwd_bwd_ms_warm"],
        "warm_note": "the same step replayed on one buffer set: inputs and weights hit in the Infinity Cache",
        "fwd_ms": head["fwd_ms"],
        "warm_fwd_ms": head["fwd_ms_warm"],
        "eager_ms_per_step": t_eager * 1e3,
        "launch": "one HIP graph replay per step (eager launch time in eager_ms_per_step)",
        "runtime_settings": {GRAPH_SUBMIT_ENV: os.environ.get(GRAPH_SUBMIT_ENV)},
        "in_graph_ms_per_step": t_chain,
        "in_graph_note": f"{n_chain} steps (one per buffer set) captured in ONE graph, time per replay / {n_chain}: the "
                         "block as one of several layers of a captured model; `value` instead pays the idle time "
                         "between two graph replays once per step",
        "block_hbm_frac_fwd_bwd": bytes_fb / (t_step * HBM_PEAK),
        "block_hbm_frac_fwd_bwd_warm": bytes_fb / (head["fwd_bwd_ms_warm"] * 1e-3 * HBM_PEAK),
        "block_hbm_frac_fwd": bytes_f / (head["fwd_ms"] * 1e-3 * HBM_PEAK),
        "block_alg_bytes_fwd_bwd": bytes_fb,
        "block_alg_bytes_fwd": bytes_f,
    }

    if not args.no_sweep:
        sweep = {}
        for kk in (9, 13, 17):
            if kk == k:
                r = head
            else:
                mk = make_block(D, kk, dtype)
                r = measure_block(mk, (B, H, W, D), dtype, "normal", args.steps, args.warmup)
                del mk
            sweep[f"k{kk}"] = {n: round(r[n], 5) for n in ("fwd_ms", "fwd_bwd_ms", "fwd_bwd_ms_warm", "hbm_frac_fwd",
                                                            "hbm_frac_fwd_bwd")}
        result["sweep"] = sweep
        # The same block at other batch sizes (not the metric: how the fixed cost per launch amortises)
        batches = {}
        for bb in (8, 64, 128):
            r = measure_block(m, (bb, H, W, D), dtype, "normal", args.steps, args.warmup, with_forward=False)
            batches[f"B{bb}"] = {"fwd_bwd_ms": round(r["fwd_bwd_ms"], 5), "hbm_frac_fwd_bwd": round(r["hbm_frac_fwd_bwd"], 4)}
        result["batch_sweep"] = batches

    if not args.no_configs:
        cfg = {}
        # stand-alone depthwise conv forward, bf16, x [32,56,56,128], k = 9/13/17
        cfg["dwconv_fwd_bf16_32x56x56x128"] = conv_rows(B, H, W, D, dtype)
        # the same in fp32 (vector kernel)
        cfg["dwconv_fwd_fp32_32x56x56x128"] = {
            kk: {n: v for n, v in row.items() if n in ("us", "hbm_frac")}
            for kk, row in conv_rows(B, H, W, D, torch.float32).items()}
        # high-resolution stage: fp16, x [8,112,112,96], k = 17
        mk = make_block(96, 17, torch.float16)
        cfg["convblock_fp16_8x112x112x96_k17"] = {n: round(v, 5) for n, v in measure_block(
            mk, (8, 112, 112, 96), torch.float16, "normal", args.steps, args.warmup).items()}
        # ragged shapes: x [3,57,61,200] ~ U(-2,2), k = 9 and 15, fp32 and bf16
        for dn in ("fp32", "bf16"):
            for kk in (9, 15):
                mk = make_block(200, kk, DTYPES[dn])
                cfg[f"convblock_{dn}_3x57x61x200_k{kk}"] = {n: round(v, 5) for n, v in measure_block(
                    mk, (3, 57, 61, 200), DTYPES[dn], "uniform", args.steps, args.warmup).items()}
        # the headline block in fp32
        mk = make_block(D, k, torch.float32)
        cfg["convblock_fp32_32x56x56x128_k13"] = {n: round(v, 5) for n, v in measure_block(
            mk, (B, H, W, D), torch.float32, "normal", args.steps, args.warmup).items()}
        del mk
        result["configs"] = cfg

    if not args.no_kernels:
        ks = kernel_rooflines(B, H, W, D, k, dtype)
        traffic = load_traffic()
        dom = max(ks, key=lambda r: r["seconds"])   # the longest launch of the step
        ai = dom["flops"] / dom["alg_bytes"]
        result["roofline"] = {
            "kernel": dom["kernel"],
            # the roofline that bounds it: its useful flops per algorithmic byte against the machine balance
            "bound": "hbm" if ai < MFMA_PEAK / HBM_PEAK else "mfma",
            "achieved": dom["alg_bytes"] / dom["seconds"] / 1e9, "peak": HBM_PEAK / 1e9, "unit": "GB/s",
            "frac": dom["alg_bytes"] / dom["seconds"] / HBM_PEAK,
            "traffic": traffic.get(dom["kernel"]), "avg_us": dom["seconds"] * 1e6,
            "flops_per_byte": ai, "machine_flops_per_byte": MFMA_PEAK / HBM_PEAK,
            "mfma_issue_frac": (dom["issued_flops"] / dom["seconds"] / MFMA_PEAK) if dom["issued_flops"] else None,
            "limiter": "not the roofline: LDS operand reads and exposed load latency (profiles/)",
            "timed": "HIP events around graph replays over rotating buffers; for dwconv_bwd3 the graph holds the launch "
                     "alone (its summations are recorded during the capture and run outside the graph; `call_us` in the "
                     "kernels row includes them), graph launch gaps included",
        }
        result["kernels"] = []
        for r in ks:
            row = {"kernel": r["kernel"], "us": round(r["seconds"] * 1e6, 2),
                   "hbm_frac": round(r["alg_bytes"] / r["seconds"] / HBM_PEAK, 4), "pipe": r["pipe"]}
            if r["issued_flops"]:
                row["mfma_issue_frac"] = round(r["issued_flops"] / r["seconds"] / MFMA_PEAK, 4)
            if r["kernel"] in traffic:
                row["traffic"] = traffic[r["kernel"]]
            if "call_seconds" in r:   # the call with its share of the deferred summation launches
                row["call_us"] = round(r["call_seconds"] * 1e6, 2)
            result["kernels"].append(row)

    if os.environ.get(GRAPH_SUBMIT_ENV) == "0":
        # the same step under the runtime's default graph submission, in a child process (the setting is read once)
        import subprocess

        try:
            env = dict(os.environ)
            env[GRAPH_SUBMIT_ENV] = "1"
            cp = subprocess.run([sys.executable, os.path.abspath(__file__), "--headline-only", "--steps", str(args.steps),
                                 "--warmup", str(args.warmup)], capture_output=True, text=True, timeout=240, env=env)
            d = json.loads(cp.stdout.strip().splitlines()[-1])
            result["default_runtime_ms_per_step"] = d["fwd_bwd_ms"]
            result["default_runtime_warm_ms_per_step"] = d["fwd_bwd_ms_warm"]
            result["default_runtime_note"] = (f"the rotated / warm step with {GRAPH_SUBMIT_ENV}=1, this image's default: the "
                                              "runtime replays pre-built dispatch packets, which costs more per replay here")
        except Exception as e:  # noqa: BLE001
            result["default_runtime_ms_per_step"] = None
            result["default_runtime_note"] = f"{type(e).__name__}: {e}"[:300]

    if not args.no_torch_gpu:
        # in a child process with a time limit: the library may build its kernels on first use
        import subprocess

        try:
            cp = subprocess.run([sys.executable, os.path.abspath(__file__), "--torch-gpu-only"], capture_output=True,
                                text=True, timeout=240)
            t_torch = json.loads(cp.stdout.strip().splitlines()[-1])["fwd_bwd_ms"]
            result["torch_gpu"] = {"fwd_bwd_ms": t_torch, "speedup": t_torch / head["fwd_bwd_ms_warm"],
                                   "what": "same block through torch-ROCm operators (NCHW conv2d 1x1 / groups=C, "
                                           "adaptive_avg_pool2d, interpolate), eager, cache-warm; speedup against "
                                           "warm_ms_per_step"}
        except Exception as e:  # noqa: BLE001 - the comparator must not take the bench line down
            result["torch_gpu"] = {"error": f"{type(e).__name__}: {e}"[:300]}

    if not args.no_cpu:
        threads = cpu_threads()
        t_bf16 = cpu_baseline(B, H, W, D, k, torch.bfloat16, threads)
        t_fp32 = cpu_baseline(B, H, W, D, k, torch.float32, threads)
        result["cpu_baseline"] = {"value": t_bf16 * 1e3, "unit": "ms", "cores": threads, "kind": "port",
                                  "fp32_value": t_fp32 * 1e3, "cpu_model": cpu_model(), "host_cpus": os.cpu_count(),
                                  "sample": "full workload: same ConvBlock fwd+bwd through torch CPU ops "
                                            "(F.conv2d groups=C, adaptive_avg_pool2d, interpolate, linear), "
                                            "median of 3 after 1 warm-up; value in bf16, fp32_value in fp32; threads = "
                                            "host processors capped by the job's OMP_NUM_THREADS share"}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
