#!/usr/bin/env python3
"""Benchmark of the ConvBlock hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-sweep]

A step is one ConvBlock forward + backward on the headline workload
(ConvBlock(128, kernel_size=13), bf16, x [32,56,56,128], seeded synthetic data, inputs
resident in HBM).  Prints ONE JSON line: ms per step, the forward-only time, the k = 9/13/17
sweep, the HBM-roofline fraction of the whole block and of the dominant kernel (timed live
with HIP events on the launch stream), and the PyTorch-CPU baseline of the same workload.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12  # B/s, MI355X published
VALU_PEAK = 157.3e12  # fp32 vector FLOP/s, MI355X published
MFMA_PEAK = 2.5e15    # dense bf16/fp16 matrix FLOP/s, MI355X published

WORKLOAD = dict(B=32, H=56, W=56, D=128, k=13, dtype="bf16")

# HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of `bench.py --kernel ...`, each
# scaled by what the same counter reads for a plain copy of known size (`bench.py --kernel copy`); the
# runs and the scale factors are recorded under profiles/.  None = not measured.
MEASURED_TRAFFIC = {
    "dwconv_fwd[32x56x56x64,k=13]": (12872 + 12544) * 1024,   # fetch 13.18 MB + write 12.85 MB
    "dwconv_dgrad[32x56x56x64,k=13]": (12872 + 12544) * 1024,  # same kernel, same shape
    "dwconv_wgrad[32x56x56x64,k=13]": (25392 + 2704 + 2721 + 21) * 1024,  # main kernel + partial reduction
}


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


def dwconv_flops_block(B, H, W, D, k, scales=(1.0, 0.5)):
    I = D // 2
    N = B * H * W
    n = B * int(H * scales[1]) * int(W * scales[1])
    f = 2 * k * k * I * (N + n)
    return f, 3 * f


def make_block(D, k, dtype, seed=0):
    import pyramid_dwconv

    torch.manual_seed(seed)
    return pyramid_dwconv.ConvBlock(dim=D, kernel_size=k).to(dtype).cuda()


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


def time_kernel_events(launch, nbuf, iters=24, reps=4):
    """Average duration of one launch.  `iters` launches (launch(i) uses buffer set i % nbuf, so that
    consecutive launches do not hit in the 256 MB Infinity Cache) are captured into a HIP graph, and the
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


def kernel_rooflines(B, H, W, D, k, dtype):
    """Times each hot kernel of the block alone at its real shapes; returns a list of dicts."""
    from pyramidconvblock_amd import avgpool, dwconv, ops, up

    I, G = D // 2, D // 4
    es = torch.empty((), dtype=dtype).element_size()
    out = []
    geo = ((1, 1), (k // 2, k // 2), (1, 1))
    for tag, (h, w) in (("full", (H, W)), ("half", (H // 2, W // 2))):
        n_el = B * h * w * I
        nbuf = max(2, int(600e6 // (2 * n_el * es)) + 1)
        xs = [torch.randn(B, h, w, I, device="cuda").to(dtype) for _ in range(nbuf)]
        gs = [torch.randn(B, h, w, I, device="cuda").to(dtype) for _ in range(nbuf)]
        wt = (torch.randn(k, k, I, device="cuda") / k).to(dtype)
        conv_bytes = es * (2 * n_el + k * k * I)
        flops = 2.0 * k * k * n_el
        for name, fn in (
            ("dwconv_fwd", lambda i: dwconv.dwconv_forward(xs[i], wt, *geo)),
            ("dwconv_dgrad", lambda i: dwconv.dwconv_dgrad(gs[i], wt, xs[i].shape, *geo)),
            ("dwconv_wgrad", lambda i: dwconv.dwconv_wgrad(xs[i], gs[i], wt.shape, *geo)),
        ):
            t = time_kernel_events(fn, nbuf)
            out.append(dict(kernel=f"{name}[{B}x{h}x{w}x{I},k={k}]", seconds=t, alg_bytes=conv_bytes, flops=flops))
        del xs, gs
    # resampling kernels of the half-resolution gate
    h, w = H // 2, W // 2
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
        out.append(dict(kernel=name, seconds=t, alg_bytes=nbytes, flops=0.0))
    # gate and the dense conv_up layer ([N,D] <-> [N,I])
    c = [torch.randn(B, H, W, I, device="cuda").to(dtype) for _ in range(nbuf)]
    xin = [torch.randn(B, H, W, D, device="cuda").to(dtype) for _ in range(4)]
    wup = (torch.randn(I, D, device="cuda") / D ** 0.5).to(dtype)
    N = B * H * W
    for name, fn, nb_, nbytes, fl in (
        ("gate_fwd", lambda i: ops.gate_forward(c[i]), nbuf, es * 1.5 * N * I, 0.0),
        ("gate_bwd", lambda i: ops.gate_backward(c[i], gbig[i]), nbuf, es * 2.5 * N * I, 0.0),
        ("dense_fwd", lambda i: ops.dense_forward(xin[i], wup), 4, es * (N * D + N * I + D * I), 2.0 * N * D * I),
        ("dense_dgrad", lambda i: ops.dense_forward(a[i], wup, w_kmajor=True), 4, es * (N * D + N * I + D * I),
         2.0 * N * D * I),
        ("dense_wgrad", lambda i: ops.dense_wgrad(a[i % 4], xin[i % 4]), 4, es * (N * D + N * I + D * I),
         2.0 * N * D * I),
        # both gradients of conv_up as the block's backward runs them: one launch, gy read once
        ("dense_bwd_pair", lambda i: ops.dense_backward_pair(a[i % 4], wup, xin[i % 4]), 4,
         es * (2 * N * D + N * I + 2 * D * I), 4.0 * N * D * I),
    ):
        t = time_kernel_events(fn, nb_)
        out.append(dict(kernel=name, seconds=t, alg_bytes=nbytes, flops=fl))
    return out


def run_single_kernel(name, iters, B, H, W, D, k, dtype):
    """Launches one hot kernel `iters` times at its shape inside the headline block (for rocprofv3 runs).
    name: {fwd,dgrad,wgrad}_{full,half} | avgpool_fwd | avgpool_bwd | bilinear_fwd | bilinear_bwd |
    dense_{fwd,dgrad,wgrad,pair} (the conv_up layer: [N,D] <-> [N,D/2]; pair = both gradients in one launch)"""
    from pyramidconvblock_amd import avgpool, dwconv, up

    I, G = D // 2, D // 4
    h, w = H // 2, W // 2
    geo = ((1, 1), (k // 2, k // 2), (1, 1))
    op, _, res = name.partition("_")
    if name == "copy":  # a plain copy of known size: the yardstick for the FETCH_SIZE / WRITE_SIZE counters
        src = torch.randn(B, H, W, I, device="cuda").to(dtype)
        dst = torch.empty_like(src)
        fn = lambda: dst.copy_(src)
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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-sweep", action="store_true", help="skip the k=9/17 sweep, the forward-only timings and the batch-size sweep")
    ap.add_argument("--no-kernels", action="store_true", help="skip the per-kernel event timings")
    ap.add_argument("--kernel", default=None, help="only launch this kernel --steps times and exit (for rocprofv3): "
                    "{fwd,dgrad,wgrad}_{full,half}, avgpool_{fwd,bwd}, bilinear_{fwd,bwd}, dense_{fwd,dgrad,wgrad}, copy")
    ap.add_argument("--k", type=int, default=WORKLOAD["k"], help="kernel size for --kernel runs")
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
        run_single_kernel(args.kernel, args.steps, B, H, W, D, args.k, dtype)
        return
    gen = torch.Generator().manual_seed(0)
    x = torch.randn(B, H, W, D, generator=gen).to(dtype).cuda().requires_grad_()
    g = torch.randn(B, H, W, D, generator=gen).to(dtype).cuda()

    def stepper(m):
        def fwd():
            with torch.no_grad():
                return m(x)

        def fwd_bwd():
            y = m(x)
            torch.autograd.backward(y, g)
            x.grad = None
            for p in m.parameters():
                p.grad = None

        return fwd, fwd_bwd

    m = make_block(D, k, dtype)
    fwd, fwd_bwd = stepper(m)
    t_eager = time_gpu(fwd_bwd, args.steps, args.warmup)
    # The step the metric is quoted on: the same forward+backward captured once into a HIP graph
    # and replayed (identical kernels and results; removes the per-launch host overhead).
    from pyramidconvblock_amd.graphs import GraphedForward, GraphedStep

    graphed = GraphedStep(m, x, g)
    t_step = time_gpu(graphed.replay, args.steps, args.warmup)
    for p in m.parameters():
        p.grad = None
    bytes_f, bytes_fb = block_alg_bytes(B, H, W, D, k, 2)
    flops_f, flops_fb = dwconv_flops_block(B, H, W, D, k)

    result = {
        "metric": "convblock_fwd_bwd_ms",
        "value": t_step * 1e3,
        "unit": "ms",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": t_step * 1e3,
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "ConvBlock(dim=128,kernel_size=13) fwd+bwd, bf16, x[32,56,56,128] N(0,1) seed 0, "
                               "default-init weights, grad_out N(0,1)"},
        "eager_ms_per_step": t_eager * 1e3,
        "launch": "one HIP graph replay per step (eager launch time in eager_ms_per_step)",
        "block_hbm_frac_fwd_bwd": bytes_fb / (t_step * HBM_PEAK),
        "block_alg_bytes_fwd_bwd": bytes_fb,
        "block_dwconv_valu_frac_fwd_bwd": flops_fb / (t_step * VALU_PEAK),
    }

    if not args.no_sweep:
        sweep = {}
        for kk in (9, 13, 17):
            mk = m if kk == k else make_block(D, kk, dtype)
            f, fb = stepper(mk)
            tf = time_gpu(GraphedForward(mk, x).replay, args.steps, args.warmup)
            tfb = t_step if kk == k else time_gpu(GraphedStep(mk, x, g).replay, args.steps, args.warmup)
            for p in mk.parameters():
                p.grad = None
            bf, bfb = block_alg_bytes(B, H, W, D, kk, 2)
            sweep[f"k{kk}"] = {"fwd_ms": tf * 1e3, "fwd_bwd_ms": tfb * 1e3, "hbm_frac_fwd": bf / (tf * HBM_PEAK),
                               "hbm_frac_fwd_bwd": bfb / (tfb * HBM_PEAK)}
        result["sweep"] = sweep
        # The same block at other batch sizes (not the metric: how the fixed cost per launch amortises)
        batches = {}
        for bb in (8, 64, 128):
            xb = torch.randn(bb, H, W, D, generator=gen).to(dtype).cuda().requires_grad_()
            gb = torch.randn(bb, H, W, D, generator=gen).to(dtype).cuda()
            tb = time_gpu(GraphedStep(m, xb, gb).replay, args.steps, args.warmup)
            for p in m.parameters():
                p.grad = None
            batches[f"B{bb}"] = {"fwd_bwd_ms": tb * 1e3,
                                 "hbm_frac_fwd_bwd": block_alg_bytes(bb, H, W, D, k, 2)[1] / (tb * HBM_PEAK)}
            del xb, gb
        result["batch_sweep"] = batches

    if not args.no_kernels:
        ks = kernel_rooflines(B, H, W, D, k, dtype)
        # Dominant kernel = largest share of the step.  Forward and input gradient are the same kernel
        # function (dwconv_mfma_k) at the same shape, so their launches count together.
        def share(r):
            return r["seconds"] * (2 if r["kernel"].startswith(("dwconv_fwd", "dwconv_dgrad")) else 1)

        dom = max(ks, key=share)
        result["roofline"] = {
            "kernel": dom["kernel"], "bound": "hbm", "achieved": dom["alg_bytes"] / dom["seconds"] / 1e9,
            "peak": HBM_PEAK / 1e9, "unit": "GB/s", "frac": dom["alg_bytes"] / dom["seconds"] / HBM_PEAK,
            "traffic": MEASURED_TRAFFIC.get(dom["kernel"]), "avg_us": dom["seconds"] * 1e6,
            "valu_frac": dom["flops"] / dom["seconds"] / VALU_PEAK,
            "mfma_frac": dom["flops"] / dom["seconds"] / MFMA_PEAK,
        }
        result["kernels"] = [{"kernel": r["kernel"], "us": round(r["seconds"] * 1e6, 2),
                              "hbm_frac": round(r["alg_bytes"] / r["seconds"] / HBM_PEAK, 4),
                              "valu_frac": round(r["flops"] / r["seconds"] / VALU_PEAK, 4),
                              "mfma_frac": round(r["flops"] / r["seconds"] / MFMA_PEAK, 4)} for r in ks]

    if not args.no_cpu:
        threads = min(os.cpu_count() or 1, 16)
        t_cpu = cpu_baseline(B, H, W, D, k, dtype, threads)
        result["cpu_baseline"] = {"value": t_cpu * 1e3, "unit": "ms", "cores": threads, "kind": "port",
                                  "sample": "full workload: same ConvBlock fwd+bwd in bf16 through torch CPU ops "
                                            "(F.conv2d groups=C, adaptive_avg_pool2d, interpolate, linear), "
                                            "median of 3 after 1 warm-up"}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
