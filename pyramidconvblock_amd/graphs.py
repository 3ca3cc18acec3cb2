"""HIP-graph capture of a forward+backward step, and replay of the same step as a list of library calls.

A ConvBlock step is ~15 short kernels; launched one by one from Python (tensor allocation, autograd) the
host is the bottleneck.  ``GraphedStep`` captures ``y = module(x); backward(y, grad)`` once into a HIP graph
(through ``torch.cuda.CUDAGraph``) and replays it.  Every kernel of libpdw.so is capture safe: no
allocation, no synchronisation, no memset nodes.

The capture also notes down the library calls themselves.  When the graph holds nothing but the kernels
of those calls, ``replay()`` issues the calls again on the current stream instead of launching the graph: the
tensors of the step live in the graph's memory pool, so the recorded pointers stay valid, the host needs a
few microseconds per call, and consecutive steps run back to back on the device, without the pause of
several microseconds between two graph launches.
"""
from __future__ import annotations

import ctypes

import torch

from . import _lib


def _graph_node_count(graph: torch.cuda.CUDAGraph) -> int:
    """Nodes of a captured graph (kept with keep_graph=True), or -1 when they cannot be counted."""
    try:
        raw = graph.raw_cuda_graph()
        hip = ctypes.CDLL("libamdhip64.so")
        n = ctypes.c_size_t(0)
        if hip.hipGraphGetNodes(ctypes.c_void_p(raw), None, ctypes.byref(n)) != 0:
            return -1
        return int(n.value)
    except Exception:  # an older torch, or no such symbol: the graph itself is replayed
        return -1


class _Captured:
    """Common part: capture `fn` into a graph while recording the library calls it makes."""

    def _capture(self, fn, dev, calls: str):
        if calls not in ("auto", "never"):
            raise ValueError("calls: 'auto' or 'never'")
        self.device = dev
        try:
            self.graph = torch.cuda.CUDAGraph(keep_graph=True)
        except TypeError:
            self.graph = torch.cuda.CUDAGraph()
        with _lib.recorded_calls() as rec:
            with torch.cuda.graph(self.graph):
                out = fn()
        self.calls = rec.calls
        # only the library's own kernels in the graph: one node per launch the library counted
        self.replays_calls = (calls == "auto" and rec.kernels > 0 and _graph_node_count(self.graph) == rec.kernels)
        return out

    def replay(self):
        if self.replays_calls:
            _lib.replay_calls(self.calls, self.device)
        else:
            self.graph.replay()
        return self.y


class GraphedStep(_Captured):
    """Captures one forward+backward of `module` on static inputs.

    After ``replay()`` the results are in ``.y`` (output), ``.x.grad`` and the parameters' ``.grad``
    (graph-owned tensors that every replay overwrites).  Copy new data into ``.x`` / ``.grad_out``
    with ``copy_`` before replaying.  ``calls="never"`` always launches the graph; ``.replays_calls`` tells
    which way ``replay()`` goes.
    """

    def __init__(self, module: torch.nn.Module, x: torch.Tensor, grad_out: torch.Tensor, warmup: int = 3,
                 calls: str = "auto"):
        self.module = module
        self.x = x.detach().clone().requires_grad_()
        self.grad_out = grad_out.detach().clone()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):  # warm up off the default stream, keeping no autograd graph alive
            for _ in range(warmup):
                self._clear()
                self._step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self._clear()
        self.y = self._capture(self._step, self.x.device, calls)
        self.param_grads = [p.grad for p in module.parameters()]

    def _clear(self):
        self.x.grad = None
        for p in self.module.parameters():
            p.grad = None

    def _step(self):
        y = self.module(self.x)
        torch.autograd.backward(y, self.grad_out)
        return y.detach()


class GraphedForward(_Captured):
    """Captures one inference forward (no autograd) of `module` on a static input."""

    def __init__(self, module: torch.nn.Module, x: torch.Tensor, warmup: int = 3, calls: str = "auto"):
        self.module = module
        self.x = x.detach().clone()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side), torch.no_grad():
            for _ in range(warmup):
                module(self.x)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()

        def fwd():
            with torch.no_grad():
                return module(self.x)

        self.y = self._capture(fwd, self.x.device, calls)
