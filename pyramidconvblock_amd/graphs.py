"""HIP-graph capture of a forward+backward step.

A ConvBlock step is a dozen short kernels (about 150 us of GPU time at [32,56,56,128]); launched
one by one from Python and the autograd engine the host takes longer than the GPU.  ``GraphedStep`` captures ``y = module(x); backward(y, grad)`` once into a HIP
graph (through ``torch.cuda.CUDAGraph``) and replays it.  Every kernel of libpdw.so is capture
safe: no allocation, no synchronisation, no memset nodes.
"""
from __future__ import annotations

import torch


class GraphedStep:
    """Captures one forward+backward of `module` on static inputs.

    After ``replay()`` the results are in ``.y`` (output), ``.x.grad`` and the parameters' ``.grad``
    (graph-owned tensors that every replay overwrites).  Copy new data into ``.x`` / ``.grad_out``
    with ``copy_`` before replaying.
    """

    def __init__(self, module: torch.nn.Module, x: torch.Tensor, grad_out: torch.Tensor, warmup: int = 3):
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
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.y = self._step()
        self.param_grads = [p.grad for p in module.parameters()]

    def _clear(self):
        self.x.grad = None
        for p in self.module.parameters():
            p.grad = None

    def _step(self):
        y = self.module(self.x)
        torch.autograd.backward(y, self.grad_out)
        return y.detach()

    def replay(self):
        self.graph.replay()
        return self.y


class GraphedForward:
    """Captures one inference forward (no autograd) of `module` on a static input."""

    def __init__(self, module: torch.nn.Module, x: torch.Tensor, warmup: int = 3):
        self.module = module
        self.x = x.detach().clone()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side), torch.no_grad():
            for _ in range(warmup):
                module(self.x)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph), torch.no_grad():
            self.y = module(self.x)

    def replay(self):
        self.graph.replay()
        return self.y
