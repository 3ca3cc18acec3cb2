"""A captured forward+backward step must give the eager results on every replay, with eager work
and synchronisation between replays (graph nodes recorded by library calls are a known hazard)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("calls", ["never", "auto"])
def test_graph_replays_match_eager(calls):
    """calls="never" launches the captured graph, "auto" issues the recorded library calls again (the block's
    step is made of library kernels only, so that is what replay() must choose)."""
    import pyramid_dwconv
    from pyramidconvblock_amd.graphs import GraphedStep

    torch.manual_seed(0)
    m = pyramid_dwconv.ConvBlock(64, kernel_size=9).to(torch.bfloat16).cuda()
    gen = torch.Generator().manual_seed(1)
    x = torch.randn(4, 28, 30, 64, generator=gen).to(torch.bfloat16).cuda()
    g = torch.randn(4, 28, 30, 64, generator=gen).to(torch.bfloat16).cuda()
    step = GraphedStep(m, x, g, calls=calls)
    assert step.replays_calls == (calls == "auto")
    graph_grads = [step.x.grad] + step.param_grads

    def eager(xin):
        for p in m.parameters():
            p.grad = None
        xe = xin.detach().clone().requires_grad_()
        y = m(xe)
        torch.autograd.backward(y, step.grad_out)
        out = [y.detach().clone(), xe.grad.clone()] + [p.grad.clone() for p in m.parameters()]
        for p, gg in zip(m.parameters(), step.param_grads):
            p.grad = gg
        return out

    for rep in range(4):
        if rep == 2:  # new input data through the static buffers
            step.x.data.copy_(torch.randn(4, 28, 30, 64, generator=gen).to(torch.bfloat16))
        ref = eager(step.x)
        step.y.zero_()
        for t in graph_grads:
            t.zero_()
        torch.cuda.synchronize()
        step.replay()
        torch.cuda.synchronize()
        for got, want in zip([step.y] + graph_grads, ref):
            assert torch.equal(got, want), f"replay {rep} differs from eager"


def test_foreign_kernels_keep_the_graph():
    """A step with a kernel that is not the library's (a torch op in the module) must be replayed as a graph:
    the list of library calls would leave that kernel out."""
    import pyramid_dwconv
    from pyramidconvblock_amd.graphs import GraphedForward, GraphedStep

    class Wrapped(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.block = pyramid_dwconv.ConvBlock(32, kernel_size=5)

        def forward(self, x):
            return self.block(x) * 2

    torch.manual_seed(0)
    m = Wrapped().to(torch.float16).cuda()
    x = torch.randn(2, 12, 16, 32, device="cuda").to(torch.float16)
    g = torch.randn_like(x)
    step = GraphedStep(m, x, g)
    assert not step.replays_calls
    want = m(x).detach()
    assert torch.equal(step.replay(), want)
    fwd = GraphedForward(m.block, x)
    assert fwd.replays_calls
    with torch.no_grad():
        want = m.block(x)
    fwd.y.zero_()
    assert torch.equal(fwd.replay(), want)
