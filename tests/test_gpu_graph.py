"""A captured forward+backward step must give the eager results on every replay, with eager work
and synchronisation between replays (graph nodes recorded by library calls are a known hazard)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dim", [64, 128])  # 128: the block runs as one library call per direction
def test_graph_replays_match_eager(dim):
    import pyramid_dwconv
    from pyramidconvblock_amd.graphs import GraphedStep

    torch.manual_seed(0)
    m = pyramid_dwconv.ConvBlock(dim, kernel_size=9).to(torch.bfloat16).cuda()
    gen = torch.Generator().manual_seed(1)
    x = torch.randn(4, 28, 32, dim, generator=gen).to(torch.bfloat16).cuda()
    g = torch.randn(4, 28, 32, dim, generator=gen).to(torch.bfloat16).cuda()
    step = GraphedStep(m, x, g)
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
            step.x.data.copy_(torch.randn(4, 28, 32, dim, generator=gen).to(torch.bfloat16))
        ref = eager(step.x)
        step.y.zero_()
        for t in graph_grads:
            t.zero_()
        torch.cuda.synchronize()
        step.replay()
        torch.cuda.synchronize()
        for got, want in zip([step.y] + graph_grads, ref):
            assert torch.equal(got, want), f"replay {rep} differs from eager"
