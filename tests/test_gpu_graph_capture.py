"""The entry points allocate nothing, sync nothing and clear memory with fill kernels only, so a
forward + backward can be captured into a HIP graph and replayed.  Every replay is checked against
the eager result on the inputs that are in the static buffers at that time, with eager work and
synchronisation between the replays."""

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_forward_backward_replays_from_a_graph():
    from verl_amd.utils.kernel import kernels

    T, H, V, tau = 600, 256, 5000, 0.8
    g = torch.Generator().manual_seed(7)

    def fresh():
        h = (torch.rand(T, H, generator=g) - 0.5).bfloat16().to(DEV)
        w = (torch.rand(V, H, generator=g) - 0.5).bfloat16().to(DEV)
        y = torch.randint(0, V, (T,), generator=g).to(DEV)
        g_lp = (torch.rand(T, generator=g) * 2 - 1).to(DEV) * (torch.rand(T, generator=g) < 0.7).to(DEV)
        g_ent = (torch.rand(T, generator=g) - 0.5).to(DEV)
        return h, w, y, g_lp, g_ent

    def run(h, w, y, g_lp, g_ent):
        lp, ent, mx, acc, eb = kernels.efficient_entropy_forward(h, w, y, 0, tau)
        dh, dw = kernels.efficient_entropy_backward(g_lp, g_ent, h, w, y, mx, acc, eb, 0, False, tau)
        return lp, ent, dh, dw

    static = fresh()
    side = torch.cuda.Stream(device=DEV)
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):  # warm-up outside the capture (attributes, lazy module loading)
            run(*static)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = run(*static)
    for it in range(4):
        new = fresh()
        for dst, src in zip(static, new):
            dst.copy_(src)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs]
        want = run(*new)  # eager, on private buffers
        torch.cuda.synchronize()
        for a, b in zip(got, want):
            assert torch.equal(a, b), it
