"""The library under HIP graph capture: every entry point only enqueues kernels on the
stream it is given (no allocation, no memset node, no synchronisation), so a caller may
capture forward + backward once and replay it.  Each replay is compared with the eager
result, with eager work and synchronisations between the replays.
"""
import pytest
import torch

import d2conv3d_amd as d2c
from _util import assert_close, rel_l2
from test_gpu_tiled import make

pytestmark = pytest.mark.gpu


def _step(ts, gout, geo):
    s, p, d, groups, G = geo
    for t in ts:
        if t is not None:
            t.grad = None
    out = d2c.deform_conv3d(*ts, s, p, d, groups, G)
    out.backward(gout)
    return out.detach(), [t.grad for t in ts]


@pytest.mark.parametrize("name,dtype", [("c128_G2_o96", torch.float32), ("c64_o320_big", torch.bfloat16),
                                        ("dw64", torch.float32), ("c64_tail", torch.bfloat16)])
def test_forward_backward_replays_from_a_graph(name, dtype, dev):
    (x, off, m, w, b), gout, geo = make(name, dtype, seed=5)
    ts = [t.to(dev).requires_grad_(True) if t is not None else None for t in (x, off, m, w, b)]
    gout = gout.to(dev)
    e_out, e_grads = _step(ts, gout, geo)
    e_out, e_grads = e_out.clone(), [g.clone() if g is not None else None for g in e_grads]

    # warm-up on a side stream, then capture (torch's protocol for graphs with autograd)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            _step(ts, gout, geo)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    for t in ts:
        if t is not None:
            t.grad = None
    with torch.cuda.graph(graph):
        out = d2c.deform_conv3d(*ts, *geo[:3], geo[3], geo[4])
        out.backward(gout)
    grads = [t.grad if t is not None else None for t in ts]

    tol = dict(rtol=1e-4, atol=1e-5) if dtype == torch.float32 else None
    for rep in range(3):
        out.zero_()
        for g in grads:
            if g is not None:
                g.fill_(7.0)                       # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        pairs = [("out", out, e_out)] + [(f"grad{i}", g, e) for i, (g, e) in enumerate(zip(grads, e_grads)) if g is not None]
        for n, a, e in pairs:
            if tol:
                assert_close(a, e, 1e-4, 1e-5 * max(1.0, e.abs().max().item()), f"{name} replay {rep} {n}")
            else:
                assert rel_l2(a, e) < 2e-2, (name, rep, n, rel_l2(a, e))


def test_plain_depthwise_conv_replays_from_a_graph(dev):
    """d2c_dwconv3d_forward / _backward under capture: its scratch is cleared by a fill kernel, not a memset node."""
    from d2conv3d_amd.depthwise_conv import depthwise_separable_conv3d
    g = torch.Generator().manual_seed(8)
    x = torch.randn(2, 16, 5, 12, 16, generator=g).to(dev).requires_grad_(True)
    w = (torch.randn(16, 1, 3, 3, 3, generator=g) / 5).to(dev).requires_grad_(True)
    b = torch.randn(16, generator=g).to(dev).requires_grad_(True)
    gout = torch.randn(2, 16, 5, 12, 16, generator=g).to(dev)
    ts = [x, w, b]

    def step():
        for t in ts:
            t.grad = None
        out = depthwise_separable_conv3d(x, w, b, 1, 1, 1)
        out.backward(gout)
        return out

    e_out = step().detach().clone()
    e_grads = [t.grad.clone() for t in ts]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    for t in ts:
        t.grad = None
    with torch.cuda.graph(graph):
        out = depthwise_separable_conv3d(x, w, b, 1, 1, 1)
        out.backward(gout)
    grads = [t.grad for t in ts]
    for rep in range(3):
        out.zero_()
        for gr in grads:
            gr.fill_(7.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert_close(out, e_out, 1e-5, 1e-6, f"replay {rep} out")
        for i, (a, e) in enumerate(zip(grads, e_grads)):
            assert_close(a, e, 1e-5, 1e-5 * max(1.0, e.abs().max().item()), f"replay {rep} grad{i}")
