"""A training step of the mapped convolution captured into a HIP graph (through the framework's
graph API) and replayed: every replay must give the eager result, with other work of the
process running between replays.  The library launches kernels only (its fills are kernels,
not memset nodes) and keeps the bias gradient on the captured stream while a capture is on."""
import numpy as np
import pytest
import torch

from conftest import relerr

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_captured_step_replays_like_the_eager_one(oracle):
    from _spherical_distortion_ext import _ops as ops
    import workloads
    rng = np.random.default_rng(11)
    H, W, B, Cin, Cout, K = 32, 64, 2, 72, 80, 9
    base = workloads.gnomonic_kernel_map(H, W, dtype=np.float64)
    m, iw = workloads.four_nearest_weighted(base, H, W, dtype=np.float32)
    tm, tiw = torch.from_numpy(m).to(DEV), torch.from_numpy(iw).to(DEV)
    w = torch.from_numpy((rng.standard_normal((Cout, Cin, K)) / 25).astype(np.float32)).to(DEV)
    b = torch.from_numpy(rng.standard_normal(Cout).astype(np.float32)).to(DEV)
    x = torch.zeros(B, Cin, H, W, device=DEV)
    g = torch.zeros(B, Cout, H, W, device=DEV)

    def step():
        y = ops.mapped_conv_forward(x, tm, tiw, w, b, K, 2)
        gi, gw, gb = ops.mapped_conv_backward(g, tm, tiw, x, w, b, K, 2)
        return y, gi, gw, gb

    def fill(seed):
        r = np.random.default_rng(seed)
        x.copy_(torch.from_numpy(r.standard_normal(tuple(x.shape)).astype(np.float32)))
        g.copy_(torch.from_numpy(r.standard_normal(tuple(g.shape)).astype(np.float32)))

    fill(0)
    step()                                   # plans are built and cached outside the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step()
    for seed in (1, 2, 3):
        fill(seed)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in outs]
        want = step()                        # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(got[0], want[0])                       # forward: the same bits
        assert torch.equal(got[1], want[1])                       # grad_input over sorted lists
        assert relerr(got[2].cpu().numpy(), want[2].cpu().numpy()) <= 1e-6
        assert relerr(got[3].cpu().numpy(), want[3].cpu().numpy()) <= 1e-6
    yo = oracle.mapped_conv_forward(x.cpu().numpy(), m, w.cpu().numpy(), b.cpu().numpy(), K, 2, iw)
    assert relerr(got[0].cpu().numpy(), yo) <= 1e-5


def test_captured_backward_of_a_large_layer():
    """grad_output of 512 MiB: eager calls fork the bias gradient onto the library's side stream,
    a captured call must not (and must still be right)."""
    from _spherical_distortion_ext import _ops as ops
    import workloads
    H, W, B, C, K = 256, 512, 8, 128, 9
    base = workloads.gnomonic_kernel_map(H, W, dtype=np.float64)
    m, iw = workloads.four_nearest_weighted(base, H, W, dtype=np.float32)
    tm, tiw = torch.from_numpy(m).to(DEV), torch.from_numpy(iw).to(DEV)
    gen = torch.Generator(device=DEV).manual_seed(5)
    x = torch.randn(B, C, H, W, device=DEV, generator=gen)
    g = torch.randn(B, C, H, W, device=DEV, generator=gen)
    w = torch.randn(C, C, K, device=DEV, generator=gen) / 30
    b = torch.randn(C, device=DEV, generator=gen)
    want = ops.mapped_conv_backward(g, tm, tiw, x, w, b, K, 2)      # eager: side stream
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ops.mapped_conv_backward(g, tm, tiw, x, w, b, K, 2)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = ops.mapped_conv_backward(g, tm, tiw, x, w, b, K, 2)
    for _ in range(2):
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(outs[0], want[0])
        assert relerr(outs[1].cpu().numpy(), want[1].cpu().numpy()) <= 1e-6
        assert relerr(outs[2].cpu().numpy(), want[2].cpu().numpy()) <= 1e-6
        want = ops.mapped_conv_backward(g, tm, tiw, x, w, b, K, 2)  # eager work in between
        torch.cuda.synchronize()
    exact = g.double().sum(dim=(0, 2, 3)).float()
    assert relerr(outs[2].cpu().numpy(), exact.cpu().numpy()) <= 1e-6
