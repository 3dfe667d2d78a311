"""The entry points allocate nothing and only enqueue kernels on the caller's
stream, so a HIP graph can capture them.  Every replay is checked against the
eager result, with eager work and synchronisation between replays."""
import pytest
import torch

import fbcuda_amd as F
from fbcuda_amd import synth
from gpu_util import dev

pytestmark = pytest.mark.gpu


def test_graph_capture_of_the_convolution_layer_and_transforms():
    d = dev()
    x = synth.normal((8, 6, 27, 27), seed=30, device=d)
    w = synth.normal((10, 6, 5, 5), seed=31, std=0.02, device=d)
    g = synth.normal((8, 10, 23, 23), seed=32, device=d)
    planes = synth.normal((300, 32, 32), seed=1, device=d)
    out, gi, gw = torch.empty_like(g), torch.empty_like(x), torch.empty_like(w)
    spec = torch.empty((300, 17, 32, 2), device=d)
    back = torch.empty_like(planes)
    ws = [torch.empty(F.conv_workspace(p, 8, 6, 10, 32), dtype=torch.uint8, device=d) for p in range(3)]

    def run():
        assert F.conv_fprop(x, w, out, 32, ws[0]) == F.Success
        assert F.conv_bprop(g, w, gi, 32, ws[1]) == F.Success
        assert F.conv_accgrad(x, g, gw, 32, ws[2], scale=0.5) == F.Success
        assert F.fbfft2D(planes, spec) == F.Success
        assert F.fbifft2D(spec, back) == F.Success

    run()
    torch.cuda.synchronize()
    want = [t.clone() for t in (out, gi, gw, spec, back)]

    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        run()  # warm-up on the capture stream
        stream.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            run()
    torch.cuda.synchronize()

    for rep in range(3):
        # new inputs each time: a replay must recompute, not return stale memory
        x.copy_(synth.normal(tuple(x.shape), seed=40 + rep, device=d))
        planes.copy_(synth.normal(tuple(planes.shape), seed=50 + rep, device=d))
        for t in (out, gi, gw, spec, back):
            t.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in (out, gi, gw, spec, back)]
        run()  # eager, same inputs
        torch.cuda.synchronize()
        for a, b in zip(got, (out, gi, gw, spec, back)):
            assert bool(torch.isfinite(a).all())
            assert torch.equal(a, b), "replay %d differs from the eager result" % rep
    assert not torch.equal(want[0], out)  # the inputs did change


def test_graph_capture_of_the_tiled_convolution():
    """All three passes of FFTIteratedConvolution in one graph (the weight-gradient
    pass clears its output with a fill kernel, which a graph can hold)."""
    d = dev()
    x = synth.uniform((4, 6, 40, 56), seed=40, device=d)
    w = synth.normal((5, 6, 9, 9), seed=41, std=0.05, device=d)
    out = torch.empty((4, 5, 32, 48), device=d)
    g = synth.normal(tuple(out.shape), seed=42, device=d)
    gi, gw = torch.empty_like(x), torch.empty_like(w)
    ins, outs, n = F.make_tile_grid(x, out, 9, 9, 32)
    gins, gouts, n2 = F.make_tile_grid(gi, g, 9, 9, 32)
    ains, aouts, n3 = F.make_tile_grid(x, g, 9, 9, 32)

    def run():
        assert F.FFTIteratedConvolution(32, ins, outs, w, F.FFT_UpdateOutput, 1.0, 4, n)
        assert F.FFTIteratedConvolution(32, gins, gouts, w, F.FFT_UpdateGradInput, 1.0, 4, n2)
        assert F.FFTIteratedConvolution(32, ains, aouts, gw, F.FFT_AccGradParameters, 0.5, 4, n3)

    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        run()
        stream.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            run()
    torch.cuda.synchronize()
    for rep in range(3):
        x.copy_(synth.uniform(tuple(x.shape), seed=60 + rep, device=d))
        for t in (out, gi, gw):
            t.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in (out, gi, gw)]
        run()
        torch.cuda.synchronize()
        assert torch.equal(got[0], out)
        # updateGradInput writes each tile's whole input window; where windows overlap
        # the last writer wins (as in the reference), so only cells that a single tile
        # covers are comparable from run to run: rows and columns below the tile step
        assert bool(torch.isfinite(got[1]).all())
        assert torch.equal(got[1][:, :, :24, :24], gi[:, :, :24, :24])
        # partial gradients meet in atomic adds: equal to rounding, not bit for bit
        assert bool(torch.isfinite(got[2]).all())
        assert float((got[2] - gw).norm() / gw.norm()) < 1e-5


def test_graph_capture_of_the_workspace_tiled_convolution_and_size_choice():
    """fbfft_iterated_conv_ws (tile descriptors read on the device, contraction launched on
    a two-dimensional grid) and the layer entry points with fftSize 0 under capture."""
    d = dev()
    x = synth.uniform((4, 6, 40, 56), seed=40, device=d)
    w = synth.normal((5, 6, 9, 9), seed=41, std=0.05, device=d)
    out = torch.empty((4, 5, 32, 48), device=d)
    out0 = torch.empty_like(out)
    g = synth.normal(tuple(out.shape), seed=42, device=d)
    gi, gw = torch.empty_like(x), torch.empty_like(w)
    ins, outs, n = F.make_tile_grid(x, out, 9, 9, 32)
    gins, gouts, n2 = F.make_tile_grid(gi, g, 9, 9, 32, F.FFT_UpdateGradInput)
    ains, aouts, n3 = F.make_tile_grid(x, g, 9, 9, 32)
    wsd = [torch.empty(F.iterated_conv_workspace(32, p, 4, m, 6, 5), dtype=torch.uint8, device=d)
           for p, m in ((0, n), (1, n2), (2, n3))]
    ws0 = torch.empty(F.conv_workspace_image(0, 4, 6, 5, 40, 56, 9, 9, 0), dtype=torch.uint8, device=d)

    def run():
        assert F.FFTIteratedConvolutionWS(32, ins, outs, w, F.FFT_UpdateOutput, 1.0, 4, n, wsd[0])
        assert F.FFTIteratedConvolutionWS(32, gins, gouts, w, F.FFT_UpdateGradInput, 1.0, 4, n2, wsd[1])
        assert F.FFTIteratedConvolutionWS(32, ains, aouts, gw, F.FFT_AccGradParameters, 0.5, 4, n3,
                                          wsd[2])
        assert F.conv_fprop(x, w, out0, 0, ws0) == F.Success

    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        run()
        stream.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            run()
    torch.cuda.synchronize()
    for rep in range(3):
        x.copy_(synth.uniform(tuple(x.shape), seed=60 + rep, device=d))
        for t in (out, out0, gi, gw):
            t.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in (out, out0, gi, gw)]
        run()
        torch.cuda.synchronize()
        for a, b in zip(got, (out, out0, gi, gw)):
            assert bool(torch.isfinite(a).all())
            assert torch.equal(a, b), "replay %d differs from the eager result" % rep
        assert float((out - out0).norm() / out0.norm()) < 1e-5
