"""fbfft_conv_fprop_static (the entry point that allocates nothing) against
fbfft_conv_fprop on the same operands, through the C ABI: two calls in a row, the
second on a smaller layer, so that what the first call left in the library's fixed
scratch array must not leak into the second."""
import numpy as np
import pytest
import torch

import fbcuda_amd as F
from fbcuda_amd import synth
from gpu_util import TOL_CONV, dev, rel

pytestmark = pytest.mark.gpu


def _layer(B, Cin, Cout, H, W, k, seed):
    x = synth.normal((B, Cin, H, W), seed=seed).to(dev())
    w = (0.05 * synth.normal((Cout, Cin, k, k), seed=seed + 1)).to(dev())
    return x, w


def _with_workspace(x, w, N):
    B, Cin, H, W = x.shape
    Cout, _, k, _ = w.shape
    out = torch.full((B, Cout, H - k + 1, W - k + 1), float("nan"), device=dev())
    ws = torch.empty(F.conv_fprop_workspace(B, Cin, Cout, N), dtype=torch.uint8, device=dev())
    assert F.conv_fprop(x, w, out, N, ws) == F.Success
    torch.cuda.synchronize()
    return out


def test_static_scratch_matches_workspace_form(oracle):
    # (B, Cin, Cout, H, W, k, fftSize): the second layer is smaller in every respect
    layers = [(16, 24, 40, 27, 27, 5, 32), (3, 5, 7, 13, 11, 3, 16)]
    outs = []
    for i, (B, Cin, Cout, H, W, k, N) in enumerate(layers):
        assert 0 < F.conv_fprop_workspace(B, Cin, Cout, N) <= F.STATIC_SCRATCH_BYTES
        x, w = _layer(B, Cin, Cout, H, W, k, 50 + 2 * i)
        out = torch.full((B, Cout, H - k + 1, W - k + 1), float("nan"), device=dev())
        assert F.conv_fprop_static(x, w, out, N) == F.Success
        outs.append((x, w, N, out))
    torch.cuda.synchronize()
    for x, w, N, out in outs:
        want = _with_workspace(x, w, N)
        got = out.cpu().numpy()
        assert np.isfinite(got).all()
        assert rel(got, want.cpu().numpy()) < TOL_CONV
        # the same kernels on the same launch geometry: identical bits
        assert np.array_equal(got, want.cpu().numpy())
    # and the smaller layer against the definition
    x, w, N, out = outs[1]
    want64 = oracle.corr2d_valid(x.cpu().numpy(), w.cpu().numpy())
    assert rel(out.cpu().numpy(), want64) < TOL_CONV


def test_static_scratch_under_graph_capture_and_without_allocation():
    """After one eager call (which looks the array up) the entry point can be captured into
    a HIP graph, every replay equals the workspace form on the inputs of that moment, and
    device memory in use is the same before and after the calls."""
    d = dev()
    B, Cin, Cout, H, W, k, N = 6, 10, 12, 27, 25, 5, 32
    x, w = _layer(B, Cin, Cout, H, W, k, 60)
    out = torch.full((B, Cout, H - k + 1, W - k + 1), float("nan"), device=d)
    empty_x = torch.zeros((0, Cin, H, W), device=d)
    empty_out = torch.zeros((0, Cout, H - k + 1, W - k + 1), device=d)
    new_x = [synth.normal(tuple(x.shape), seed=70 + r).to(d) for r in range(3)]
    torch.cuda.synchronize()
    # the set-up call: an empty batch, nothing launched
    assert F.conv_fprop_static(empty_x, w, empty_out, N) == F.Success
    _with_workspace(x, w, N)   # the layer's kernels have run once: their code is resident
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    for _ in range(3):
        assert F.conv_fprop_static(x, w, out, N) == F.Success
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0, "device memory in use changed across fbfft_conv_fprop_static"
    want = _with_workspace(x, w, N)
    assert torch.equal(out, want)

    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            assert F.conv_fprop_static(x, w, out, N, stream=stream) == F.Success
    torch.cuda.synchronize()
    for r in range(3):
        x.copy_(new_x[r])
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want = _with_workspace(x, w, N)   # eager work between the replays
        assert bool(torch.isfinite(out).all())
        assert torch.equal(out, want), "replay %d differs from the workspace form" % r


def test_static_scratch_rejects_layers_beyond_its_size():
    B, Cin, Cout, N = 128, 64, 192, 32
    assert F.conv_fprop_workspace(B, Cin, Cout, N) > F.STATIC_SCRATCH_BYTES
    x = torch.zeros((B, Cin, 27, 27), device=dev())
    w = torch.zeros((Cout, Cin, 5, 5), device=dev())
    out = torch.full((B, Cout, 23, 23), 7.0, device=dev())
    assert F.conv_fprop_static(x, w, out, N) == F.UnsupportedSize
    torch.cuda.synchronize()
    assert float((out - 7.0).abs().max()) == 0.0
