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


def test_static_scratch_rejects_layers_beyond_its_size():
    B, Cin, Cout, N = 128, 64, 192, 32
    assert F.conv_fprop_workspace(B, Cin, Cout, N) > F.STATIC_SCRATCH_BYTES
    x = torch.zeros((B, Cin, 27, 27), device=dev())
    w = torch.zeros((Cout, Cin, 5, 5), device=dev())
    out = torch.full((B, Cout, 23, 23), 7.0, device=dev())
    assert F.conv_fprop_static(x, w, out, N) == F.UnsupportedSize
    torch.cuda.synchronize()
    assert float((out - 7.0).abs().max()) == 0.0
