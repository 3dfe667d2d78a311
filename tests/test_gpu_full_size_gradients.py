"""Gradient passes at the sizes the benchmark times them on: configs[3] and configs[4]
of the convolution, through every route that has a timing (the layer entry points, the
fused tiled kernel, the tiled kernel's workspace form), each checked against the fp64
gradients of the direct correlation on seeded subsets that include borders and window
seams."""
import numpy as np
import pytest
import torch

import fbcuda_amd as F
from fbcuda_amd import synth
from gpu_util import TOL_CONV, check, dev, rel

pytestmark = pytest.mark.gpu


def grad_input_coords(rng, Nb, Cin, H, W, n, special):
    c = np.stack([rng.integers(0, Nb, n), rng.integers(0, Cin, n), rng.integers(0, H, n),
                  rng.integers(0, W, n)], axis=1).astype(np.int32)
    c[:len(special), 2:] = special
    return c


def grad_weight_coords(rng, Cout, Cin, k, n):
    c = np.stack([rng.integers(0, Cout, n), rng.integers(0, Cin, n), rng.integers(0, k, n),
                  rng.integers(0, k, n)], axis=1).astype(np.int32)
    c[:4] = [[0, 0, 0, 0], [Cout - 1, Cin - 1, k - 1, k - 1], [0, Cin - 1, 0, k - 1],
             [Cout - 1, 0, k - 1, 0]]
    return c


def at(t, coords):
    h = t.cpu().numpy()
    return h[coords[:, 0], coords[:, 1], coords[:, 2], coords[:, 3]]


def ws_bytes(nbytes):
    return torch.empty(nbytes, dtype=torch.uint8, device=dev())


def test_config3_gradients_through_the_layer_entry_points(oracle):
    """configs[3]: 128x64x27x27, 192x64x5x5, gradOutput 128x192x23x23, 32-point transforms.
    gradInput on 4096 seeded elements (corners and edges first), gradWeight on 512."""
    d = dev()
    x = synth.normal((128, 64, 27, 27), seed=30, device=d)
    w = synth.normal((192, 64, 5, 5), seed=31, std=0.02, device=d)
    g = synth.normal((128, 192, 23, 23), seed=32, device=d)
    gi = torch.full_like(x, float("nan"))
    gw = torch.full_like(w, float("nan"))
    assert F.conv_bprop(g, w, gi, 32, ws_bytes(F.conv_workspace(1, 128, 64, 192, 32))) == F.Success
    assert F.conv_accgrad(x, g, gw, 32, ws_bytes(F.conv_workspace(2, 128, 64, 192, 32))) == F.Success
    torch.cuda.synchronize()
    assert bool(torch.isfinite(gi).all()) and bool(torch.isfinite(gw).all())
    xh, wh, gh = x.cpu().numpy(), w.cpu().numpy(), g.cpu().numpy()
    rng = np.random.default_rng(35)
    ci = grad_input_coords(rng, 128, 64, 27, 27, 4096,
                           [[0, 0], [26, 26], [0, 26], [26, 0], [4, 4], [22, 22], [3, 23], [13, 0]])
    check("configs[3] fbfft_conv_bprop vs fp64 (4096 elements)", at(gi, ci),
          oracle.corr2d_grad_input_at(gh, wh, 27, 27, ci), TOL_CONV)
    cw = grad_weight_coords(rng, 192, 64, 5, 512)
    check("configs[3] fbfft_conv_accgrad vs fp64 (512 elements)", at(gw, cw),
          oracle.corr2d_grad_weight_at(xh, gh, 5, 5, cw), TOL_CONV)


@pytest.fixture(scope="module")
def config4():
    d = dev()
    x = synth.uniform((16, 32, 256, 256), seed=40, device=d)
    w = synth.normal((32, 32, 9, 9), seed=41, std=0.05, device=d)
    g = synth.normal((16, 32, 248, 248), seed=42, device=d)
    rng = np.random.default_rng(48)
    # seams of the input-gradient grid (windows of 24) and of the shared grid, corners, edges
    ci = grad_input_coords(rng, 16, 32, 256, 256, 4096,
                           [[0, 0], [255, 255], [0, 255], [255, 0], [23, 24], [24, 23], [47, 48],
                            [239, 240], [240, 239], [7, 8], [8, 7], [247, 248], [248, 247]])
    cw = grad_weight_coords(rng, 32, 32, 9, 256)
    return x, w, g, ci, cw


@pytest.fixture(scope="module")
def config4_reference(oracle, config4):
    x, w, g, ci, cw = config4
    xh, wh, gh = x.cpu().numpy(), w.cpu().numpy(), g.cpu().numpy()
    return (oracle.corr2d_grad_input_at(gh, wh, 256, 256, ci),
            oracle.corr2d_grad_weight_at(xh, gh, 9, 9, cw))


def test_config4_gradients_through_the_layer_entry_points(config4, config4_reference):
    """configs[4] (121 windows of 32x32 per image) through fbfft_conv_bprop / fbfft_conv_accgrad."""
    x, w, g, ci, cw = config4
    want_i, want_w = config4_reference
    gi = torch.full_like(x, float("nan"))
    gw = torch.full_like(w, float("nan"))
    assert F.conv_bprop(g, w, gi, 32,
                        ws_bytes(F.conv_workspace_image(1, 16, 32, 32, 256, 256, 9, 9, 32))) == F.Success
    assert F.conv_accgrad(x, g, gw, 32,
                          ws_bytes(F.conv_workspace_image(2, 16, 32, 32, 256, 256, 9, 9, 32))) == F.Success
    torch.cuda.synchronize()
    assert bool(torch.isfinite(gi).all()) and bool(torch.isfinite(gw).all())
    check("configs[4] fbfft_conv_bprop vs fp64 (4096 elements)", at(gi, ci), want_i, TOL_CONV)
    check("configs[4] fbfft_conv_accgrad vs fp64 (256 elements)", at(gw, cw), want_w, TOL_CONV)


@pytest.mark.parametrize("route", ["fused", "workspace"])
def test_config4_gradients_through_the_tile_descriptors(config4, config4_reference, route):
    """configs[4] on FFTIteratedConvolution's own operands: updateGradInput on the grid of
    disjoint gradInput windows, accGradParameters on the forward pass's grid - the fused
    kernel (fbfft_iterated_conv) and the workspace form (fbfft_iterated_conv_ws)."""
    x, w, g, ci, cw = config4
    want_i, want_w = config4_reference

    def run(ins, outs, weight, pass_, n):
        if route == "fused":
            ok = F.FFTIteratedConvolution(32, ins, outs, weight, pass_, 1.0, 16, n)
        else:
            nbytes = F.iterated_conv_workspace(32, pass_, 16, n, 32, 32)
            ok = F.FFTIteratedConvolutionWS(32, ins, outs, weight, pass_, 1.0, 16, n, ws_bytes(nbytes))
        torch.cuda.synchronize()
        return ok

    gi = torch.full_like(x, float("nan"))
    bins, bouts, nb = F.make_tile_grid(gi, g, 9, 9, 32, F.FFT_UpdateGradInput)
    assert nb == 121
    assert run(bins, bouts, w, F.FFT_UpdateGradInput, nb)
    assert bool(torch.isfinite(gi).all())
    check("configs[4] updateGradInput, %s route, vs fp64" % route, at(gi, ci), want_i, TOL_CONV)

    gw = torch.full_like(w, float("nan"))
    ins, outs, n = F.make_tile_grid(x, g, 9, 9, 32)
    assert n == 121
    assert run(ins, outs, gw, F.FFT_AccGradParameters, n)
    assert bool(torch.isfinite(gw).all())
    check("configs[4] accGradParameters, %s route, vs fp64" % route, at(gw, cw), want_w, TOL_CONV)
