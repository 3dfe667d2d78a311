"""GPU parity of the convolution layer on images LARGER than the transform
(fbfft_conv_fprop / bprop / accgrad with fftSize <= 32 and H, W > fftSize): the
image is cut into the overlapping windows of FFTIteratedConvolution's tiling
(fbfft/FFTIteratedConvolution.cuh:71-88) and the windows go through the bin-major
pipeline.  Checked against fp64 direct correlation and its gradients."""
import numpy as np
import pytest
import torch

import fbcuda_amd as F
from fbcuda_amd import synth
from gpu_util import check, TOL_CONV, dev, rel

pytestmark = pytest.mark.gpu


def ws(pass_, Bn, Cin, Cout, H, W, k, N):
    n = F.conv_workspace_image(pass_, Bn, Cin, Cout, H, W, k, k, N)
    assert n > 0
    return torch.empty(n, dtype=torch.uint8, device=dev())


SHAPES = [
    # N, H, W, k, B, Cin, Cout
    (8, 14, 17, 3, 3, 5, 7),        # ragged edge tiles both ways
    (16, 30, 25, 5, 2, 3, 4),
    (32, 40, 56, 9, 2, 3, 4),
    (32, 33, 32, 5, 3, 4, 5),       # one extra row of tiles holding a single output row
    (16, 16, 40, 3, 2, 2, 3),       # tiled along x only
    (8, 50, 9, 1, 4, 2, 9),         # 1 x 1 filter: windows do not overlap
    (16, 37, 37, 16, 1, 2, 2),      # filter as large as the transform: one output per tile
    (32, 70, 64, 7, 5, 18, 33),     # several plane groups per workgroup row
    (16, 31, 33, 4, 3, 3, 3),       # even filter: odd window origins (4-byte load path)
    # few planes, many windows: the weight gradient is a short-sided product with a long
    # reduction, which the register kernels cut into ranges (partials added by the inverse)
    (8, 30, 30, 3, 24, 3, 5),       # both sides short: four ranges
    (8, 30, 30, 3, 24, 3, 40),      # one side short: sixteen ranges
    (16, 40, 40, 5, 40, 4, 6),      # 16-point windows: two ranges
    (8, 30, 30, 3, 24, 40, 48),     # no short side: the LDS kernel's reduction in four ranges
]


@pytest.mark.parametrize("N,H,W,k,Bn,Cin,Cout", SHAPES)
def test_tiled_layer_three_passes(oracle, N, H, W, k, Bn, Cin, Cout):
    d = dev()
    x = synth.uniform((Bn, Cin, H, W), seed=40, device=d)
    w = synth.normal((Cout, Cin, k, k), seed=41, std=0.05, device=d)
    xh, wh = x.cpu().numpy(), w.cpu().numpy()
    out = torch.full((Bn, Cout, H - k + 1, W - k + 1), float("nan"), device=d)
    assert F.conv_fprop(x, w, out, N, ws(0, Bn, Cin, Cout, H, W, k, N)) == F.Success
    torch.cuda.synchronize()
    assert rel(out.cpu().numpy(), oracle.corr2d_valid(xh, wh)) < TOL_CONV

    g = synth.normal(tuple(out.shape), seed=42, device=d)
    gh = g.cpu().numpy()
    gi = torch.full_like(x, float("nan"))
    assert F.conv_bprop(g, w, gi, N, ws(1, Bn, Cin, Cout, H, W, k, N)) == F.Success
    torch.cuda.synchronize()
    assert rel(gi.cpu().numpy(), oracle.corr2d_grad_input(gh, wh, H, W)) < TOL_CONV

    gw0 = synth.normal(tuple(w.shape), seed=43, device=d)
    for accumulate in (False, True):
        gw = gw0.clone() if accumulate else torch.full_like(w, float("nan"))
        assert F.conv_accgrad(x, g, gw, N, ws(2, Bn, Cin, Cout, H, W, k, N), scale=0.5,
                              accumulate=accumulate) == F.Success
        torch.cuda.synchronize()
        want = 0.5 * oracle.corr2d_grad_weight(xh, gh, k, k) + (gw0.cpu().numpy() if accumulate else 0.0)
        assert rel(gw.cpu().numpy(), want) < TOL_CONV


def test_tiled_layer_strided_operands(oracle):
    """Views with gaps between rows, planes and images, and an odd base offset."""
    N, H, W, k, Bn, Cin, Cout = 16, 29, 35, 3, 2, 3, 4
    d = dev()
    store = synth.uniform((Bn, Cin + 1, H + 2, W + 3), seed=44, device=d)
    x = store[:, 1:, 1:H + 1, 1:W + 1]
    w = synth.normal((Cout, Cin, k, k), seed=45, std=0.05, device=d)
    ostore = torch.full((Bn, Cout, H - k + 3, W - k + 2), float("nan"), device=d)
    out = ostore[:, :, 2:, 1:]
    assert F.conv_fprop(x, w, out, N, ws(0, Bn, Cin, Cout, H, W, k, N)) == F.Success
    torch.cuda.synchronize()
    want = oracle.corr2d_valid(x.contiguous().cpu().numpy(), w.cpu().numpy())
    assert rel(out.cpu().numpy(), want) < TOL_CONV
    assert bool(torch.isnan(ostore[:, :, :2]).all()) and bool(torch.isnan(ostore[:, :, :, 0]).all())


def test_tiled_layer_argument_checks():
    d = dev()
    x = torch.zeros(1, 2, 80, 80, device=d)
    w = torch.zeros(3, 2, 5, 5, device=d)
    o = torch.zeros(1, 3, 76, 76, device=d)
    big = torch.empty(F.conv_workspace_image(0, 1, 2, 3, 80, 80, 5, 5, 32), dtype=torch.uint8, device=d)
    assert F.conv_fprop(x, w, o, 32, big) == F.Success
    # the workspace of a one-tile layer is too small for the tiled one
    small = torch.empty(F.conv_workspace(0, 1, 2, 3, 32), dtype=torch.uint8, device=d)
    assert F.conv_fprop(x, w, o, 32, small) == F.UnsupportedDimension
    # 64- and 128-point layers are not tiled
    assert F.conv_workspace_image(0, 1, 2, 3, 80, 80, 5, 5, 64) == 0
    assert F.conv_fprop(x, w, o, 64, big) == F.UnsupportedSize
    # equal to the plain query when the image fits
    assert F.conv_workspace_image(1, 4, 5, 6, 27, 27, 5, 5, 32) == F.conv_workspace(1, 4, 5, 6, 32)
    torch.cuda.synchronize()


def test_config4_through_the_layer_entry_point(oracle):
    """configs[4]: 16x32x256x256 * 32x32x9x9 -> 16x32x248x248 with 32-point transforms
    (121 windows per image); fp64 direct correlation on 4096 seeded output pixels, seams
    and corners included."""
    d = dev()
    x = synth.uniform((16, 32, 256, 256), seed=40, device=d)
    w = synth.normal((32, 32, 9, 9), seed=41, std=0.05, device=d)
    out = torch.full((16, 32, 248, 248), float("nan"), device=d)
    assert F.conv_fprop(x, w, out, 32, ws(0, 16, 32, 32, 256, 256, 9, 32)) == F.Success
    torch.cuda.synchronize()
    assert bool(torch.isfinite(out).all())
    rng = np.random.default_rng(47)
    coords = np.stack([rng.integers(0, 16, 4096), rng.integers(0, 32, 4096),
                       rng.integers(0, 248, 4096), rng.integers(0, 248, 4096)], axis=1).astype(np.int32)
    coords[:8, 2:] = [[0, 0], [247, 247], [23, 24], [24, 23], [239, 240], [240, 239], [0, 247], [247, 0]]
    want = oracle.corr2d_valid_at(x.cpu().numpy(), w.cpu().numpy(), coords)
    oh = out.cpu().numpy()
    got = oh[coords[:, 0], coords[:, 1], coords[:, 2], coords[:, 3]]
    check("configs[4] fbfft_conv_fprop vs fp64 (4096 pixels)", got, want, TOL_CONV)


@pytest.mark.parametrize("H,W,k", [(60, 60, 5), (14, 12, 3), (8, 8, 3), (27, 27, 5)])
def test_fft_size_zero_is_the_library_choice(oracle, H, W, k):
    """fftSize = 0: each pass runs on fbfft_conv_choose_fft_size's transform for that pass
    and gives that transform's results bit for bit."""
    d = dev()
    Bn, Cin, Cout = 3, 4, 5
    x = synth.uniform((Bn, Cin, H, W), seed=40, device=d)
    w = synth.normal((Cout, Cin, k, k), seed=41, std=0.05, device=d)
    g = synth.normal((Bn, Cout, H - k + 1, W - k + 1), seed=42, device=d)
    chosen = [F.conv_choose_fft_size(p, Bn, Cin, Cout, H, W, k, k) for p in range(3)]
    assert all(N in (8, 16, 32) for N in chosen)
    res = []
    for sizes in ((0, 0, 0), chosen):
        out, gi, gw = torch.empty_like(g), torch.empty_like(x), torch.empty_like(w)
        assert F.conv_fprop(x, w, out, sizes[0], ws(0, Bn, Cin, Cout, H, W, k, sizes[0])) == F.Success
        assert F.conv_bprop(g, w, gi, sizes[1], ws(1, Bn, Cin, Cout, H, W, k, sizes[1])) == F.Success
        assert F.conv_accgrad(x, g, gw, sizes[2], ws(2, Bn, Cin, Cout, H, W, k, sizes[2])) == F.Success
        torch.cuda.synchronize()
        res.append((out, gi, gw))
    for a, b in zip(*res):
        assert torch.equal(a, b)
    xh, wh, gh = x.cpu().numpy(), w.cpu().numpy(), g.cpu().numpy()
    assert rel(res[0][0].cpu().numpy(), oracle.corr2d_valid(xh, wh)) < TOL_CONV
    assert rel(res[0][1].cpu().numpy(), oracle.corr2d_grad_input(gh, wh, H, W)) < TOL_CONV
    assert rel(res[0][2].cpu().numpy(), oracle.corr2d_grad_weight(xh, gh, k, k)) < TOL_CONV
    out = torch.empty_like(g)
    assert F.conv_fprop_static(x, w, out, 0) == F.Success
    torch.cuda.synchronize()
    assert torch.equal(out, res[0][0])
