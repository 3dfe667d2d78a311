"""GPU parity of fbfft_iterated_conv_ws: FFTIteratedConvolution's operands (device
arrays of tile descriptors, fbfft/FFTIteratedConvolution.cuh:71-88, 624-755) through
a caller-owned workspace and the three kernels of the layer entry points.  Checked
against the CPU transcription on the same descriptors, against fp64 direct
correlation and its gradients, and against the fused kernel (fbfft_iterated_conv)."""
import numpy as np
import pytest
import torch

import fbcuda_amd as F
from fbcuda_amd import synth
from gpu_util import check, TOL_CONV, dev, rel
from test_gpu_iterated_conv import tiles_for

pytestmark = pytest.mark.gpu


def workspace(N, pass_, Nb, n, Cin, Cout):
    nbytes = F.iterated_conv_workspace(N, pass_, Nb, n, Cin, Cout)
    assert nbytes > 0
    return torch.empty(nbytes, dtype=torch.uint8, device=dev())


def run_ws(N, ins, outs, w, pass_, scale, Nb, n):
    Cout, Cin = w.shape[0], w.shape[1]
    ok = F.FFTIteratedConvolutionWS(N, ins, outs, w, pass_, scale, Nb, n,
                                    workspace(N, pass_, Nb, n, Cin, Cout))
    torch.cuda.synchronize()
    return ok


@pytest.mark.parametrize("N,k,H,W,Nb,Cin,Cout", [
    (8, 3, 14, 17, 3, 5, 7),
    (16, 5, 30, 25, 2, 3, 4),
    (32, 9, 40, 56, 2, 3, 4),
    (32, 5, 32, 32, 5, 9, 10),
    (8, 1, 9, 9, 17, 2, 33),
    (32, 7, 70, 64, 3, 40, 36),     # more than 32 planes on both sides: the LDS contraction
    (16, 4, 31, 33, 3, 3, 3),       # even filter: odd window origins
])
def test_three_passes_vs_oracle_and_fused_kernel(oracle, N, k, H, W, Nb, Cin, Cout):
    d = dev()
    x = synth.uniform((Nb, Cin, H, W), seed=40, device=d)
    w = synth.normal((Cout, Cin, k, k), seed=41, std=0.05, device=d)
    xh, wh = x.cpu().numpy(), w.cpu().numpy()
    iv, ov = tiles_for(H, W, k, N)
    oshape = (Nb, Cout, H - k + 1, W - k + 1)

    # updateOutput
    out = torch.full(oshape, float("nan"), device=d)
    ins, n = F.make_tiles(x, iv)
    outs, _ = F.make_tiles(out, ov)
    assert run_ws(N, ins, outs, w, F.FFT_UpdateOutput, 1.0, Nb, n)
    got = out.cpu().numpy()
    want = np.zeros(oshape, np.float32)
    assert oracle.iterated_conv(N, xh.copy(), iv, want, ov, wh, 0) == 1
    assert rel(got, want) < TOL_CONV
    assert rel(got, oracle.corr2d_valid(xh, wh)) < TOL_CONV
    fused = torch.full(oshape, float("nan"), device=d)
    fouts, _ = F.make_tiles(fused, ov)
    assert F.FFTIteratedConvolution(N, ins, fouts, w, F.FFT_UpdateOutput, 1.0, Nb, n)
    torch.cuda.synchronize()
    assert rel(got, fused.cpu().numpy()) < 1e-5

    # accGradParameters (overwrites weight with scale * gradient)
    g = synth.normal(oshape, seed=42, device=d)
    gh = g.cpu().numpy()
    gouts, _ = F.make_tiles(g, ov)
    gw = torch.full_like(w, float("nan"))
    assert run_ws(N, ins, gouts, gw, F.FFT_AccGradParameters, 0.5, Nb, n)
    gw_want = np.zeros_like(wh)
    assert oracle.iterated_conv(N, xh.copy(), iv, gh.copy(), ov, gw_want, 2, 0.5) == 1
    assert rel(gw.cpu().numpy(), gw_want) < TOL_CONV
    assert rel(gw.cpu().numpy(), 0.5 * oracle.corr2d_grad_weight(xh, gh, k, k)) < TOL_CONV

    # updateGradInput on its own grid (disjoint gradInput windows)
    gin = torch.full_like(x, 7.0)
    bins, bouts, nb = F.make_tile_grid(gin, g, k, k, N, F.FFT_UpdateGradInput)
    assert run_ws(N, bins, bouts, w, F.FFT_UpdateGradInput, 1.0, Nb, nb)
    assert rel(gin.cpu().numpy(), oracle.corr2d_grad_input(gh, wh, H, W)) < TOL_CONV


def test_padded_descriptors_and_ragged_views(oracle):
    """padL / padU inside the descriptors shift the data within the FFT plane; a batch
    larger than a view's image count and a filter with more planes than a view holds
    read zeros there, as in the fused kernel."""
    N, k, Nb, Cin, Cout = 16, 3, 2, 2, 3
    d = dev()
    x = synth.uniform((Nb, Cin, 10, 11), seed=45, device=d)
    w = synth.normal((Cout, Cin, k, k), seed=46, std=0.05, device=d)
    iv = [(0, 0, 10, 11, 2, 3)]
    ov = [(0, 0, 8, 9, 2, 3)]
    out = torch.full((Nb, Cout, 8, 9), float("nan"), device=d)
    ins, n = F.make_tiles(x, iv)
    outs, _ = F.make_tiles(out, ov)
    assert run_ws(N, ins, outs, w, F.FFT_UpdateOutput, 1.0, Nb, n)
    want = np.zeros((Nb, Cout, 8, 9), np.float32)
    assert oracle.iterated_conv(N, x.cpu().numpy(), iv, want, ov, w.cpu().numpy(), 0) == 1
    assert rel(out.cpu().numpy(), want) < TOL_CONV
    assert rel(out.cpu().numpy(), oracle.corr2d_valid(x.cpu().numpy(), w.cpu().numpy())) < TOL_CONV
    # batchSize 3 on views that hold 2 images, and a filter with one more input plane than
    # the input view holds: the extra image stores nothing, the extra plane adds nothing
    w2 = torch.cat([w, synth.normal((Cout, 1, k, k), seed=47, std=0.05, device=d)], dim=1).contiguous()
    out2 = torch.full((Nb, Cout, 8, 9), float("nan"), device=d)
    outs2, _ = F.make_tiles(out2, ov)
    assert run_ws(N, ins, outs2, w2, F.FFT_UpdateOutput, 1.0, Nb + 1, n)
    assert torch.equal(out2, out)
    fused = torch.full((Nb, Cout, 8, 9), float("nan"), device=d)
    fouts, _ = F.make_tiles(fused, ov)
    assert F.FFTIteratedConvolution(N, ins, fouts, w2, F.FFT_UpdateOutput, 1.0, Nb + 1, n)
    torch.cuda.synchronize()
    assert rel(out2.cpu().numpy(), fused.cpu().numpy()) < 1e-5


def test_strided_views_odd_strides(oracle):
    """Descriptors over non-contiguous tensors with odd row strides: 4-byte accesses."""
    N, k, Nb, Cin, Cout, H, W = 16, 3, 2, 3, 2, 20, 23
    d = dev()
    xbig = synth.uniform((Nb, Cin, H + 1, W + 2), seed=48, device=d)
    x = xbig[:, :, 1:, 1:W + 1]
    w = synth.normal((Cout, Cin, k, k), seed=49, std=0.05, device=d)
    obig = torch.full((Nb, Cout, H - k + 1, W - k + 4), float("nan"), device=d)
    out = obig[:, :, :, 3:]
    iv, ov = tiles_for(H, W, k, N)
    ins, n = F.make_tiles(x, iv)
    outs, _ = F.make_tiles(out, ov)
    assert run_ws(N, ins, outs, w, F.FFT_UpdateOutput, 1.0, Nb, n)
    assert rel(out.cpu().numpy(), oracle.corr2d_valid(x.cpu().numpy(), w.cpu().numpy())) < TOL_CONV
    assert bool(torch.isnan(obig[:, :, :, :3]).all())  # nothing written outside the views


@pytest.mark.parametrize("seed", range(12))
def test_random_tilings(oracle, seed):
    rng = np.random.default_rng(7000 + seed)
    N = int(rng.choice([8, 16, 32]))
    k = int(rng.integers(1, min(N - 1, 9) + 1))
    H, W = int(rng.integers(k, 3 * N)), int(rng.integers(k, 3 * N))
    Nb, Cin, Cout = int(rng.integers(1, 20)), int(rng.integers(1, 40)), int(rng.integers(1, 40))
    d = dev()
    x = synth.uniform((Nb, Cin, H, W), seed=seed, device=d)
    w = synth.normal((Cout, Cin, k, k), seed=seed + 1, std=0.05, device=d)
    out = torch.full((Nb, Cout, H - k + 1, W - k + 1), float("nan"), device=d)
    ins, outs, n = F.make_tile_grid(x, out, k, k, N)
    tag = (N, k, H, W, Nb, Cin, Cout, n)
    assert run_ws(N, ins, outs, w, F.FFT_UpdateOutput, 1.0, Nb, n), tag
    xh, wh = x.cpu().numpy(), w.cpu().numpy()
    assert rel(out.cpu().numpy(), oracle.corr2d_valid(xh, wh)) < TOL_CONV, tag
    g = synth.normal(tuple(out.shape), seed=seed + 2, device=d)
    gins, gouts, n2 = F.make_tile_grid(x, g, k, k, N)
    gw = torch.full_like(w, float("nan"))
    assert run_ws(N, gins, gouts, gw, F.FFT_AccGradParameters, 0.25, Nb, n2), tag
    assert rel(gw.cpu().numpy(), 0.25 * oracle.corr2d_grad_weight(xh, g.cpu().numpy(), k, k)) < TOL_CONV, tag
    gin = torch.full_like(x, float("nan"))
    bins, bouts, n3 = F.make_tile_grid(gin, g, k, k, N, F.FFT_UpdateGradInput)
    assert run_ws(N, bins, bouts, w, F.FFT_UpdateGradInput, 1.0, Nb, n3), tag
    assert rel(gin.cpu().numpy(), oracle.corr2d_grad_input(g.cpu().numpy(), wh, H, W)) < TOL_CONV, tag


def test_weight_gradient_is_reproducible_and_return_codes():
    N, k, H, W, Nb, Cin, Cout = 16, 5, 60, 52, 6, 5, 7
    d = dev()
    x = synth.uniform((Nb, Cin, H, W), seed=70, device=d)
    g = synth.normal((Nb, Cout, H - k + 1, W - k + 1), seed=71, device=d)
    ins, outs, n = F.make_tile_grid(x, g, k, k, N)
    runs = []
    for _ in range(3):
        gw = torch.full((Cout, Cin, k, k), float("nan"), device=d)
        assert run_ws(N, ins, outs, gw, F.FFT_AccGradParameters, 0.5, Nb, n)
        runs.append(gw.cpu().numpy())
    assert np.array_equal(runs[0], runs[1]) and np.array_equal(runs[0], runs[2])
    w = torch.zeros((Cout, Cin, k, k), device=d)
    ws = workspace(N, 0, Nb, n, Cin, Cout)
    L = F.lib()
    args = (ins.data_ptr(), outs.data_ptr(), F.view(w))
    assert L.fbfft_iterated_conv_ws(N, *args, 3, 1.0, Nb, n, ws.data_ptr(), ws.numel(), None) == 0
    assert L.fbfft_iterated_conv_ws(64, *args, 0, 1.0, Nb, n, ws.data_ptr(), ws.numel(), None) == 0
    assert L.fbfft_iterated_conv_ws(N, *args, 0, 1.0, Nb, n, ws.data_ptr(), 1024, None) == \
        -F.UnsupportedDimension
    assert L.fbfft_iterated_conv_ws(N, *args, 0, 1.0, Nb, n, None, 0, None) == -F.UnsupportedDimension
    assert L.fbfft_iterated_conv_ws(N, *args, 0, 1.0, 0, n, None, 0, None) == 1  # nothing to do
    assert F.iterated_conv_workspace(64, 0, Nb, n, Cin, Cout) == 0
    torch.cuda.synchronize()


def test_config4_forward_through_the_workspace(oracle):
    """configs[4] on FFTIteratedConvolution's own descriptors: 121 tiles of 32x32,
    fp64 direct correlation on 4096 seeded output pixels incl. tile seams."""
    d = dev()
    x = synth.uniform((16, 32, 256, 256), seed=40, device=d)
    w = synth.normal((32, 32, 9, 9), seed=41, std=0.05, device=d)
    out = torch.full((16, 32, 248, 248), float("nan"), device=d)
    ins, outs, n = F.make_tile_grid(x, out, 9, 9, 32)
    assert n == 121
    assert run_ws(32, ins, outs, w, F.FFT_UpdateOutput, 1.0, 16, n)
    assert bool(torch.isfinite(out).all())
    rng = np.random.default_rng(47)
    coords = np.stack([rng.integers(0, 16, 4096), rng.integers(0, 32, 4096),
                       rng.integers(0, 248, 4096), rng.integers(0, 248, 4096)], axis=1).astype(np.int32)
    coords[:8, 2:] = [[0, 0], [247, 247], [23, 24], [24, 23], [239, 240], [240, 239], [0, 247], [247, 0]]
    want = oracle.corr2d_valid_at(x.cpu().numpy(), w.cpu().numpy(), coords)
    oh = out.cpu().numpy()
    check("configs[4] fbfft_iterated_conv_ws updateOutput vs fp64 (4096 pixels)",
          oh[coords[:, 0], coords[:, 1], coords[:, 2], coords[:, 3]], want, TOL_CONV)
