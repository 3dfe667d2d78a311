"""GPU parity of FFTIteratedConvolution (C ABI fbfft_iterated_conv): the fused
tiled convolution, all three passes, against the CPU transcription on the same
tile descriptors and against fp64 direct correlation."""
import numpy as np
import pytest
import torch

import fbcuda_amd as F
from fbcuda_amd import synth
from gpu_util import check, TOL_CONV, dev, rel

pytestmark = pytest.mark.gpu


def tiles_for(H, W, k, N):
    """Overlapping N x N input windows with origin stride N-k+1 and the valid
    output window of each: the descriptors the reference's caller builds."""
    oH, oW, step = H - k + 1, W - k + 1, N - k + 1
    iv, ov = [], []
    for y0 in range(0, oH, step):
        for x0 in range(0, oW, step):
            iv.append((y0, x0, min(N, H - y0), min(N, W - x0), 0, 0))
            ov.append((y0, x0, min(step, oH - y0), min(step, oW - x0), 0, 0))
    return iv, ov


def run_pass(N, x, iv, out, ov, w, pass_, scale=1.0):
    d = dev()
    xd, od, wd = torch.from_numpy(x).to(d), torch.from_numpy(out).to(d), torch.from_numpy(w).to(d)
    ins, n1 = F.make_tiles(xd, iv)
    outs, n2 = F.make_tiles(od, ov)
    assert n1 == n2
    launched = F.FFTIteratedConvolution(N, ins, outs, wd, pass_, scale, x.shape[0], n1)
    torch.cuda.synchronize()
    return launched, xd.cpu().numpy(), od.cpu().numpy(), wd.cpu().numpy()


@pytest.mark.parametrize("N,k,H,W,Nb,Cin,Cout", [
    (8, 3, 14, 17, 3, 5, 7),       # ragged planes: partial A / W groups
    (16, 5, 30, 25, 2, 3, 4),
    (32, 9, 40, 56, 2, 3, 4),
    (32, 5, 32, 32, 5, 9, 10),     # one tile, more planes than one workgroup covers
    (8, 1, 9, 9, 17, 2, 33),
])
def test_three_passes_vs_oracle(oracle, N, k, H, W, Nb, Cin, Cout):
    x = synth.uniform((Nb, Cin, H, W), seed=40).numpy()
    w = synth.normal((Cout, Cin, k, k), seed=41, std=0.05).numpy()
    iv, ov = tiles_for(H, W, k, N)
    oshape = (Nb, Cout, H - k + 1, W - k + 1)

    # updateOutput
    launched, _, got, _ = run_pass(N, x, iv, np.full(oshape, np.nan, np.float32), ov, w, F.FFT_UpdateOutput)
    assert launched
    want = np.zeros(oshape, np.float32)
    assert oracle.iterated_conv(N, x.copy(), iv, want, ov, w, 0) == 1
    assert rel(got, want) < TOL_CONV
    assert rel(got, oracle.corr2d_valid(x, w)) < TOL_CONV

    # accGradParameters (overwrites weight with scale * gradient)
    g = synth.normal(oshape, seed=42).numpy()
    launched, _, _, gw = run_pass(N, x, iv, g, ov, np.full_like(w, np.nan), F.FFT_AccGradParameters, 0.5)
    assert launched
    gw_want = np.zeros_like(w)
    assert oracle.iterated_conv(N, x.copy(), iv, g.copy(), ov, gw_want, 2, 0.5) == 1
    assert rel(gw, gw_want) < TOL_CONV
    assert rel(gw, 0.5 * oracle.corr2d_grad_weight(x, g, k, k)) < TOL_CONV

    # updateGradInput stores (does not accumulate) each tile's result, as the reference
    # does, so it runs on its own grid: disjoint gradInput windows with pads kH-1 / kW-1,
    # each fed by the N x N gradOutput window around it (fbfft_make_tiles_for_pass)
    d = dev()
    gin_d = torch.full(x.shape, 7.0, device=d)
    g_d, w_d = torch.from_numpy(g).to(d), torch.from_numpy(w).to(d)
    bins, bouts, nb = F.make_tile_grid(gin_d, g_d, k, k, N, F.FFT_UpdateGradInput)
    assert nb == -(-H // (N - k + 1)) * -(-W // (N - k + 1))
    assert F.FFTIteratedConvolution(N, bins, bouts, w_d, F.FFT_UpdateGradInput, 1.0, Nb, nb)
    torch.cuda.synchronize()
    assert rel(gin_d.cpu().numpy(), oracle.corr2d_grad_input(g, w, H, W)) < TOL_CONV
    # the overlapping grid of the other passes is only defined for a single tile
    if len(iv) == 1:
        gin0 = np.full_like(x, 7.0)
        launched, gin, _, _ = run_pass(N, gin0, iv, g, ov, w, F.FFT_UpdateGradInput)
        assert launched
        gin_want = gin0.copy()
        assert oracle.iterated_conv(N, gin_want, iv, g.copy(), ov, w, 1) == 1
        assert rel(gin, gin_want) < TOL_CONV
        assert rel(gin, oracle.corr2d_grad_input(g, w, H, W)) < TOL_CONV


@pytest.mark.parametrize("N", [8, 16, 32])
def test_grad_input_single_tiles(oracle, N):
    """Non-overlapping tiles so that the write order between tiles cannot matter."""
    k, Nb, Cin, Cout = 3, 3, 4, 5
    H = W = 2 * N
    x0 = np.zeros((Nb, Cin, H, W), np.float32)
    o = N - k + 1
    g = np.zeros((Nb, Cout, 2 * o, 2 * o), np.float32)
    g[:] = synth.normal(g.shape, seed=43).numpy()
    w = synth.normal((Cout, Cin, k, k), seed=44, std=0.05).numpy()
    iv = [(y, x, N, N, 0, 0) for y in (0, N) for x in (0, N)]
    ov = [(y, x, o, o, 0, 0) for y in (0, o) for x in (0, o)]
    launched, gin, _, _ = run_pass(N, x0, iv, g, ov, w, F.FFT_UpdateGradInput)
    assert launched
    want = x0.copy()
    assert oracle.iterated_conv(N, want, iv, g.copy(), ov, w, 1) == 1
    assert rel(gin, want) < TOL_CONV


def test_padded_descriptors(oracle):
    """padL / padU inside the descriptors shift the data within the FFT plane."""
    N, k, Nb, Cin, Cout = 16, 3, 2, 2, 3
    x = synth.uniform((Nb, Cin, 10, 11), seed=45).numpy()
    w = synth.normal((Cout, Cin, k, k), seed=46, std=0.05).numpy()
    iv = [(0, 0, 10, 11, 2, 3)]
    ov = [(0, 0, 8, 9, 2, 3)]
    out0 = np.full((Nb, Cout, 8, 9), np.nan, np.float32)
    launched, _, got, _ = run_pass(N, x, iv, out0, ov, w, F.FFT_UpdateOutput)
    want = np.zeros_like(out0)
    assert launched and oracle.iterated_conv(N, x.copy(), iv, want, ov, w, 0) == 1
    assert rel(got, want) < TOL_CONV
    assert rel(got, oracle.corr2d_valid(x, w)) < TOL_CONV


def test_return_codes():
    d = dev()
    x = torch.zeros((1, 1, 8, 8), device=d)
    o = torch.zeros((1, 1, 6, 6), device=d)
    w = torch.zeros((1, 1, 3, 3), device=d)
    ins, n = F.make_tiles(x, [(0, 0, 8, 8, 0, 0)])
    outs, _ = F.make_tiles(o, [(0, 0, 6, 6, 0, 0)])
    assert F.FFTIteratedConvolution(8, ins, outs, w, 0, 1.0, 1, n) is True
    assert F.FFTIteratedConvolution(8, ins, outs, w, 3, 1.0, 1, n) is False    # unknown pass
    assert F.FFTIteratedConvolution(64, ins, outs, w, 0, 1.0, 1, n) is False   # unsupported size
    torch.cuda.synchronize()


def test_config4_forward(oracle):
    """configs[4]: 16x32x256x256 * 32x32x9x9 in 121 tiles of 32x32 -> 16x32x248x248;
    fp64 direct correlation on 4096 seeded output pixels."""
    d = dev()
    x = synth.uniform((16, 32, 256, 256), seed=40, device=d)
    w = synth.normal((32, 32, 9, 9), seed=41, std=0.05, device=d)
    out = torch.full((16, 32, 248, 248), float("nan"), device=d)
    iv, ov = tiles_for(256, 256, 9, 32)
    assert len(iv) == 121 and iv[-1][2:4] == (16, 16) and ov[-1][2:4] == (8, 8)
    ins, n = F.make_tiles(x, iv)
    outs, _ = F.make_tiles(out, ov)
    assert F.FFTIteratedConvolution(32, ins, outs, w, F.FFT_UpdateOutput, 1.0, 16, n)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(out).all())
    rng = np.random.default_rng(47)
    coords = np.stack([rng.integers(0, 16, 4096), rng.integers(0, 32, 4096),
                       rng.integers(0, 248, 4096), rng.integers(0, 248, 4096)], axis=1).astype(np.int32)
    coords[:8, 2:] = [[0, 0], [247, 247], [23, 24], [24, 23], [239, 240], [240, 239], [0, 247], [247, 0]]
    want = oracle.corr2d_valid_at(x.cpu().numpy(), w.cpu().numpy(), coords)
    oh = out.cpu().numpy()
    got = oh[coords[:, 0], coords[:, 1], coords[:, 2], coords[:, 3]]
    check("configs[4] FFTIteratedConvolution updateOutput vs fp64 (4096 pixels)", got, want, TOL_CONV)


def test_library_tile_grid_matches_reference_tiling(oracle):
    """fbfft_make_tiles builds the descriptors that tiles_for spells out; the
    forward pass over them equals fp64 direct correlation."""
    N, k, H, W, Nb, Cin, Cout = 16, 5, 37, 30, 2, 3, 4
    d = dev()
    x = synth.uniform((Nb, Cin, H, W), seed=40, device=d)
    w = synth.normal((Cout, Cin, k, k), seed=41, std=0.05, device=d)
    out = torch.full((Nb, Cout, H - k + 1, W - k + 1), float("nan"), device=d)
    ins, outs, n = F.make_tile_grid(x, out, k, k, N)
    iv, ov = tiles_for(H, W, k, N)
    ins2, n2 = F.make_tiles(x, iv)
    outs2, _ = F.make_tiles(out, ov)
    assert n == n2 and bool((ins == ins2).all()) and bool((outs == outs2).all())
    assert F.FFTIteratedConvolution(N, ins, outs, w, F.FFT_UpdateOutput, 1.0, Nb, n)
    torch.cuda.synchronize()
    assert rel(out.cpu().numpy(), oracle.corr2d_valid(x.cpu().numpy(), w.cpu().numpy())) < TOL_CONV


@pytest.mark.parametrize("seed", range(16))
def test_random_tilings(oracle, seed):
    """All three passes on a seeded random image / filter / plane count with the
    library's own tile grids, against fp64 direct correlation and its gradients."""
    rng = np.random.default_rng(5000 + seed)
    N = int(rng.choice([8, 16, 32]))
    k = int(rng.integers(1, min(N - 1, 9) + 1))
    H, W = int(rng.integers(k, 3 * N)), int(rng.integers(k, 3 * N))
    Nb, Cin, Cout = int(rng.integers(1, 20)), int(rng.integers(1, 12)), int(rng.integers(1, 20))
    d = dev()
    x = synth.uniform((Nb, Cin, H, W), seed=seed, device=d)
    w = synth.normal((Cout, Cin, k, k), seed=seed + 1, std=0.05, device=d)
    out = torch.full((Nb, Cout, H - k + 1, W - k + 1), float("nan"), device=d)
    ins, outs, n = F.make_tile_grid(x, out, k, k, N)
    tag = (N, k, H, W, Nb, Cin, Cout, n)
    assert F.FFTIteratedConvolution(N, ins, outs, w, F.FFT_UpdateOutput, 1.0, Nb, n), tag
    torch.cuda.synchronize()
    xh, wh = x.cpu().numpy(), w.cpu().numpy()
    assert rel(out.cpu().numpy(), oracle.corr2d_valid(xh, wh)) < TOL_CONV, tag
    g = synth.normal(tuple(out.shape), seed=seed + 2, device=d)
    gins, gouts, n2 = F.make_tile_grid(x, g, k, k, N)
    gw = torch.full_like(w, float("nan"))
    assert F.FFTIteratedConvolution(N, gins, gouts, gw, F.FFT_AccGradParameters, 0.25, Nb, n2), tag
    torch.cuda.synchronize()
    assert rel(gw.cpu().numpy(), 0.25 * oracle.corr2d_grad_weight(xh, g.cpu().numpy(), k, k)) < TOL_CONV, tag
    gin = torch.full_like(x, float("nan"))
    bins, bouts, n3 = F.make_tile_grid(gin, g, k, k, N, F.FFT_UpdateGradInput)
    assert F.FFTIteratedConvolution(N, bins, bouts, w, F.FFT_UpdateGradInput, 1.0, Nb, n3), tag
    torch.cuda.synchronize()
    assert rel(gin.cpu().numpy(), oracle.corr2d_grad_input(g.cpu().numpy(), wh, H, W)) < TOL_CONV, tag


def test_deterministic_weight_gradient_is_reproducible(oracle):
    """FBFFT_DETERMINISTIC: accGradParameters in the reference's fixed order gives the same
    bits on every run (the default schedule adds range partials atomically, in any order)
    and the same values as the fp64 gradient."""
    N, k, H, W, Nb, Cin, Cout = 16, 5, 60, 52, 6, 5, 7
    d = dev()
    x = synth.uniform((Nb, Cin, H, W), seed=70, device=d)
    g = synth.normal((Nb, Cout, H - k + 1, W - k + 1), seed=71, device=d)
    ins, outs, n = F.make_tile_grid(x, g, k, k, N)
    runs = []
    for _ in range(3):
        gw = torch.full((Cout, Cin, k, k), float("nan"), device=d)
        assert F.FFTIteratedConvolution(N, ins, outs, gw, F.FFT_AccGradParameters, 0.5, Nb, n,
                                        deterministic=True)
        torch.cuda.synchronize()
        runs.append(gw.cpu().numpy())
    assert np.array_equal(runs[0], runs[1]) and np.array_equal(runs[0], runs[2])
    want = 0.5 * oracle.corr2d_grad_weight(x.cpu().numpy(), g.cpu().numpy(), k, k)
    assert rel(runs[0], want) < TOL_CONV
    # the default schedule agrees to rounding
    gw = torch.full((Cout, Cin, k, k), float("nan"), device=d)
    assert F.FFTIteratedConvolution(N, ins, outs, gw, F.FFT_AccGradParameters, 0.5, Nb, n)
    torch.cuda.synchronize()
    assert rel(gw.cpu().numpy(), runs[0]) < TOL_CONV
    # unknown flag bits: not launched
    rc = F.lib().fbfft_iterated_conv_ex(N, ins.data_ptr(), outs.data_ptr(), F.view(gw), 2, 0.5, Nb, n, 6,
                                        None)
    assert rc == 0


def test_layer_weight_gradient_is_reproducible():
    """fbfft_conv_accgrad on a tiled image: a fixed reduction order inside the contraction,
    no atomics - the same bits on every run."""
    N, k, H, W, Nb, Cin, Cout = 32, 5, 80, 71, 4, 6, 5
    d = dev()
    x = synth.uniform((Nb, Cin, H, W), seed=72, device=d)
    g = synth.normal((Nb, Cout, H - k + 1, W - k + 1), seed=73, device=d)
    ws = torch.empty(F.conv_workspace_image(2, Nb, Cin, Cout, H, W, k, k, N), dtype=torch.uint8, device=d)
    runs = []
    for _ in range(3):
        gw = torch.full((Cout, Cin, k, k), float("nan"), device=d)
        assert F.conv_accgrad(x, g, gw, N, ws) == F.Success
        torch.cuda.synchronize()
        runs.append(gw.cpu().numpy())
    assert np.array_equal(runs[0], runs[1]) and np.array_equal(runs[0], runs[2])
