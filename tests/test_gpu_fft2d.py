"""GPU parity of fbfft2D / fbifft2D (C ABI fbfft_r2c_2d / fbfft_c2r_2d) against
the CPU oracle: fp32 transcription, fp64 DFT, golden fixtures, edge cases and
size-independent properties at the benchmark's full size."""
import os

import numpy as np
import pytest
import torch

import fbcuda_amd as F
from fbcuda_amd import synth
from gpu_util import TOL_FFT, c, check, dev, fft2d, ifft2d, rel

pytestmark = pytest.mark.gpu
GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "fft_vectors.npz"))
SIZES = [8, 16, 32, 64, 128]


@pytest.mark.parametrize("key", [k[4:] for k in GOLD.files if k.startswith("x2d_")])
def test_golden(key):
    N, h, w, padL, padU = map(int, key.split("_"))
    rc, out = fft2d(GOLD["x2d_" + key], N, padL, padU)
    assert rc == F.Success
    assert rel(c(out), GOLD["f2d_" + key]) < TOL_FFT


@pytest.mark.parametrize("N", SIZES)
@pytest.mark.parametrize("case", ["full", "ragged", "padded", "tiny"])
@pytest.mark.parametrize("B", [1, 5, 67])
def test_forward_inverse_vs_oracle(oracle, N, case, B):
    h, w, padL, padU = {"full": (N, N, 0, 0), "ragged": (N - 5, N - 3, 0, 0),
                        "padded": (N - 5, N - 4, 2, 3), "tiny": (5, 5, 0, 0)}[case]
    x = synth.normal((B, h, w), seed=N + B).numpy()
    rc, got = fft2d(x, N, padL, padU)
    assert rc == F.Success
    _, want32 = oracle.fbfft2d(x, N, padL, padU)
    want64 = oracle.dft2d_r2c(x, N, padL, padU)
    assert rel(got, want32) < TOL_FFT
    assert rel(got, want64) < TOL_FFT
    # inverse of the oracle's spectrum, cropped on store; cells outside stay untouched
    rc, back = ifft2d(want32, h, w, padL, padU)
    assert rc == F.Success
    _, back32 = oracle.fbifft2d(want32, h, w, padL, padU)
    assert rel(back, back32) < TOL_FFT
    assert rel(back, N * N * x.astype(np.float64)) < TOL_FFT


@pytest.mark.parametrize("N", SIZES)
def test_inverse_writes_only_the_window(oracle, N):
    """crop-on-store: a real tensor smaller than N x N receives exactly its window."""
    x = synth.normal((3, N, N), seed=77).numpy()
    _, spec = oracle.fbfft2d(x, N)
    h, w, padL, padU = N - 9 if N > 9 else 3, N - 5, 1, 2
    rc, got = ifft2d(spec, h, w, padL, padU)
    assert rc == F.Success
    want = N * N * x[:, padU:padU + h, padL:padL + w].astype(np.float64)
    assert rel(got, want) < TOL_FFT


@pytest.mark.parametrize("N", [8, 16, 32])
def test_inverse_lane0_quirk(oracle, N):
    """Imaginary parts of F[0][0] and F[N/2][0] are ignored (fbfft/FFT2D32.cuh:313-315)."""
    x = synth.normal((2, N, N), seed=5).numpy()
    _, spec = oracle.fbfft2d(x, N)
    spec[:, 0, 0, 1] = 3.0
    spec[:, N // 2, 0, 1] = -4.0
    _, got = ifft2d(spec, N, N)
    _, want = oracle.fbifft2d(spec, N, N)
    assert rel(got, want) < TOL_FFT
    assert rel(got, N * N * x.astype(np.float64)) < TOL_FFT


@pytest.mark.parametrize("N", SIZES)
def test_strided_operands(oracle, N):
    """Non-contiguous views: padded batch / row strides on both operands."""
    B = 6
    x = synth.normal((B, N, N), seed=9).numpy()
    big = torch.zeros((B, N + 3, N + 4), device=dev())
    real = big[:, 1:N + 1, 2:N + 2]
    real.copy_(torch.from_numpy(x))
    wide = torch.full((B, N // 2 + 2, N + 2, 2), float("nan"), device=dev())
    spec = wide[:, :N // 2 + 1, 1:N + 1, :]
    assert F.fbfft2D(real, spec) == F.Success
    torch.cuda.synchronize()
    _, want = oracle.fbfft2d(x, N)
    assert rel(spec.cpu().numpy(), want) < TOL_FFT
    back = torch.zeros_like(big)
    assert F.fbifft2D(spec, back[:, 1:N + 1, 2:N + 2]) == F.Success
    torch.cuda.synchronize()
    assert rel(back[:, 1:N + 1, 2:N + 2].cpu().numpy(), N * N * x.astype(np.float64)) < TOL_FFT
    assert float(back[:, 0].abs().max()) == 0.0  # nothing outside the view was written


def test_error_codes():
    d = dev()
    real = torch.zeros((4, 32, 32), device=d)
    assert F.fbfft2D(real, torch.zeros((4, 17, 32, 2), device=d)) == F.Success
    assert F.fbfft2D(real, torch.zeros((4, 129, 256, 2), device=d)) == F.UnsupportedSize
    assert F.fbfft2D(real, torch.zeros((4, 7, 12, 2), device=d)) == F.UnsupportedSize
    assert F.fbfft2D(real, torch.zeros((4, 15, 32, 2), device=d)) == F.UnsupportedSize
    assert F.fbfft2D(real, torch.zeros((4, 16, 32, 2), device=d)) == F.Success  # packed rows
    assert F.fbfft2D(torch.zeros((4, 64, 64), device=d),
                     torch.zeros((4, 32, 64, 2), device=d)) == F.UnsupportedSize  # N <= 32 only
    assert F.fbfft2D(real, torch.zeros((3, 17, 32, 2), device=d)) == F.UnsupportedDimension
    assert F.fbfft2D(real, torch.zeros((4, 17, 32), device=d)) == F.UnsupportedDimension
    assert F.fbfft2D(torch.zeros((4, 40, 32), device=d),
                     torch.zeros((4, 17, 32, 2), device=d)) == F.UnsupportedSize
    assert F.fbifft2D(torch.zeros((4, 129, 256, 2), device=d), real) == F.UnsupportedSize
    # empty batch is a successful no-op
    assert F.fbfft2D(torch.zeros((0, 32, 32), device=d), torch.zeros((0, 17, 32, 2), device=d)) == F.Success
    torch.cuda.synchronize()


def per_plane_rel(got, want):
    """Largest rel-L2 of any single plane (a whole-tensor norm could hide one bad plane)."""
    B = got.shape[0]
    a = np.asarray(got, np.float64).reshape(B, -1)
    b = np.asarray(want, np.float64).reshape(B, -1)
    return float((np.linalg.norm(a - b, axis=1) / np.maximum(np.linalg.norm(b, axis=1), 1e-300)).max())


@pytest.mark.parametrize("N,B", [(32, 16384), (8, 1 << 20), (16, 1 << 18), (64, 16384), (128, 4096)])
def test_full_size_properties(oracle, N, B):
    """Benchmark sizes: round trip ifft(fft(x)) = N^2 x on the whole tensor, linearity, and
    parity with the CPU transcription plane by plane - on every one of configs[1]'s 16384
    planes, on 256 seeded planes (first and last included) of each configs[2] size - for
    the forward transform and, on the transcription's own spectra, for the inverse."""
    d = dev()
    seed = {32: 1, 8: 5, 16: 6, 64: 8, 128: 9}[N]
    x = synth.normal((B, N, N), seed=seed, device=d)
    spec = torch.empty((B, N // 2 + 1, N, 2), device=d)
    assert F.fbfft2D(x, spec) == F.Success
    back = torch.empty_like(x)
    assert F.fbifft2D(spec, back) == F.Success
    torch.cuda.synchronize()
    err = (back / (N * N) - x).double().norm() / x.double().norm()
    print("parity round trip %dx%d over all %d planes: %.2e" % (N, N, B, float(err)))
    assert float(err) < TOL_FFT
    if N == 32:
        pick = np.arange(B)
    else:
        pick = np.unique(np.concatenate([[0, 1, B - 2, B - 1],
                                         np.random.default_rng(seed).choice(B, 252, replace=False)]))
    xp = x.cpu().numpy()[pick]
    rc, want = oracle.fbfft2d(xp, N)
    assert rc == 0
    got = spec.cpu().numpy()[pick]
    tag = "%dx%d, %d of %d planes" % (N, N, len(pick), B)
    check("fbfft2D vs transcription (%s)" % tag, got, want, TOL_FFT)
    check("fbfft2D vs fp64 DFT (first 64 of them)", got[:64], oracle.dft2d_r2c(xp[:64], N), TOL_FFT)
    worst = per_plane_rel(got, want)
    print("parity fbfft2D worst single plane (%s): %.2e" % (tag, worst))
    assert worst < TOL_FFT
    # inverse: the same spectra (the transcription's) into both implementations
    rc, want_back = oracle.fbifft2d(want, N, N)
    assert rc == 0
    sd = torch.from_numpy(want).to(d)
    bd = torch.full((len(pick), N, N), float("nan"), device=d)
    assert F.fbifft2D(sd, bd) == F.Success
    torch.cuda.synchronize()
    check("fbifft2D vs transcription, same spectra (%s)" % tag, bd.cpu().numpy(), want_back, TOL_FFT)
    assert per_plane_rel(bd.cpu().numpy(), want_back) < TOL_FFT
    del sd, bd
    # linearity on a slice: F(2x + y) = 2F(x) + F(y)
    n = min(B // 2, 4096)
    z = (2 * x[:n] + x[n:2 * n]).contiguous()
    sz = torch.empty((n, N // 2 + 1, N, 2), device=d)
    assert F.fbfft2D(z, sz) == F.Success
    torch.cuda.synchronize()
    lin = (sz - (2 * spec[:n] + spec[n:2 * n])).double().norm() / sz.double().norm()
    assert float(lin) < TOL_FFT


@pytest.mark.parametrize("N,B", [(32, 9001), (16, 33333), (8, 110001)])
def test_two_groups_per_wave_tail(oracle, N, B):
    """Batch sizes in the one-to-two-round regime, where a wave transforms two groups
    of planes and prefetches the second: odd group counts and a ragged last group."""
    d = dev()
    x = synth.normal((B, N, N), seed=12, device=d)
    spec = torch.full((B, N // 2 + 1, N, 2), float("nan"), device=d)
    back = torch.full((B, N, N), float("nan"), device=d)
    assert F.fbfft2D(x, spec) == F.Success
    assert F.fbifft2D(spec, back) == F.Success
    torch.cuda.synchronize()
    assert bool(torch.isfinite(spec).all()) and bool(torch.isfinite(back).all())
    err = (back / (N * N) - x).double().norm() / x.double().norm()
    assert float(err) < TOL_FFT
    pick = [0, 1, B // 2, B - 130, B - 5, B - 4, B - 3, B - 2, B - 1]
    _, want = oracle.fbfft2d(x[pick].cpu().numpy(), N)
    assert rel(spec[pick].cpu().numpy(), want) < TOL_FFT


@pytest.mark.parametrize("N", [2, 4])
@pytest.mark.parametrize("B", [1, 2, 5, 1000])
def test_warp_kernel_sizes(oracle, N, B):
    """N = 2 and 4 (the reference's plane-pairing warp kernel, fbfft/FBFFT2D-inl.cuh:611-612):
    transposed [kx half][ky] layout, odd batches, windows and padding."""
    for h, w, padL, padU in [(N, N, 0, 0), (N - 1, N, 0, 0), (N - 1, N - 1, 1, 1)]:
        x = synth.normal((B, h, w), seed=100 + N + B).numpy()
        rc, got = fft2d(x, N, padL, padU)
        assert rc == F.Success
        _, want32 = oracle.fbfft2d(x, N, padL, padU)
        assert rel(got, want32) < TOL_FFT
        assert rel(got, oracle.dft2d_r2c(x, N, padL, padU)) < TOL_FFT
        rc, back = ifft2d(want32, h, w, padL, padU)
        assert rc == F.Success
        _, back32 = oracle.fbifft2d(want32, h, w, padL, padU)
        assert rel(back, back32) < TOL_FFT
        assert rel(back, N * N * x.astype(np.float64)) < TOL_FFT
    # strided views on both sides
    x = synth.normal((B, N, N), seed=7).numpy()
    big = torch.zeros((B, N + 1, N + 3), device=dev())
    real = big[:, 1:, 2:N + 2]
    real.copy_(torch.from_numpy(x))
    wide = torch.full((B, N // 2 + 2, N + 1, 2), float("nan"), device=dev())
    spec = wide[:, 1:, :N, :]
    assert F.fbfft2D(real, spec) == F.Success
    torch.cuda.synchronize()
    assert rel(spec.cpu().numpy(), oracle.dft2d_r2c(x, N)) < TOL_FFT
    assert bool(torch.isnan(wide[:, 0]).all()) and bool(torch.isnan(wide[:, :, N]).all())


@pytest.mark.parametrize("seed", range(40))
def test_random_windows_and_views(oracle, seed):
    """Seeded random draw over size, batch, window, padding (also windows that
    hang over the right / bottom edge, which MemoryAccess.cuh:19-25 clips), and
    views that are transposed or padded in memory."""
    rng = np.random.default_rng(1000 + seed)
    N = int(rng.choice([2, 4, 8, 16, 32, 64, 128]))
    B = int(rng.integers(1, 20))
    h, w = int(rng.integers(1, N + 1)), int(rng.integers(1, N + 1))
    padL, padU = (int(rng.integers(0, N // 2 + 1)), int(rng.integers(0, N // 2 + 1))) \
        if rng.random() < 0.6 else (0, 0)
    x = synth.normal((B, h, w), seed=seed).numpy()
    d = dev()
    kind = int(rng.integers(0, 3))
    if kind == 0:                                   # contiguous
        real = torch.from_numpy(x).to(d)
    elif kind == 1:                                 # padded rows and batch stride
        big = torch.zeros((B, h + 2, w + 3), device=d)
        real = big[:, 1:h + 1, 2:w + 2]
        real.copy_(torch.from_numpy(x))
    else:                                           # x and y swapped in memory
        real = torch.from_numpy(np.ascontiguousarray(x.transpose(0, 2, 1))).to(d).transpose(1, 2)
    if rng.random() < 0.5:
        spec = torch.full((B, N // 2 + 1, N, 2), float("nan"), device=d)
    else:
        wide = torch.full((B + 1, N // 2 + 2, N + 1, 2), float("nan"), device=d)
        spec = wide[1:, 1:, :N, :]
    assert F.fbfft2D(real, spec, padL, padU) == F.Success
    torch.cuda.synchronize()
    _, want32 = oracle.fbfft2d(x, N, padL, padU)
    got = spec.cpu().numpy()
    assert rel(got, want32) < TOL_FFT, (N, B, h, w, padL, padU, kind)
    assert rel(got, oracle.dft2d_r2c(x, N, padL, padU)) < TOL_FFT
    # and back into a view of the same geometry
    # (cells of the window that hang over the edge keep what they held)
    back = torch.full_like(real, 7.0)
    assert F.fbifft2D(spec, back, padL, padU) == F.Success
    torch.cuda.synchronize()
    _, back32 = oracle.fbifft2d(want32, h, w, padL, padU, out=np.full((B, h, w), 7.0, np.float32))
    assert rel(back.cpu().numpy(), back32) < TOL_FFT, (N, B, h, w, padL, padU, kind)


@pytest.mark.parametrize("N,h,w,padL,padU", [
    (64, 60, 60, 0, 0), (64, 60, 60, 4, 3), (64, 17, 8, 8, 40), (64, 64, 64, 4, 1),
    (128, 124, 124, 0, 0), (128, 124, 120, 4, 2), (128, 31, 64, 60, 100), (128, 5, 4, 124, 0)])
def test_windows_that_move_as_16_byte_words(oracle, N, h, w, padL, padU):
    """Windows whose rows start on 16-byte boundaries with width and left edge
    multiples of 4 take the float4 loader of the 64 / 128 kernels (also hanging
    over the right edge)."""
    B = 5
    x = synth.normal((B, h, w), seed=N + h).numpy()
    rc, got = fft2d(x, N, padL, padU)
    assert rc == F.Success
    _, want32 = oracle.fbfft2d(x, N, padL, padU)
    assert rel(got, want32) < TOL_FFT
    assert rel(got, oracle.dft2d_r2c(x, N, padL, padU)) < TOL_FFT


@pytest.mark.parametrize("N", [8, 16, 32])
def test_odd_plane_stride_mixes_the_window_load_paths(oracle, N):
    """Even window, even row stride, odd plane stride: every other plane starts on an
    8-byte boundary, so the planes of one wave take different load paths."""
    B, h, w = 11, N // 2, N // 2 - 2
    x = synth.normal((B, h, w), seed=5 * N).numpy()
    flat = torch.zeros(B * (h * w + 1) + 8, device=dev())
    real = flat.as_strided((B, h, w), (h * w + 1, w, 1))
    real.copy_(torch.from_numpy(x))
    spec = torch.full((B, N // 2 + 1, N, 2), float("nan"), device=dev())
    assert F.fbfft2D(real, spec, 2, 1) == F.Success
    torch.cuda.synchronize()
    _, want = oracle.fbfft2d(x, N, 2, 1)
    assert rel(spec.cpu().numpy(), want) < TOL_FFT
    back = torch.zeros_like(flat).as_strided((B, h, w), (h * w + 1, w, 1))
    assert F.fbifft2D(spec, back, 2, 1) == F.Success
    torch.cuda.synchronize()
    assert rel(back.cpu().numpy(), N * N * x.astype(np.float64)) < TOL_FFT


@pytest.mark.parametrize("N", [4, 8, 32, 64])
@pytest.mark.parametrize("h,w", [(0, 3), (3, 0)])
def test_empty_window_gives_zero_spectra(N, h, w):
    """B > 0 planes whose real window is empty are all padding: zeros, not stale data."""
    x = torch.zeros((3, h, w), device=dev())
    out = torch.full((3, N // 2 + 1, N, 2), float("nan"), device=dev())
    assert F.fbfft2D(x, out) == F.Success
    torch.cuda.synchronize()
    assert float(out.abs().max()) == 0.0


@pytest.mark.parametrize("N,B", [(32, 8195), (32, 12289), (32, 14336), (32, 14339), (16, 30727),
                                 (16, 53760), (16, 53767), (8, 98317), (8, 172032), (8, 172049)])
def test_batches_either_side_of_the_two_groups_per_wave_switch(oracle, N, B):
    """Batches just above one round of resident waves, at 1.75 rounds (the last that pair)
    and just beyond (one group per wave again), odd tails included: every plane of the
    forward transform against the transcription, and the inverse on its spectra."""
    d = dev()
    x = synth.normal((B, N, N), seed=70 + N, device=d)
    spec = torch.full((B, N // 2 + 1, N, 2), float("nan"), device=d)
    assert F.fbfft2D(x, spec) == F.Success
    back = torch.full_like(x, float("nan"))
    assert F.fbifft2D(spec, back) == F.Success
    torch.cuda.synchronize()
    rc, want = oracle.fbfft2d(x.cpu().numpy(), N)
    assert rc == 0
    got = spec.cpu().numpy()
    assert np.isfinite(got).all()
    assert per_plane_rel(got, want) < TOL_FFT
    err = (back / (N * N) - x).double().norm() / x.double().norm()
    assert bool(torch.isfinite(back).all()) and float(err) < TOL_FFT
