"""GPU parity of fbfft1D / fbifft1D (C ABI fbfft_r2c_1d / fbfft_c2r_1d)."""
import os

import numpy as np
import pytest
import torch

import fbcuda_amd as F
from fbcuda_amd import synth
from gpu_util import check, TOL_FFT, c, dev, rel

pytestmark = pytest.mark.gpu
GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "fft_vectors.npz"))
SIZES = [2, 4, 8, 16, 32, 64, 128, 256]


def fft1d(x, padL=0):
    xd = torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to(dev())
    B, N = x.shape
    out = torch.full((B, N // 2 + 1, 2), float("nan"), device=dev())
    rc = F.fbfft1D(xd, out, padL)
    torch.cuda.synchronize()
    return rc, out.cpu().numpy()


def ifft1d(spec, padL=0, fill=float("nan")):
    sd = torch.from_numpy(np.ascontiguousarray(spec, dtype=np.float32)).to(dev())
    B, nc, _ = spec.shape
    out = torch.full((B, 2 * (nc - 1)), fill, device=dev())
    rc = F.fbifft1D(out, sd, padL)
    torch.cuda.synchronize()
    return rc, out.cpu().numpy()


@pytest.mark.parametrize("N", [8, 32, 256])
def test_golden(N):
    rc, out = fft1d(GOLD["x1d_%d" % N])
    assert rc == F.Success
    assert rel(c(out), GOLD["f1d_%d" % N]) < TOL_FFT


@pytest.mark.parametrize("N", SIZES)
@pytest.mark.parametrize("B", [1, 2, 7, 300, 1025])
def test_vs_oracle(oracle, N, B):
    x = synth.uniform((B, N), seed=N + B).numpy()
    rc, got = fft1d(x)
    assert rc == F.Success
    _, want32 = oracle.fbfft1d(x)
    assert rel(got, want32) < TOL_FFT
    assert rel(got, oracle.dft1d_r2c(x)) < TOL_FFT
    rc, back = ifft1d(want32)
    assert rc == F.Success
    _, back32 = oracle.fbifft1d(want32)
    assert rel(back, back32) < TOL_FFT
    assert rel(back, N * x.astype(np.float64)) < TOL_FFT


def test_config0_full(oracle):
    """configs[0]: 4096 rows of 32 points, U[-1,1], seed 0, whole tensor."""
    x = synth.uniform((4096, 32), seed=0).numpy()
    rc, got = fft1d(x)
    assert rc == F.Success and got.shape == (4096, 17, 2)
    _, want = oracle.fbfft1d(x)
    check("configs[0] fbfft1D vs transcription (4096 rows)", got, want, TOL_FFT)
    check("configs[0] fbfft1D vs fp64 DFT", got, oracle.dft1d_r2c(x), TOL_FFT)
    rc, back = ifft1d(got)
    check("configs[0] round trip", back, 32 * x.astype(np.float64), TOL_FFT)


@pytest.mark.parametrize("N", [4, 16, 32, 128])
def test_padl_quirk(oracle, N):
    """padL shifts right and drops the tail on load; the inverse writes the first
    row of each pair un-shifted and the second shifted (fbfft/FBFFTCommon.cuh:325, :425-427)."""
    padL, B = 3 if N > 4 else 1, 5
    x = synth.uniform((B, N), seed=11).numpy()
    rc, got = fft1d(x, padL)
    _, want = oracle.fbfft1d(x, padL)
    assert rc == F.Success and rel(got, want) < TOL_FFT
    rc, back = ifft1d(want, padL, fill=777.0)
    _, back32 = oracle.fbifft1d(want, padL, out=np.full((B, N), 777.0, np.float32))
    assert rc == F.Success
    assert np.array_equal(back == 777.0, back32 == 777.0)
    assert rel(back, back32) < TOL_FFT


def test_strided_and_errors(oracle):
    d = dev()
    N, B = 64, 9
    x = synth.uniform((B, N), seed=3).numpy()
    big = torch.zeros((B, 2 * N + 2), device=d)
    real = big[:, 1:2 * N + 1:2]                       # x stride 2, odd offset
    real.copy_(torch.from_numpy(x))
    wide = torch.full((B, N, 2), float("nan"), device=d)
    spec = wide[:, :N // 2 + 1, :]                     # padded batch stride
    assert F.fbfft1D(real, spec) == F.Success
    torch.cuda.synchronize()
    _, want = oracle.fbfft1d(x)
    assert rel(spec.cpu().numpy(), want) < TOL_FFT
    assert F.fbifft1D(real, spec) == F.Success
    torch.cuda.synchronize()
    assert rel(real.cpu().numpy(), N * x.astype(np.float64)) < TOL_FFT
    assert float(big[:, 0::2].abs().max()) == 0.0
    # unsupported sizes and shapes
    for n in (3, 6, 512):
        assert F.fbfft1D(torch.zeros((2, n), device=d), torch.zeros((2, n // 2 + 1, 2), device=d)) == F.UnsupportedSize
    assert F.fbfft1D(torch.zeros((2, 32), device=d), torch.zeros((2, 16, 2), device=d)) == F.UnsupportedDimension
    assert F.fbfft1D(torch.zeros((2, 32), device=d), torch.zeros((3, 17, 2), device=d)) == F.UnsupportedDimension
    assert F.fbfft1D(torch.zeros((0, 32), device=d), torch.zeros((0, 17, 2), device=d)) == F.Success
    torch.cuda.synchronize()


@pytest.mark.parametrize("N,B", [(32, 1 << 21), (64, (1 << 20) + 77), (128, (1 << 19) + 5), (256, 1 << 18)])
def test_large_batch_roundtrip(N, B):
    d = dev()
    x = synth.uniform((B, N), seed=2, device=d)
    spec = torch.empty((B, N // 2 + 1, 2), device=d)
    back = torch.empty_like(x)
    assert F.fbfft1D(x, spec) == F.Success
    assert F.fbifft1D(back, spec) == F.Success
    torch.cuda.synchronize()
    assert float((back / N - x).double().norm() / x.double().norm()) < TOL_FFT


@pytest.mark.parametrize("seed", range(30))
def test_random_batches_pads_and_views(oracle, seed):
    """Seeded random draw over size, batch (odd tails), padL and memory layout of
    both operands; forward against the transcription and the fp64 DFT of the
    shifted row, inverse against the transcription (sentinel where it writes nothing)."""
    rng = np.random.default_rng(2000 + seed)
    N = int(rng.choice(SIZES))
    B = int(rng.integers(1, 600))
    padL = int(rng.integers(0, N // 2 + 1)) if rng.random() < 0.4 else 0
    x = synth.uniform((B, N), seed=seed).numpy()
    d = dev()
    kind = int(rng.integers(0, 3))
    if kind == 0:
        real = torch.from_numpy(x).to(d)
    elif kind == 1:                                    # padded batch stride
        big = torch.zeros((B, N + 6), device=d)
        real = big[:, 4:N + 4]
        real.copy_(torch.from_numpy(x))
    else:                                              # rows along the slow axis
        real = torch.from_numpy(np.ascontiguousarray(x.T)).to(d).t()
    if rng.random() < 0.5:
        spec = torch.full((B, N // 2 + 1, 2), float("nan"), device=d)
    else:
        wide = torch.full((B, N // 2 + 3, 2), float("nan"), device=d)
        spec = wide[:, 1:N // 2 + 2, :]
    assert F.fbfft1D(real, spec, padL) == F.Success
    torch.cuda.synchronize()
    _, want = oracle.fbfft1d(x, padL)
    got = spec.cpu().numpy()
    assert rel(got, want) < TOL_FFT, (N, B, padL, kind)
    shifted = np.zeros_like(x)
    shifted[:, padL:] = x[:, :N - padL]
    assert rel(got, oracle.dft1d_r2c(shifted)) < TOL_FFT
    back = torch.full_like(real, 777.0)
    assert F.fbifft1D(back, spec, padL) == F.Success
    torch.cuda.synchronize()
    _, back32 = oracle.fbifft1d(want, padL, out=np.full((B, N), 777.0, np.float32))
    bh = back.cpu().numpy()
    assert np.array_equal(bh == 777.0, back32 == 777.0), (N, B, padL, kind)
    assert rel(bh, back32) < TOL_FFT, (N, B, padL, kind)
