"""The reference's two-call forms for 64 x 64 and 128 x 128 (scratch owned by the
caller) give the same result as the oracle and as the single-kernel path."""
import numpy as np
import pytest
import torch

import fbcuda_amd as F
from fbcuda_amd import synth
from gpu_util import TOL_FFT, dev, rel

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("N", [64, 128])
@pytest.mark.parametrize("B", [1, 4, 5])
@pytest.mark.parametrize("case", ["full", "padded", "aligned", "aligned_narrow"])
def test_two_call_forward_and_inverse(oracle, N, B, case):
    d = dev()
    # "aligned*": width and left edge multiples of 4 (16-byte loads of the first pass)
    h, w, padL, padU = {"full": (N, N, 0, 0), "padded": (N - 9, N - 6, 4, 3),
                        "aligned": (N - 9, N - 8, 4, 3), "aligned_narrow": (7, 12, 8, 0)}[case]
    x = synth.normal((B, h, w), seed=N + B).numpy()
    xd = torch.from_numpy(x).to(d)
    nc = N // 2 + 1
    # forward: real -> scratch [B][N][N/2+1] -> dst [B][N/2+1][N]
    scratch = torch.full((B, N, nc, 2), float("nan"), device=d)
    dst = torch.full((B, nc, N, 2), float("nan"), device=d)
    assert F.fbfft2D(xd, scratch, padL, padU) == F.Success
    assert F.fbfft2D_pass2(scratch, dst) == F.Success
    torch.cuda.synchronize()
    _, want = oracle.fbfft2d(x, N, padL, padU)
    assert rel(dst.cpu().numpy(), want) < TOL_FFT
    # the scratch holds the row transforms: rfft along x of the padded plane
    X = np.zeros((B, N, N))
    X[:, padU:padU + h, padL:padL + w] = x
    rows = np.fft.rfft(X, axis=2)
    sc = scratch.cpu().numpy()
    assert rel(sc[..., 0] + 1j * sc[..., 1], rows) < TOL_FFT
    single = torch.empty_like(dst)
    assert F.fbfft2D(xd, single, padL, padU) == F.Success
    torch.cuda.synchronize()
    assert rel(single.cpu().numpy(), dst.cpu().numpy()) < TOL_FFT
    # inverse: src [B][N/2+1][N] -> scratch [B][N][N] (planes paired) -> real
    spec = torch.from_numpy(want).to(d)
    iscratch = torch.zeros((B, N, N, 2), device=d)
    back = torch.full((B, h, w), float("nan"), device=d)
    assert F.fbifft2D_pass1(spec, iscratch) == F.Success
    assert F.fbifft2D(iscratch, back, padL, padU) == F.Success
    torch.cuda.synchronize()
    _, back32 = oracle.fbifft2d(want, h, w, padL, padU)
    assert rel(back.cpu().numpy(), back32) < TOL_FFT
    assert rel(back.cpu().numpy(), N * N * x.astype(np.float64)) < TOL_FFT


def test_two_call_errors():
    d = dev()
    z = lambda *s: torch.zeros(s, device=d)
    assert F.fbfft2D_pass2(z(2, 32, 17, 2), z(2, 17, 32, 2)) == F.UnsupportedSize
    assert F.fbfft2D_pass2(z(2, 64, 33, 2), z(2, 33, 32, 2)) == F.UnsupportedSize
    assert F.fbfft2D_pass2(z(2, 64, 33, 2), z(3, 33, 64, 2)) == F.UnsupportedDimension
    assert F.fbifft2D_pass1(z(2, 17, 32, 2), z(2, 32, 32, 2)) == F.UnsupportedSize
    assert F.fbifft2D_pass1(z(2, 33, 64, 2), z(2, 64, 32, 2)) == F.UnsupportedSize
    assert F.fbifft2D_pass1(z(4, 33, 64, 2), z(1, 64, 64, 2)) == F.UnsupportedDimension
    torch.cuda.synchronize()
