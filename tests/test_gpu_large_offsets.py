"""Operands whose element offsets pass 2^31 (more than 8 GiB of fp32 per tensor):
the strides of a view are ints, as in the reference's DeviceTensor, but plane and
row offsets must be formed in 64 bits.  The first and the last planes / rows of
each batch are checked against the oracle; everything between is covered by a
round trip over the whole batch."""
import numpy as np
import pytest
import torch

import fbcuda_amd as F
from gpu_util import TOL_FFT, dev, rel

pytestmark = pytest.mark.gpu


def fill(shape, seed):
    g = torch.Generator(device=dev())
    g.manual_seed(seed)
    return torch.randn(shape, device=dev(), generator=g)


def needs(gib):
    free, _ = torch.cuda.mem_get_info()
    if free < gib * (1 << 30):
        pytest.skip("needs %d GiB of free device memory" % gib)


def roundtrip_error(x, back, scale, chunk):
    """max over chunks of planes/rows of the relative round-trip error (on the device)"""
    worst = 0.0
    for i in range(0, x.shape[0], chunk):
        a, b = x[i:i + chunk].double(), back[i:i + chunk].double() / scale
        worst = max(worst, float((a - b).norm() / a.norm()))
    return worst


def test_2d_batch_beyond_2_31_elements(oracle):
    N, B = 32, (1 << 21) + 5          # input 2^31 + 5120 floats, spectrum 2.28e9 floats
    needs(30)
    x = fill((B, N, N), 11)
    spec = torch.empty((B, N // 2 + 1, N, 2), device=dev())
    assert F.fbfft2D(x, spec) == F.Success
    torch.cuda.synchronize()
    for sl in (slice(0, 3), slice(B - 7, B)):
        _, want = oracle.fbfft2d(x[sl].cpu().numpy(), N)
        assert rel(spec[sl].cpu().numpy(), want) < TOL_FFT
    back = torch.empty_like(x)
    assert F.fbifft2D(spec, back) == F.Success
    torch.cuda.synchronize()
    assert roundtrip_error(x, back, N * N, 1 << 18) < TOL_FFT


def test_1d_batch_beyond_2_31_elements(oracle):
    N, B = 256, (1 << 23) + 3         # input 2^31 + 768 floats
    needs(30)
    x = fill((B, N), 12)
    spec = torch.empty((B, N // 2 + 1, 2), device=dev())
    assert F.fbfft1D(x, spec) == F.Success
    torch.cuda.synchronize()
    for sl in (slice(0, 3), slice(B - 5, B)):
        want = oracle.dft1d_r2c(x[sl].cpu().numpy())
        assert rel(spec[sl].cpu().numpy(), want) < TOL_FFT
    back = torch.empty_like(x)
    assert F.fbifft1D(back, spec) == F.Success
    torch.cuda.synchronize()
    assert roundtrip_error(x, back, N, 1 << 20) < TOL_FFT


def test_2d_large_planes_beyond_2_31_elements(oracle):
    N, B = 128, (1 << 17) + 2         # input 2^31 + 32768 floats
    needs(30)
    x = fill((B, N, N), 13)
    spec = torch.empty((B, N // 2 + 1, N, 2), device=dev())
    assert F.fbfft2D(x, spec) == F.Success
    torch.cuda.synchronize()
    for sl in (slice(0, 1), slice(B - 2, B)):
        _, want = oracle.fbfft2d(x[sl].cpu().numpy(), N)
        assert rel(spec[sl].cpu().numpy(), want) < TOL_FFT
    back = torch.empty_like(x)
    assert F.fbifft2D(spec, back) == F.Success
    torch.cuda.synchronize()
    assert roundtrip_error(x, back, N * N, 1 << 14) < TOL_FFT
