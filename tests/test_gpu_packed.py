"""GPU parity of the packed spectrum format (the Unpack = false store and the
PackedInput = true inverse of fbfft/FFT2D32.cuh:302-316, 421-427) and of the contraction
on packed operands (fbfft_transpose_mm_packed; product rule of
fbfft/FFTIteratedConvolution.cuh:161-186), through the C ABI, against the CPU
transcription and the fp64 definitions."""
import numpy as np
import pytest
import torch

import fbcuda_amd as F
from fbcuda_amd import synth
from gpu_util import TOL_CONV, TOL_FFT, c, dev, rel
from packed_util import as_float, pack, unpack

pytestmark = pytest.mark.gpu


def fwd_packed(x, N, padL=0, padU=0):
    xd = torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to(dev())
    out = torch.full((x.shape[0], N // 2, N, 2), float("nan"), device=dev())
    rc = F.fbfft2D(xd, out, padL, padU)
    torch.cuda.synchronize()
    return rc, out.cpu().numpy()


def inv_packed(P, h, w, padL=0, padU=0):
    pd = torch.from_numpy(np.ascontiguousarray(P, dtype=np.float32)).to(dev())
    out = torch.full((P.shape[0], h, w), float("nan"), device=dev())
    rc = F.fbifft2D(pd, out, padL, padU)
    torch.cuda.synchronize()
    return rc, out.cpu().numpy()


@pytest.mark.parametrize("N,B,h,w,padL,padU", [
    (8, 1, 8, 8, 0, 0), (8, 37, 8, 8, 0, 0), (16, 8, 16, 16, 0, 0), (16, 21, 11, 7, 3, 2),
    (32, 4, 32, 32, 0, 0), (32, 9, 32, 32, 0, 0), (32, 130, 27, 27, 0, 0), (32, 7, 5, 5, 0, 0),
    (32, 3, 20, 31, 1, 9), (16, 1025, 16, 16, 0, 0), (8, 4099, 8, 8, 0, 0),
])
def test_packed_forward_and_inverse(oracle, N, B, h, w, padL, padU):
    x = synth.normal((B, h, w), seed=N + B).numpy()
    rc, got = fwd_packed(x, N, padL, padU)
    assert rc == F.Success
    _, want32 = oracle.fbfft2d_packed(x, N, padL, padU)
    assert rel(c(got), c(want32)) < TOL_FFT
    want64 = pack(c(oracle.dft2d_r2c(x, N, padL, padU)))
    assert rel(c(got), want64) < TOL_FFT
    # the unpacked store of the same planes carries the same numbers
    from gpu_util import fft2d
    _, unp = fft2d(x, N, padL, padU)
    assert rel(unpack(c(got)), c(unp)) < TOL_FFT
    # packed inverse, cropped back to the window
    rc, back = inv_packed(got, h, w, padL, padU)
    assert rc == F.Success
    assert rel(back, N * N * x.astype(np.float64)) < TOL_FFT
    _, back32 = oracle.fbifft2d_packed(got, h, w, padL, padU)
    assert rel(back, back32) < TOL_FFT


def test_packed_strided_views(oracle):
    """Packed spectra through non-contiguous views (plane stride with a gap, rows with a
    gap): the generic copy paths."""
    N, B = 32, 6
    x = synth.normal((B, N, N), seed=5).to(dev())
    store = torch.full((B, N // 2 + 3, N + 2, 2), float("nan"), device=dev())
    spec = store[:, 1:N // 2 + 1, 1:N + 1, :]
    assert F.fbfft2D(x, spec) == F.Success
    torch.cuda.synchronize()
    _, want = oracle.fbfft2d_packed(x.cpu().numpy(), N)
    assert rel(c(spec.cpu().numpy()), c(want)) < TOL_FFT
    assert bool(torch.isnan(store[:, 0]).all()) and bool(torch.isnan(store[:, :, 0]).all())
    back = torch.empty_like(x)
    assert F.fbifft2D(spec, back) == F.Success
    torch.cuda.synchronize()
    assert rel(back.cpu().numpy(), N * N * x.cpu().numpy().astype(np.float64)) < TOL_FFT


ROLES = [(False, True), (True, False), (False, False)]


def mm_packed(A, B, conjA, conjB, invNorm, C0=None):
    Ad, Bd = torch.from_numpy(A).to(dev()), torch.from_numpy(B).to(dev())
    I = A.shape[1] if conjA else A.shape[0]
    J = B.shape[0] if conjB else B.shape[1]
    Cd = (torch.full((I, J) + A.shape[2:], float("nan"), device=dev()) if C0 is None
          else torch.from_numpy(C0).to(dev()))
    rc = F.transposeMM(Ad, Bd, Cd, invNorm, conjA, conjB, C0 is not None, packed=True)
    torch.cuda.synchronize()
    return rc, Cd.cpu().numpy()


@pytest.mark.parametrize("conjA,conjB", ROLES)
@pytest.mark.parametrize("N,I,J,K", [(8, 5, 7, 3), (16, 33, 70, 9), (32, 64, 64, 16), (32, 70, 3, 5),
                                     (8, 1, 1, 1), (16, 130, 65, 4)])
def test_packed_contraction(oracle, N, I, J, K, conjA, conjB):
    A = synth.normal(((K, I) if conjA else (I, K)) + (N // 2, N, 2), seed=11).numpy()
    B = synth.normal(((J, K) if conjB else (K, J)) + (N // 2, N, 2), seed=12).numpy()
    rc, got = mm_packed(A, B, conjA, conjB, 0.125)
    assert rc == F.Success
    want32 = oracle.transpose_mm_packed(A, B, conjA, conjB, 0.125)
    assert rel(c(got), c(want32)) < TOL_FFT
    UA, UB = unpack(c(A)), unpack(c(B))
    a = np.conj(UA).transpose(1, 0, 2, 3) if conjA else UA
    b = np.conj(UB).transpose(1, 0, 2, 3) if conjB else UB
    want64 = pack(0.125 * np.einsum("ikyx,kjyx->ijyx", a, b))
    assert rel(c(got), want64) < TOL_FFT
    C0 = synth.normal((I, J, N // 2, N, 2), seed=13).numpy()
    rc, acc = mm_packed(A, B, conjA, conjB, 0.125, C0=C0)
    assert rc == F.Success
    assert rel(c(acc), c(oracle.transpose_mm_packed(A, B, conjA, conjB, 0.125, C=C0))) < TOL_FFT


def test_packed_contraction_rejects_other_shapes():
    d = dev()
    A = torch.zeros((4, 3, 17, 32, 2), device=d)   # unpacked spectra are not packed operands
    assert F.transposeMM(A, A, A, 1.0, False, True, packed=True) == F.UnsupportedSize
    A4 = torch.zeros((4, 3, 16 * 32, 2), device=d)  # rank 4: the row length is not known
    assert F.transposeMM(A4, A4, A4, 1.0, False, True, packed=True) == F.UnsupportedDimension
    A64 = torch.zeros((2, 2, 32, 64, 2), device=d)  # the format exists for N <= 32 only
    assert F.transposeMM(A64, A64, A64, 1.0, False, True, packed=True) == F.UnsupportedSize


@pytest.mark.parametrize("Nb,Cin,Cout", [(4, 5, 6), (16, 64, 24)])
def test_packed_layer_config3_shapes(oracle, Nb, Cin, Cout):
    """configs[3] plane shapes (27x27 activations, 5x5 filters, 32-point transforms, 23x23
    valid output) composed from the primitives on PACKED spectra: fbfft2D -> transposeMM ->
    fbifft2D.  Equals the fp64 direct correlation and the same composition on unpacked
    spectra."""
    N, H, k = 32, 27, 5
    o = H - k + 1
    d = dev()
    x = synth.normal((Nb, Cin, H, H), seed=30, device=d)
    w = synth.normal((Cout, Cin, k, k), seed=31, std=0.02, device=d)

    def layer(rows, packed):
        X = torch.empty((Nb, Cin, rows, N, 2), device=d)
        W = torch.empty((Cout, Cin, rows, N, 2), device=d)
        O = torch.empty((Nb, Cout, rows, N, 2), device=d)
        out = torch.full((Nb, Cout, o, o), float("nan"), device=d)
        assert F.fbfft2D(x.view(-1, H, H), X.view(-1, rows, N, 2)) == F.Success
        assert F.fbfft2D(w.view(-1, k, k), W.view(-1, rows, N, 2)) == F.Success
        assert F.transposeMM(X, W, O, 1.0 / (N * N), False, True, packed=packed) == F.Success
        assert F.fbifft2D(O.view(-1, rows, N, 2), out.view(-1, o, o)) == F.Success
        torch.cuda.synchronize()
        return out.cpu().numpy()

    got = layer(N // 2, True)
    want = oracle.corr2d_valid(x.cpu().numpy(), w.cpu().numpy())
    assert rel(got, want) < TOL_CONV
    assert rel(got, layer(N // 2 + 1, False)) < TOL_CONV
