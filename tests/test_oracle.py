"""Pins the CPU oracle without executing the reference (which is CUDA-only and
ships no vectors for this path): closed forms, invariants, brute force on tiny
inputs, numpy.fft fixtures, and the fp64 definitions against each other."""
import os

import numpy as np
import pytest

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "fft_vectors.npz"))
TOL = 1e-5      # rel-L2 per transform
TOL64 = 1e-12   # fp64 definitions


def c(a):
    return a[..., 0] + 1j * a[..., 1]


def rel(a, b):
    return np.linalg.norm(np.ravel(a) - np.ravel(b)) / np.linalg.norm(np.ravel(b))


def embed(x, N, padL, padU):
    X = np.zeros((x.shape[0], N, N))
    X[:, padU:padU + x.shape[1], padL:padL + x.shape[2]] = x
    return X


def spec2d(X, N):
    F = np.fft.fft2(X)
    if N >= 64 or N < 8:
        F = np.transpose(F, (0, 2, 1))
    return F[:, :N // 2 + 1, :]


def test_twiddle_table_is_correctly_rounded(oracle):
    tw = oracle.twiddle_table()
    k = np.arange(128)
    assert np.array_equal(tw[:, 0], np.cos(np.pi * k / 128).astype(np.float32) * (k != 64))
    assert np.array_equal(tw[:, 1], np.sin(np.pi * k / 128).astype(np.float32))
    assert tw[0, 0] == 1.0 and tw[0, 1] == 0.0 and tw[64, 0] == 0.0 and tw[64, 1] == 1.0


def test_twiddle_copies_identical():
    root = os.path.dirname(os.path.dirname(__file__))
    a = open(os.path.join(root, "oracle", "twiddles_f32.inc")).read()
    b = open(os.path.join(root, "fbcuda_amd", "csrc", "twiddles_f32.inc")).read()
    assert a == b


@pytest.mark.parametrize("N", [8, 32, 256])
def test_golden_1d(oracle, N):
    x, f = GOLD["x1d_%d" % N], GOLD["f1d_%d" % N]
    rc, out = oracle.fbfft1d(x)
    assert rc == 0
    assert rel(c(out), f) < TOL
    assert rel(c(oracle.dft1d_r2c(x)), f) < TOL64


@pytest.mark.parametrize("key", [k[4:] for k in GOLD.files if k.startswith("x2d_")])
def test_golden_2d(oracle, key):
    N, h, w, padL, padU = map(int, key.split("_"))
    x, f = GOLD["x2d_" + key], GOLD["f2d_" + key]
    rc, out = oracle.fbfft2d(x, N, padL, padU)
    assert rc == 0
    assert out.shape == (x.shape[0], N // 2 + 1, N, 2)
    assert rel(c(out), f) < TOL
    assert rel(c(oracle.dft2d_r2c(x, N, padL, padU)), f) < TOL64


@pytest.mark.parametrize("N", [2, 4, 8, 16, 32, 64, 128, 256])
@pytest.mark.parametrize("B", [1, 2, 5])
def test_1d_vs_numpy_and_roundtrip(oracle, N, B):
    rng = np.random.default_rng(N * 10 + B)
    x = rng.uniform(-1, 1, (B, N)).astype(np.float32)
    rc, out = oracle.fbfft1d(x)
    assert rc == 0
    assert rel(c(out), np.fft.rfft(x.astype(np.float64), axis=1)) < TOL
    rc, back = oracle.fbifft1d(out)
    assert rel(back, N * x.astype(np.float64)) < TOL  # unnormalised inverse: gain N
    assert rel(oracle.idft1d_c2r(out), N * x.astype(np.float64)) < TOL


def test_1d_unsupported_sizes(oracle):
    for N in (3, 6, 512):
        rc, _ = oracle.fbfft1d(np.zeros((2, N), np.float32))
        assert rc == 1


def test_1d_padl_quirk(oracle):
    """padL shifts right and drops the tail on load; on the inverse store row b
    is written un-shifted and row b+1 shifted (FBFFTCommon.cuh:325, :425-427)."""
    N, padL = 16, 3
    rng = np.random.default_rng(5)
    x = rng.uniform(-1, 1, (2, N)).astype(np.float32)
    shifted = np.zeros_like(x)
    shifted[:, padL:] = x[:, :N - padL]
    rc, out = oracle.fbfft1d(x, padL)
    assert rel(c(out), np.fft.rfft(shifted.astype(np.float64), axis=1)) < TOL
    sentinel = np.full((2, N), 777.0, np.float32)
    rc, back = oracle.fbifft1d(out, padL, out=sentinel.copy())
    full = N * shifted.astype(np.float64)
    assert np.allclose(back[0, padL:], full[0, padL:], atol=1e-4)
    assert np.all(back[0, :padL] == 777.0)
    assert np.allclose(back[1, :N - padL], full[1, padL:], atol=1e-4)
    assert np.all(back[1, N - padL:] == 777.0)


@pytest.mark.parametrize("N", [8, 16, 32, 64, 128])
def test_2d_closed_forms(oracle, N):
    # unit impulse at (y0, x0): e^{-2 pi i (ky y0 + kx x0)/N}
    y0, x0 = 3, 5
    x = np.zeros((1, N, N), np.float32)
    x[0, y0, x0] = 1.0
    rc, out = oracle.fbfft2d(x, N)
    k = np.arange(N)
    full = np.exp(-2j * np.pi * (k[:, None] * y0 + k[None, :] * x0) / N)  # [ky][kx]
    want = full[:N // 2 + 1, :] if N <= 32 else full.T[:N // 2 + 1, :]
    assert rel(c(out)[0], want) < TOL
    assert rel(c(oracle.dft2d_r2c(x, N))[0], want) < TOL64
    # constant plane: N^2 at DC only
    rc, out = oracle.fbfft2d(np.ones((1, N, N), np.float32), N)
    want = np.zeros((N // 2 + 1, N), complex)
    want[0, 0] = N * N
    assert np.abs(c(out)[0] - want).max() < 1e-3
    # checkerboard (-1)^(x+y): N^2 at (N/2, N/2) only
    yy, xx = np.mgrid[0:N, 0:N]
    rc, out = oracle.fbfft2d(((-1.0) ** (yy + xx))[None].astype(np.float32), N)
    want = np.zeros((N // 2 + 1, N), complex)
    want[N // 2, N // 2] = N * N
    assert np.abs(c(out)[0] - want).max() < 1e-3
    # single cosine along x with frequency 3: two bins on the kx axis
    rc, out = oracle.fbfft2d(np.cos(2 * np.pi * 3 * xx / N)[None].astype(np.float32), N)
    want = np.zeros((N, N), complex)  # [ky][kx]
    want[0, 3] = want[0, N - 3] = N * N / 2
    want = want[:N // 2 + 1, :] if N <= 32 else want.T[:N // 2 + 1, :]
    assert np.abs(c(out)[0] - want).max() < 2e-3


@pytest.mark.parametrize("N", [8, 16, 32, 64, 128])
@pytest.mark.parametrize("case", ["full", "ragged", "padded", "tiny"])
def test_2d_vs_numpy_roundtrip_invariants(oracle, N, case):
    rng = np.random.default_rng(N)
    h, w, padL, padU = {"full": (N, N, 0, 0), "ragged": (N - 5, N - 3, 0, 0),
                        "padded": (N - 5, N - 4, 2, 3), "tiny": (5, 5, 0, 0)}[case]
    B = 3  # odd: exercises the unpaired plane of the N >= 64 inverse
    x = rng.standard_normal((B, h, w)).astype(np.float32)
    rc, out = oracle.fbfft2d(x, N, padL, padU)
    assert rc == 0
    X = embed(x, N, padL, padU)
    assert rel(c(out), spec2d(X, N)) < TOL
    # crop-on-store equals crop-after; unnormalised inverse has gain N^2
    rc, back = oracle.fbifft2d(out, h, w, padL, padU)
    assert rel(back, N * N * x.astype(np.float64)) < TOL
    # linearity
    y = rng.standard_normal((B, h, w)).astype(np.float32)
    _, oy = oracle.fbfft2d(y, N, padL, padU)
    _, oxy = oracle.fbfft2d((2 * x + y).astype(np.float32), N, padL, padU)
    assert rel(c(oxy), 2 * c(out) + c(oy)) < TOL
    # Parseval with Hermitian weights on the halved axis
    wts = np.full(N // 2 + 1, 2.0)
    wts[0] = wts[N // 2] = 1.0
    energy = (np.abs(c(out)) ** 2 * wts[None, :, None]).sum(axis=(1, 2)) / (N * N)
    assert np.allclose(energy, (X ** 2).sum(axis=(1, 2)), rtol=1e-5)
    # halved-axis rows 0 and N/2 are Hermitian along the full axis
    for r in (0, N // 2):
        row = c(out)[:, r, :]
        assert np.abs(row - np.conj(np.roll(row[:, ::-1], 1, axis=1))).max() < 1e-3 * N
    # shift theorem for padL / padU against the unpadded transform
    if case == "padded":
        _, o0 = oracle.fbfft2d(x, N, 0, 0)
        k = np.arange(N)
        ph = np.exp(-2j * np.pi * (k[:, None] * padU + k[None, :] * padL) / N)
        ph = ph[:N // 2 + 1, :] if N <= 32 else ph.T[:N // 2 + 1, :]
        assert rel(c(out), c(o0) * ph[None]) < TOL


@pytest.mark.parametrize("N", [2, 4])
@pytest.mark.parametrize("B", [1, 2, 5])
def test_2d_warp_sizes(oracle, N, B):
    """N = 2 and 4 go through the plane-pairing warp kernel and use the transposed
    [kx half][ky] layout; an odd batch leaves the last plane unpaired."""
    rng = np.random.default_rng(10 * N + B)
    for h, w, padL, padU in [(N, N, 0, 0), (N - 1, N, 0, 0), (N - 1, N - 1, 1, 1)]:
        x = rng.standard_normal((B, h, w)).astype(np.float32)
        rc, out = oracle.fbfft2d(x, N, padL, padU)
        assert rc == 0 and out.shape == (B, N // 2 + 1, N, 2)
        X = embed(x, N, padL, padU)
        assert rel(c(out), spec2d(X, N)) < TOL
        assert rel(c(oracle.dft2d_r2c(x, N, padL, padU)), spec2d(X, N)) < TOL64
        rc, back = oracle.fbifft2d(out, h, w, padL, padU)
        assert rc == 0 and rel(back, N * N * x.astype(np.float64)) < TOL
    # closed forms, literal: impulse at (y0, x0) = (1, N-1); out[kx][ky]
    x = np.zeros((1, N, N), np.float32)
    x[0, 1, N - 1] = 1.0
    _, out = oracle.fbfft2d(x, N)
    k = np.arange(N)
    want = np.exp(-2j * np.pi * (k[None, :] * 1 + k[:, None] * (N - 1)) / N)[:N // 2 + 1]  # [kx][ky]
    assert np.abs(c(out)[0] - want).max() < 1e-6
    # an x-only ramp has energy only at ky = 0: tells [kx][ky] from [ky][kx]
    ramp = np.tile(np.arange(N, dtype=np.float32), (N, 1))[None]
    _, out = oracle.fbfft2d(ramp, N)
    assert np.abs(c(out)[0][:, 1:]).max() < 1e-6 and abs(c(out)[0][1, 0]) > 1.0


def test_2d_unsupported_sizes(oracle):
    for N in (1, 12, 256):
        rc, _ = oracle.fbfft2d(np.zeros((1, N, N), np.float32), N)
        assert rc == 1


def test_2d_inverse_lane0_quirk(oracle):
    """The N <= 32 inverse keeps only the real parts of F[0][0] and F[N/2][0]
    (FFT2D32.cuh:313-315): perturbing their imaginary parts changes nothing."""
    N = 16
    rng = np.random.default_rng(1)
    x = rng.standard_normal((1, N, N)).astype(np.float32)
    _, spec = oracle.fbfft2d(x, N)
    _, a = oracle.fbifft2d(spec, N, N)
    spec2 = spec.copy()
    spec2[0, 0, 0, 1] = 5.0
    spec2[0, N // 2, 0, 1] = -7.0
    _, b = oracle.fbifft2d(spec2, N, N)
    assert np.array_equal(a, b)


@pytest.mark.parametrize("conjA,conjB", [(0, 1), (1, 0), (0, 0)])
def test_transpose_mm(oracle, conjA, conjB):
    rng = np.random.default_rng(3)
    I, J, K, XY = 5, 6, 7, 40
    A = rng.standard_normal(((K, I) if conjA else (I, K)) + (XY, 2)).astype(np.float32)
    B = rng.standard_normal(((J, K) if conjB else (K, J)) + (XY, 2)).astype(np.float32)
    Ac, Bc = c(A).astype(complex), c(B).astype(complex)
    if conjA:
        Ac = np.conj(Ac).transpose(1, 0, 2)
    if conjB:
        Bc = np.conj(Bc).transpose(1, 0, 2)
    want = 0.25 * np.einsum("ikx,kjx->ijx", Ac, Bc)
    assert rel(c(oracle.transpose_mm(A, B, conjA, conjB, 0.25)), want) < TOL
    assert rel(c(oracle.transpose_mm64(A, B, conjA, conjB, 0.25)), want) < TOL64
    # accumulate: invNorm scales the accumulated-into value too (MM-inl.cuh:322-324)
    C0 = rng.standard_normal((I, J, XY, 2)).astype(np.float32)
    got = oracle.transpose_mm(A, B, conjA, conjB, 0.25, C=C0)
    assert rel(c(got), want + 0.25 * c(C0)) < TOL


def test_corr64_against_torch(oracle):
    import torch
    rng = np.random.default_rng(4)
    x = rng.standard_normal((2, 3, 9, 10)).astype(np.float32)
    w = rng.standard_normal((4, 3, 3, 2)).astype(np.float32)
    xt = torch.from_numpy(x).double().requires_grad_()
    wt = torch.from_numpy(w).double().requires_grad_()
    out = torch.nn.functional.conv2d(xt, wt)
    assert rel(oracle.corr2d_valid(x, w), out.detach().numpy()) < TOL64
    g = rng.standard_normal(tuple(out.shape)).astype(np.float32)
    out.backward(torch.from_numpy(g).double())
    assert rel(oracle.corr2d_grad_input(g, w, 9, 10), xt.grad.numpy()) < TOL64
    assert rel(oracle.corr2d_grad_weight(x, g, 3, 2), wt.grad.numpy()) < TOL64
    coords = np.array([[0, 0, 0, 0], [1, 3, 6, 8], [1, 2, 3, 4]], np.int32)
    at = oracle.corr2d_valid_at(x, w, coords)
    assert np.allclose(at, [out[tuple(cc)].item() for cc in coords], rtol=1e-12)
    # the subset forms of the two gradients: every element, against torch's autograd
    # (borders, where part of the filter hangs over the edge of gradOutput, included)
    gi_all = np.array([(n, ch, y, xx) for n in range(2) for ch in range(3) for y in range(9)
                       for xx in range(10)], np.int32)
    got = oracle.corr2d_grad_input_at(g, w, 9, 10, gi_all).reshape(2, 3, 9, 10)
    assert rel(got, xt.grad.numpy()) < TOL64
    gw_all = np.array([(f, ch, u, v) for f in range(4) for ch in range(3) for u in range(3)
                       for v in range(2)], np.int32)
    got = oracle.corr2d_grad_weight_at(x, g, 3, 2, gw_all).reshape(4, 3, 3, 2)
    assert rel(got, wt.grad.numpy()) < TOL64
    # a shuffled subset returns the same values in the order asked for
    pick = rng.permutation(len(gi_all))[:17]
    assert np.allclose(oracle.corr2d_grad_input_at(g, w, 9, 10, gi_all[pick]),
                       xt.grad.numpy().reshape(-1)[pick], rtol=1e-12, atol=1e-14)


def tiles_for(H, W, k, N):
    """Overlapping N x N input windows with origin stride N-k+1 and their valid output windows."""
    oH, oW, step = H - k + 1, W - k + 1, N - k + 1
    iv, ov = [], []
    for y0 in range(0, oH, step):
        for x0 in range(0, oW, step):
            iv.append((y0, x0, min(N, H - y0), min(N, W - x0), 0, 0))
            ov.append((y0, x0, min(step, oH - y0), min(step, oW - x0), 0, 0))
    return iv, ov


@pytest.mark.parametrize("N,k,H,W", [(8, 3, 14, 17), (16, 5, 30, 25), (32, 9, 40, 56)])
def test_iterated_conv_passes(oracle, N, k, H, W):
    rng = np.random.default_rng(N)
    Nb, Cin, Cout = 2, 3, 4
    x = rng.uniform(-1, 1, (Nb, Cin, H, W)).astype(np.float32)
    w = (0.05 * rng.standard_normal((Cout, Cin, k, k))).astype(np.float32)
    iv, ov = tiles_for(H, W, k, N)
    out = np.zeros((Nb, Cout, H - k + 1, W - k + 1), np.float32)
    assert oracle.iterated_conv(N, x, iv, out, ov, w, 0) == 1
    assert rel(out, oracle.corr2d_valid(x, w)) < 1e-4
    g = rng.standard_normal(out.shape).astype(np.float32)
    gw = np.zeros_like(w)
    assert oracle.iterated_conv(N, x, iv, g, ov, gw, 2, 0.5) == 1
    assert rel(gw, 0.5 * oracle.corr2d_grad_weight(x, g, k, k)) < 1e-4
    # gradInput: one tile covering the whole (small) plane
    xs = np.zeros((Nb, Cin, N, N), np.float32)
    gs = rng.standard_normal((Nb, Cout, N - k + 1, N - k + 1)).astype(np.float32)
    assert oracle.iterated_conv(N, xs, [(0, 0, N, N, 0, 0)], gs, [(0, 0, N - k + 1, N - k + 1, 0, 0)], w, 1) == 1
    assert rel(xs, oracle.corr2d_grad_input(gs, w, N, N)) < 1e-4
    assert oracle.iterated_conv(N, x, iv, out, ov, w, 7) == 0   # unknown pass code
    assert oracle.iterated_conv(64, x, iv, out, ov, w, 0) == 0  # unsupported size


def test_brute_force_tiny(oracle):
    """N = 8, B = 3 (odd tail of the 1D pairing) against a literal double sum."""
    rng = np.random.default_rng(8)
    x = rng.standard_normal((3, 8)).astype(np.float32)
    _, out = oracle.fbfft1d(x)
    want = np.array([[sum(x[b, n] * np.exp(-2j * np.pi * k * n / 8) for n in range(8))
                      for k in range(5)] for b in range(3)])
    assert rel(c(out), want) < TOL


# ---- packed spectrum format (FFT2D32.cuh:421-427, :302-316; product rule of
# FFTIteratedConvolution.cuh:161-186) ----

from packed_util import as_float, pack, unpack  # noqa: E402


def test_pack_unpack_helpers_are_inverse():
    rng = np.random.default_rng(3)
    X = rng.standard_normal((2, 16, 16))
    U = np.fft.fft2(X)[:, :9, :]
    assert np.allclose(unpack(pack(U)), U, atol=1e-12)
    P = rng.standard_normal((3, 8, 16)) + 1j * rng.standard_normal((3, 8, 16))
    assert np.allclose(pack(unpack(P)), P, atol=1e-12)


@pytest.mark.parametrize("N,h,w,padL,padU", [(8, 8, 8, 0, 0), (16, 16, 16, 0, 0), (32, 32, 32, 0, 0),
                                              (32, 27, 27, 0, 0), (16, 5, 7, 3, 2), (8, 3, 3, 5, 4)])
def test_packed_forward_is_the_packed_dft(oracle, N, h, w, padL, padU):
    rng = np.random.default_rng(N + h)
    x = rng.standard_normal((5, h, w)).astype(np.float32)
    rc, got = oracle.fbfft2d_packed(x, N, padL, padU)
    assert rc == 0 and got.shape == (5, N // 2, N, 2)
    want = pack(spec2d(embed(x.astype(np.float64), N, padL, padU), N))
    assert rel(c(got), want) < TOL
    # and against the transcription of the unpacked store
    _, unp = oracle.fbfft2d(x, N, padL, padU)
    assert rel(unpack(c(got)), c(unp)) < TOL


@pytest.mark.parametrize("N,h,w,padL,padU", [(8, 8, 8, 0, 0), (16, 16, 16, 0, 0), (32, 32, 32, 0, 0),
                                              (32, 23, 23, 0, 0), (16, 9, 6, 2, 5)])
def test_packed_inverse_inverts_the_packed_dft(oracle, N, h, w, padL, padU):
    rng = np.random.default_rng(7 * N + w)
    X = rng.standard_normal((4, N, N))
    P = as_float(pack(spec2d(X, N)))
    rc, back = oracle.fbifft2d_packed(P, h, w, padL, padU)
    assert rc == 0
    assert rel(back, N * N * X[:, padU:padU + h, padL:padL + w]) < TOL


@pytest.mark.parametrize("conjA,conjB", [(False, True), (True, False), (False, False)])
@pytest.mark.parametrize("N", [8, 16, 32])
def test_packed_contraction_is_the_contraction_of_the_unpacked_spectra(oracle, N, conjA, conjB):
    rng = np.random.default_rng(100 + N)
    I, J, K = 3, 4, 5

    def spectra(d0, d1):
        return as_float(pack(spec2d(rng.standard_normal((d0 * d1, N, N)), N)).reshape(d0, d1, N // 2, N))

    A = spectra(*((K, I) if conjA else (I, K)))
    B = spectra(*((J, K) if conjB else (K, J)))
    got = oracle.transpose_mm_packed(A, B, conjA, conjB, 0.25)
    UA, UB = unpack(c(A)), unpack(c(B))
    a = np.conj(UA).transpose(1, 0, 2, 3) if conjA else UA
    b = np.conj(UB).transpose(1, 0, 2, 3) if conjB else UB
    want = 0.25 * np.einsum("ikyx,kjyx->ijyx", a, b)
    assert rel(unpack(c(got)), want) < TOL
    assert rel(c(got), pack(want)) < TOL
    # Accumulate: invNorm scales the accumulated-into value as well (MM-inl.cuh:322-324)
    C0 = spectra(I, J)
    acc = oracle.transpose_mm_packed(A, B, conjA, conjB, 0.25, C=C0)
    assert rel(c(acc), pack(want + 0.25 * unpack(c(C0)))) < TOL


def test_packed_layer_equals_direct_correlation(oracle):
    """packed FFT -> packed contraction -> packed inverse = fp64 valid correlation."""
    N, Nb, Cin, Cout, H, k = 16, 2, 3, 4, 13, 4
    rng = np.random.default_rng(9)
    x = rng.standard_normal((Nb, Cin, H, H)).astype(np.float32)
    w = rng.standard_normal((Cout, Cin, k, k)).astype(np.float32)
    _, X = oracle.fbfft2d_packed(x.reshape(-1, H, H), N)
    _, W = oracle.fbfft2d_packed(w.reshape(-1, k, k), N)
    X = X.reshape(Nb, Cin, N // 2, N, 2)
    W = W.reshape(Cout, Cin, N // 2, N, 2)
    O = oracle.transpose_mm_packed(X, W, False, True, 1.0 / (N * N))
    o = H - k + 1
    _, out = oracle.fbifft2d_packed(O.reshape(-1, N // 2, N, 2), o, o)
    assert rel(out.reshape(Nb, Cout, o, o), oracle.corr2d_valid(x, w)) < 1e-4
