"""GPU parity of transposeMM (C ABI fbfft_transpose_mm) and of the FFT convolution
forward pass built from the primitives (fbfft_conv_fprop)."""
import numpy as np
import pytest
import torch

import fbcuda_amd as F
from fbcuda_amd import synth
from gpu_util import check, TOL_CONV, TOL_FFT, dev, rel

pytestmark = pytest.mark.gpu


def mm(A, B, conjA, conjB, invNorm, C0=None):
    Ad = torch.from_numpy(A).to(dev())
    Bd = torch.from_numpy(B).to(dev())
    I = A.shape[1] if conjA else A.shape[0]
    J = B.shape[0] if conjB else B.shape[1]
    if C0 is None:
        Cd = torch.full((I, J) + A.shape[2:], float("nan"), device=dev())
    else:
        Cd = torch.from_numpy(C0).to(dev())
    rc = F.transposeMM(Ad, Bd, Cd, invNorm, conjA, conjB, C0 is not None)
    torch.cuda.synchronize()
    return rc, Cd.cpu().numpy()


ROLES = [(False, True), (True, False), (False, False)]  # updateOutput, accGrad, updateGradInput


@pytest.mark.parametrize("conjA,conjB", ROLES)
@pytest.mark.parametrize("I,J,K,shape", [
    (32, 32, 4, (5, 8)),        # one tile, xy = 40 (N = 8 spectra)
    (64, 96, 16, (9, 16)),      # N = 16 spectra
    (33, 7, 5, (17, 32)),       # ragged I/J/K, xy = 544
    (1, 3, 3, (5, 8)),          # batch 1, RGB-like reduction
    (40, 70, 64, (3, 2)),       # xy = 6: partial bin chunk
    (8, 8, 9, (3, 3)),          # odd xy (last bin has no pair), three slices with a tail
    (16, 8, 1, (1, 5)),         # a single k
    (70, 130, 12, (1, 13)),     # several tiles both ways, odd xy
    (9, 5, 3, (33, 64)),        # N = 64 spectra (MM-inl.cuh:778 has no instantiation for them)
    (4, 6, 5, (65, 128)),       # N = 128 spectra
])
def test_mm_vs_oracle(oracle, conjA, conjB, I, J, K, shape):
    xy = shape[0] * shape[1]
    A = synth.normal(((K, I) if conjA else (I, K)) + shape + (2,), seed=1).numpy()
    B = synth.normal(((J, K) if conjB else (K, J)) + shape + (2,), seed=2).numpy()
    rc, got = mm(A, B, conjA, conjB, 0.125)
    assert rc == F.Success
    A3 = A.reshape(A.shape[0], A.shape[1], xy, 2)
    B3 = B.reshape(B.shape[0], B.shape[1], xy, 2)
    want32 = oracle.transpose_mm(A3, B3, conjA, conjB, 0.125)
    want64 = oracle.transpose_mm64(A3, B3, conjA, conjB, 0.125)
    got3 = got.reshape(I, J, xy, 2)
    assert rel(got3, want32) < TOL_FFT
    assert rel(got3, want64) < TOL_FFT
    # Accumulate: invNorm scales the accumulated-into value as well (MM-inl.cuh:322-324)
    C0 = synth.normal((I, J) + shape + (2,), seed=3).numpy()
    rc, acc = mm(A, B, conjA, conjB, 0.125, C0=C0)
    assert rc == F.Success
    want_acc = oracle.transpose_mm(A3, B3, conjA, conjB, 0.125, C=C0.reshape(I, J, xy, 2))
    assert rel(acc.reshape(I, J, xy, 2), want_acc) < TOL_FFT


@pytest.mark.parametrize("conjA,conjB", ROLES)
def test_mm_cancellation_per_element(oracle, conjA, conjB):
    """The contraction forms a complex product from three real products; its imaginary
    and real parts are differences of larger terms.  Operands with |re| close to |im| and
    a long reduction make those differences cancel: every element must stay within a
    bound relative to sum_k (|a_re|+|a_im|)(|b_re|+|b_im|), not just in the norm."""
    I, J, K, xy = 40, 24, 512, 12
    rng = np.random.default_rng(77)

    def near_diagonal(shape):
        mag = rng.uniform(0.5, 2.0, shape) * rng.choice([-1.0, 1.0], shape)
        eps = rng.uniform(-1e-3, 1e-3, shape)
        return np.stack([mag, mag * (1.0 + eps)], axis=-1).astype(np.float32)

    A = near_diagonal(((K, I) if conjA else (I, K)) + (xy,))
    B = near_diagonal(((J, K) if conjB else (K, J)) + (xy,))
    rc, got = mm(A, B, conjA, conjB, 1.0)
    assert rc == F.Success
    want = oracle.transpose_mm64(A, B, conjA, conjB, 1.0)
    absA = np.abs(A).sum(-1).astype(np.float64)
    absB = np.abs(B).sum(-1).astype(np.float64)
    a_ik = absA.transpose(1, 0, 2) if conjA else absA            # [I][K][xy]
    b_kj = absB.transpose(1, 0, 2) if conjB else absB            # [K][J][xy]
    scale = np.einsum("ikx,kjx->ijx", a_ik, b_kj)
    eps32 = float(np.finfo(np.float32).eps)
    bound = (K ** 0.5 + 8) * eps32 * scale
    err = np.abs(got.astype(np.float64) - want).max(-1)
    assert (err <= bound).all(), float((err / bound).max())


def test_mm_empty_reduction():
    """K = 0: C = invNorm * (accumulate ? C : 0); the operands have no elements."""
    d = dev()
    A = torch.zeros((4, 0, 40, 2), device=d)
    B = torch.zeros((5, 0, 40, 2), device=d)
    C = torch.full((4, 5, 40, 2), 3.0, device=d)
    assert F.transposeMM(A, B, C, 0.5, False, True, True) == F.Success
    torch.cuda.synchronize()
    assert float((C - 1.5).abs().max()) == 0.0
    assert F.transposeMM(A, B, C, 0.5, False, True, False) == F.Success
    torch.cuda.synchronize()
    assert float(C.abs().max()) == 0.0


def test_mm_rank3_rank4_and_errors():
    d = dev()
    A = torch.zeros((4, 6, 40, 2), device=d)
    B = torch.zeros((5, 6, 40, 2), device=d)
    C = torch.zeros((4, 5, 40, 2), device=d)
    assert F.transposeMM(A, B, C, 1.0, False, True) == F.Success
    assert F.transposeMM(A, B, torch.zeros((4, 6, 40, 2), device=d), 1.0, False, True) == F.UnsupportedDimension
    assert F.transposeMM(A, B, C, 1.0, False, False) == F.UnsupportedDimension  # K mismatch
    assert F.transposeMM(A, B[:, :, ::2], C, 1.0, False, True) == F.UnsupportedDimension  # strided xy
    assert F.transposeMM(A[..., 0], B[..., 0], C[..., 0], 1.0, False, True) == F.UnsupportedDimension
    torch.cuda.synchronize()


def test_mm_config3_shape_subset(oracle):
    """configs[3] contraction shape (128 x 64 x 192 over 544 bins): full GPU run,
    fp64 check on a seeded subset of (i, j) pairs."""
    d = dev()
    I, K, J, xy = 128, 64, 192, 544
    A = synth.normal((I, K, 17, 32, 2), seed=30, device=d)
    B = synth.normal((J, K, 17, 32, 2), seed=31, device=d)
    C = torch.empty((I, J, 17, 32, 2), device=d)
    assert F.transposeMM(A, B, C, 1.0 / 1024, False, True) == F.Success
    torch.cuda.synchronize()
    ii = [0, 5, 31, 32, 77, 127]
    jj = [0, 1, 63, 64, 100, 191]
    want = oracle.transpose_mm64(A[ii].cpu().numpy().reshape(len(ii), K, xy, 2),
                                 B[jj].cpu().numpy().reshape(len(jj), K, xy, 2), False, True, 1.0 / 1024)
    got = C[ii][:, jj].cpu().numpy().reshape(len(ii), len(jj), xy, 2)
    assert rel(got, want) < TOL_FFT


def conv(x, w, N):
    d = dev()
    xd, wd = torch.from_numpy(x).to(d), torch.from_numpy(w).to(d)
    Bn, Cin, H, W = x.shape
    Cout, _, kH, kW = w.shape
    out = torch.full((Bn, Cout, H - kH + 1, W - kW + 1), float("nan"), device=d)
    ws = torch.empty(F.conv_fprop_workspace(Bn, Cin, Cout, N), dtype=torch.uint8, device=d)
    rc = F.conv_fprop(xd, wd, out, N, ws)
    torch.cuda.synchronize()
    return rc, out.cpu().numpy()


@pytest.mark.parametrize("N,H,W,k,Bn,Cin,Cout", [
    (8, 8, 8, 3, 2, 3, 4), (16, 13, 16, 5, 3, 5, 7), (32, 27, 27, 5, 4, 8, 6), (32, 32, 30, 1, 2, 2, 2),
    (64, 60, 57, 5, 3, 5, 4), (64, 64, 64, 11, 1, 3, 6), (128, 100, 128, 7, 2, 3, 2)])
def test_conv_fprop_small(oracle, N, H, W, k, Bn, Cin, Cout):
    x = synth.normal((Bn, Cin, H, W), seed=30).numpy()
    w = synth.normal((Cout, Cin, k, k), seed=31, std=0.02).numpy()
    rc, got = conv(x, w, N)
    assert rc == F.Success
    assert rel(got, oracle.corr2d_valid(x, w)) < TOL_CONV


def test_conv_fprop_config3(oracle):
    """configs[3]: 128x64x27x27 * 192x64x5x5 -> 128x192x23x23; fp64 direct
    correlation on 4096 seeded output pixels plus two whole (n, f) planes."""
    d = dev()
    x = synth.normal((128, 64, 27, 27), seed=30, device=d)
    w = synth.normal((192, 64, 5, 5), seed=31, std=0.02, device=d)
    out = torch.full((128, 192, 23, 23), float("nan"), device=d)
    ws = torch.empty(F.conv_fprop_workspace(128, 64, 192, 32), dtype=torch.uint8, device=d)
    assert F.conv_fprop(x, w, out, 32, ws) == F.Success
    torch.cuda.synchronize()
    assert bool(torch.isfinite(out).all())
    rng = np.random.default_rng(33)
    coords = np.stack([rng.integers(0, 128, 4096), rng.integers(0, 192, 4096),
                       rng.integers(0, 23, 4096), rng.integers(0, 23, 4096)], axis=1).astype(np.int32)
    xh, wh, oh = x.cpu().numpy(), w.cpu().numpy(), out.cpu().numpy()
    want = oracle.corr2d_valid_at(xh, wh, coords)
    got = oh[coords[:, 0], coords[:, 1], coords[:, 2], coords[:, 3]]
    check("configs[3] fbfft_conv_fprop vs fp64 (4096 pixels)", got, want, TOL_CONV)
    full = oracle.corr2d_valid(xh[[0, 127]], wh[[0, 191]])
    assert rel(oh[[0, 127]][:, [0, 191]], full) < TOL_CONV


SHAPES = [(8, 8, 8, 3, 2, 3, 4), (16, 13, 16, 5, 3, 5, 7), (32, 27, 27, 5, 4, 8, 6),
          (32, 32, 30, 1, 2, 2, 2), (32, 20, 31, 7, 5, 150, 9), (16, 16, 16, 3, 70, 3, 140),
          # 64- and 128-point transforms: plane-major spectra through transposeMM
          (64, 60, 57, 5, 3, 5, 4), (64, 64, 64, 11, 1, 3, 6), (128, 100, 128, 7, 2, 3, 2)]


def workspace(pass_, Bn, Cin, Cout, N):
    return torch.empty(F.conv_workspace(pass_, Bn, Cin, Cout, N), dtype=torch.uint8, device=dev())


@pytest.mark.parametrize("N,H,W,k,Bn,Cin,Cout", SHAPES)
def test_conv_bprop(oracle, N, H, W, k, Bn, Cin, Cout):
    """updateGradInput against the fp64 gradient of the direct correlation."""
    go = synth.normal((Bn, Cout, H - k + 1, W - k + 1), seed=32).numpy()
    w = synth.normal((Cout, Cin, k, k), seed=31, std=0.02).numpy()
    d = dev()
    gi = torch.full((Bn, Cin, H, W), float("nan"), device=d)
    rc = F.conv_bprop(torch.from_numpy(go).to(d), torch.from_numpy(w).to(d), gi, N,
                      workspace(1, Bn, Cin, Cout, N))
    torch.cuda.synchronize()
    assert rc == F.Success
    assert rel(gi.cpu().numpy(), oracle.corr2d_grad_input(go, w, H, W)) < TOL_CONV


@pytest.mark.parametrize("accumulate", [False, True])
@pytest.mark.parametrize("N,H,W,k,Bn,Cin,Cout", SHAPES)
def test_conv_accgrad(oracle, N, H, W, k, Bn, Cin, Cout, accumulate):
    """accGradParameters against the fp64 gradient; with accumulate the old
    gradient stays and the new one is added with weight `scale`."""
    x = synth.normal((Bn, Cin, H, W), seed=30).numpy()
    go = synth.normal((Bn, Cout, H - k + 1, W - k + 1), seed=32).numpy()
    d = dev()
    gw0 = synth.normal((Cout, Cin, k, k), seed=34).numpy()
    gw = torch.from_numpy(gw0.copy()).to(d) if accumulate else \
        torch.full((Cout, Cin, k, k), float("nan"), device=d)
    scale = 0.25
    rc = F.conv_accgrad(torch.from_numpy(x).to(d), torch.from_numpy(go).to(d), gw, N,
                        workspace(2, Bn, Cin, Cout, N), scale=scale, accumulate=accumulate)
    torch.cuda.synchronize()
    assert rc == F.Success
    want = scale * oracle.corr2d_grad_weight(x, go, k, k) + (gw0 if accumulate else 0.0)
    assert rel(gw.cpu().numpy(), want) < TOL_CONV


def test_conv_passes_are_adjoint():
    """configs[3] shapes: <conv(x, w), g> = <x, bprop(g, w)> = <w, accgrad(x, g)> ties the three
    passes together at full size without a CPU reference."""
    d = dev()
    x = synth.normal((128, 64, 27, 27), seed=30, device=d)
    w = synth.normal((192, 64, 5, 5), seed=31, std=0.02, device=d)
    g = synth.normal((128, 192, 23, 23), seed=32, device=d)
    out, gi, gw = torch.empty_like(g), torch.empty_like(x), torch.empty_like(w)
    assert F.conv_fprop(x, w, out, 32, workspace(0, 128, 64, 192, 32)) == F.Success
    assert F.conv_bprop(g, w, gi, 32, workspace(1, 128, 64, 192, 32)) == F.Success
    assert F.conv_accgrad(x, g, gw, 32, workspace(2, 128, 64, 192, 32)) == F.Success
    torch.cuda.synchronize()
    a = float((out.double() * g.double()).sum())
    b = float((x.double() * gi.double()).sum())
    c = float((w.double() * gw.double()).sum())
    assert abs(a - b) <= 1e-4 * abs(a) and abs(a - c) <= 1e-4 * abs(a)


def test_conv_pass_argument_checks():
    d = dev()
    x = torch.zeros(2, 3, 16, 16, device=d)
    w = torch.zeros(4, 3, 3, 3, device=d)
    o = torch.zeros(2, 4, 14, 14, device=d)
    ws = workspace(1, 2, 3, 4, 16)
    assert F.conv_bprop(o, w, x, 16, ws) == F.Success
    assert F.conv_bprop(o, w, x, 256, ws) == F.UnsupportedSize
    assert F.conv_bprop(o, w, x, 64, ws[:4096]) == F.UnsupportedDimension   # workspace too small
    assert F.conv_bprop(o[:, :3], w, x, 16, ws) == F.UnsupportedDimension
    assert F.conv_accgrad(x, o, w[:, :, :2], 16, ws) == F.UnsupportedDimension
    assert F.conv_bprop(o, w, x, 16, ws[:16]) == F.UnsupportedDimension
    assert F.conv_workspace(3, 2, 3, 4, 16) == 0


def test_conv_fprop_wide_layer(oracle):
    """128 images x 256 output planes: enough 128-row GEMM tiles per bin (4 x 544) that the
    pipeline keeps the 128 x 64 tile instead of the 64 x 64 one."""
    d = dev()
    x = synth.normal((128, 8, 27, 27), seed=60, device=d)
    w = synth.normal((256, 8, 5, 5), seed=61, std=0.05, device=d)
    out = torch.full((128, 256, 23, 23), float("nan"), device=d)
    assert F.conv_fprop(x, w, out, 32, workspace(0, 128, 8, 256, 32)) == F.Success
    torch.cuda.synchronize()
    assert bool(torch.isfinite(out).all())
    rng = np.random.default_rng(62)
    coords = np.stack([rng.integers(0, 128, 4096), rng.integers(0, 256, 4096),
                       rng.integers(0, 23, 4096), rng.integers(0, 23, 4096)], axis=1).astype(np.int32)
    want = oracle.corr2d_valid_at(x.cpu().numpy(), w.cpu().numpy(), coords)
    oh = out.cpu().numpy()
    assert rel(oh[coords[:, 0], coords[:, 1], coords[:, 2], coords[:, 3]], want) < TOL_CONV
    # whole planes at the corners of the (image, plane) grid
    full = oracle.corr2d_valid(x.cpu().numpy()[[0, 127]], w.cpu().numpy()[[0, 255]])
    assert rel(oh[[0, 127]][:, [0, 255]], full) < TOL_CONV


def test_conv_split_path_strided_operands(oracle):
    """64-point layer on views whose planes do not collapse into one batch (one
    transform launch per image) and an accumulating weight gradient through a view."""
    d = dev()
    Bn, Cin, Cout, H, W, k = 3, 4, 5, 50, 64, 9
    xbig = synth.normal((Bn, Cin + 2, H, W), seed=70, device=d)
    x = xbig[:, 1:1 + Cin]
    w = synth.normal((Cout, Cin, k, k), seed=71, std=0.05, device=d)
    out = torch.full((Bn, Cout, H - k + 1, W - k + 1), float("nan"), device=d)
    assert F.conv_fprop(x, w, out, 64, workspace(0, Bn, Cin, Cout, 64)) == F.Success
    torch.cuda.synchronize()
    xh, wh = x.cpu().numpy().copy(), w.cpu().numpy()
    assert rel(out.cpu().numpy(), oracle.corr2d_valid(xh, wh)) < TOL_CONV
    go = synth.normal(tuple(out.shape), seed=72, device=d)
    gwbig = synth.normal((Cout, Cin, k + 3, k + 1), seed=73, device=d)
    gw0 = gwbig.cpu().numpy().copy()
    gw = gwbig[:, :, 2:2 + k, 1:1 + k]
    assert F.conv_accgrad(x, go, gw, 64, workspace(2, Bn, Cin, Cout, 64), scale=0.5,
                          accumulate=True) == F.Success
    torch.cuda.synchronize()
    want = gw0.copy()
    want[:, :, 2:2 + k, 1:1 + k] += 0.5 * oracle.corr2d_grad_weight(xh, go.cpu().numpy(), k, k)
    assert rel(gwbig.cpu().numpy(), want) < TOL_CONV


@pytest.mark.parametrize("seed", range(24))
def test_mm_random_shapes_and_views(oracle, seed):
    """Seeded random draw over I, J, K, the bin count, the role and accumulation,
    with operands that are views into larger buffers (padded leading strides)."""
    rng = np.random.default_rng(3000 + seed)
    I, J, K = (int(v) for v in rng.integers(1, 140, 3))
    shape = (int(rng.integers(1, 10)), int(rng.integers(1, 20)))
    xy = shape[0] * shape[1]
    conjA, conjB = ROLES[int(rng.integers(0, 3))]
    acc = bool(rng.integers(0, 2))
    d = dev()

    def operand(d0, d1, s):
        full = synth.normal((d0 + 1, d1 + 2) + shape + (2,), seed=s, device=d)
        return full[1:, 1:d1 + 1]                      # leading strides larger than the extents
    A = operand(*((K, I) if conjA else (I, K)), 1 + seed)
    B = operand(*((J, K) if conjB else (K, J)), 2 + seed)
    C = operand(I, J, 3 + seed)
    C0 = C.cpu().numpy().copy()
    assert F.transposeMM(A, B, C, 0.5, conjA, conjB, acc) == F.Success
    torch.cuda.synchronize()
    A3 = A.cpu().numpy().reshape(A.shape[0], A.shape[1], xy, 2)
    B3 = B.cpu().numpy().reshape(B.shape[0], B.shape[1], xy, 2)
    want = oracle.transpose_mm(A3, B3, conjA, conjB, 0.5, C=C0.reshape(I, J, xy, 2) if acc else None)
    assert rel(C.cpu().numpy().reshape(I, J, xy, 2), want) < TOL_FFT, (I, J, K, shape, conjA, conjB, acc)


@pytest.mark.parametrize("seed", range(24))
def test_conv_layer_random_shapes(oracle, seed):
    """All three passes on a seeded random layer (FFT size, image and filter
    extents, plane counts), the input being a channel slice of a larger tensor."""
    rng = np.random.default_rng(4000 + seed)
    N = int(rng.choice([8, 16, 32, 64, 128], p=[0.2, 0.25, 0.3, 0.15, 0.1]))
    H, W = int(rng.integers(max(2, N // 2), N + 1)), int(rng.integers(max(2, N // 2), N + 1))
    kH, kW = int(rng.integers(1, min(H, 9) + 1)), int(rng.integers(1, min(W, 9) + 1))
    Bn, Cin, Cout = int(rng.integers(1, 9)), int(rng.integers(1, 12)), int(rng.integers(1, 12))
    if N >= 64:
        Bn, Cin, Cout = min(Bn, 3), min(Cin, 4), min(Cout, 4)
    d = dev()
    xbig = synth.normal((Bn, Cin + 1, H, W), seed=seed, device=d)
    x = xbig[:, 1:]
    w = synth.normal((Cout, Cin, kH, kW), seed=seed + 100, std=0.1, device=d)
    go = synth.normal((Bn, Cout, H - kH + 1, W - kW + 1), seed=seed + 200, device=d)
    tag = (N, H, W, kH, kW, Bn, Cin, Cout)
    xh, wh, gh = x.cpu().numpy().copy(), w.cpu().numpy(), go.cpu().numpy()

    out = torch.full_like(go, float("nan"))
    assert F.conv_fprop(x, w, out, N, workspace(0, Bn, Cin, Cout, N)) == F.Success
    gi = torch.full((Bn, Cin, H, W), float("nan"), device=d)
    assert F.conv_bprop(go, w, gi, N, workspace(1, Bn, Cin, Cout, N)) == F.Success
    gw = torch.full_like(w, float("nan"))
    assert F.conv_accgrad(x, go, gw, N, workspace(2, Bn, Cin, Cout, N), scale=2.0) == F.Success
    torch.cuda.synchronize()
    assert rel(out.cpu().numpy(), oracle.corr2d_valid(xh, wh)) < TOL_CONV, tag
    assert rel(gi.cpu().numpy(), oracle.corr2d_grad_input(gh, wh, H, W)) < TOL_CONV, tag
    assert rel(gw.cpu().numpy(), 2.0 * oracle.corr2d_grad_weight(xh, gh, kH, kW)) < TOL_CONV, tag


@pytest.mark.parametrize("seed", range(8))
def test_conv_layer_random_shapes_many_planes(oracle, seed):
    """All three passes on seeded random layers whose plane counts (33 .. 72 images and
    output planes, 3 .. 40 input planes) put more than 32 rows on both sides of the
    per-bin contraction: 64-row and 128-row tiles that lie inside the product whole next
    to tiles that hang over its edges, reductions with and without a partial last slice."""
    rng = np.random.default_rng(5000 + seed)
    N = int(rng.choice([8, 16]))
    H, W = int(rng.integers(N // 2, N + 1)), int(rng.integers(N // 2, N + 1))
    kH, kW = int(rng.integers(1, 4)), int(rng.integers(1, 4))
    Bn, Cin, Cout = int(rng.integers(33, 73)), int(rng.integers(3, 41)), int(rng.integers(33, 73))
    d = dev()
    x = synth.normal((Bn, Cin, H, W), seed=seed, device=d)
    w = synth.normal((Cout, Cin, kH, kW), seed=seed + 100, std=0.1, device=d)
    go = synth.normal((Bn, Cout, H - kH + 1, W - kW + 1), seed=seed + 200, device=d)
    tag = (N, H, W, kH, kW, Bn, Cin, Cout)
    xh, wh, gh = x.cpu().numpy(), w.cpu().numpy(), go.cpu().numpy()

    out = torch.full_like(go, float("nan"))
    assert F.conv_fprop(x, w, out, N, workspace(0, Bn, Cin, Cout, N)) == F.Success
    gi = torch.full_like(x, float("nan"))
    assert F.conv_bprop(go, w, gi, N, workspace(1, Bn, Cin, Cout, N)) == F.Success
    gw = torch.full_like(w, float("nan"))
    assert F.conv_accgrad(x, go, gw, N, workspace(2, Bn, Cin, Cout, N)) == F.Success
    torch.cuda.synchronize()
    assert rel(out.cpu().numpy(), oracle.corr2d_valid(xh, wh)) < TOL_CONV, tag
    assert rel(gi.cpu().numpy(), oracle.corr2d_grad_input(gh, wh, H, W)) < TOL_CONV, tag
    assert rel(gw.cpu().numpy(), oracle.corr2d_grad_weight(xh, gh, kH, kW)) < TOL_CONV, tag


@pytest.mark.parametrize("Cin", [5, 8, 12, 24, 40])
def test_conv_fprop_many_full_tiles(oracle, Cin):
    """512 x 512 outputs per bin in 8-point transforms: more 64 x 64 tiles of the contraction
    than workgroups resident at once, so every workgroup walks several tiles; the reduction
    lengths give one, two, three and five k-slices per tile."""
    N, H, k, Bn, Cout = 8, 8, 3, 512, 512
    x = synth.normal((Bn, Cin, H, H), seed=80).numpy()
    w = synth.normal((Cout, Cin, k, k), seed=81, std=0.1).numpy()
    rc, got = conv(x, w, N)
    assert rc == F.Success
    assert rel(got, oracle.corr2d_valid(x, w)) < TOL_CONV


@pytest.mark.parametrize("conjA,conjB", ROLES)
@pytest.mark.parametrize("K", [1, 2, 3, 4, 6, 7, 13])
@pytest.mark.parametrize("shape", [(1, 2), (1, 8), (5, 2), (3, 8), (2, 17)])
def test_mm_aligned_operands_k_tails(oracle, conjA, conjB, K, shape):
    """Even bin counts in contiguous tensors take the kernel that copies slices of four
    k straight into LDS: every remainder of K modulo four, bin counts below, at and
    between multiples of the eight bins of a work item, tiles with clamped rows."""
    I, J = 70, 37
    xy = shape[0] * shape[1]
    A = synth.normal(((K, I) if conjA else (I, K)) + shape + (2,), seed=11 + K).numpy()
    B = synth.normal(((J, K) if conjB else (K, J)) + shape + (2,), seed=12 + K).numpy()
    C0 = synth.normal((I, J) + shape + (2,), seed=13).numpy()
    A3 = A.reshape(A.shape[0], A.shape[1], xy, 2)
    B3 = B.reshape(B.shape[0], B.shape[1], xy, 2)
    for start in (None, C0):
        rc, got = mm(A, B, conjA, conjB, 0.25, C0=start)
        assert rc == F.Success
        want = oracle.transpose_mm(A3, B3, conjA, conjB, 0.25,
                                   C=None if start is None else start.reshape(I, J, xy, 2))
        assert rel(got.reshape(I, J, xy, 2), want) < TOL_FFT
        if start is None:
            assert rel(got.reshape(I, J, xy, 2), oracle.transpose_mm64(A3, B3, conjA, conjB, 0.25)) < TOL_FFT


@pytest.mark.parametrize("I,J,K,shape", [
    (128, 128, 5, (16, 32)),   # 512 work items of 64 x 32: two per CU, the larger tile
    (128, 96, 6, (17, 32)),    # 408 of them: uneven, the smaller tile
])
def test_mm_both_tile_shapes_of_the_aligned_path(oracle, I, J, K, shape):
    """The aligned path picks 64- or 32-row tiles by how evenly the work items spread
    over the CUs; one layer for each choice, both roles with a conjugation."""
    xy = shape[0] * shape[1]
    for conjA, conjB in ROLES[:2]:
        A = synth.normal(((K, I) if conjA else (I, K)) + shape + (2,), seed=21).numpy()
        B = synth.normal(((J, K) if conjB else (K, J)) + shape + (2,), seed=22).numpy()
        rc, got = mm(A, B, conjA, conjB, 0.5)
        assert rc == F.Success
        want = oracle.transpose_mm(A.reshape(A.shape[0], A.shape[1], xy, 2),
                                   B.reshape(B.shape[0], B.shape[1], xy, 2), conjA, conjB, 0.5)
        assert rel(got.reshape(I, J, xy, 2), want) < TOL_FFT


@pytest.mark.parametrize("seed", range(10))
def test_mm_random_aligned_shapes(oracle, seed):
    """Seeded random draw over contiguous operands with an even bin count (the kernel that
    copies slices straight into LDS): I and J from below one tile to several, so that tiles
    inside C whole - stored from a scalar base without tests - meet tiles that hang over its
    last rows, columns or bins; every role, with and without accumulation."""
    rng = np.random.default_rng(6000 + seed)
    I, J, K = int(rng.integers(20, 200)), int(rng.integers(20, 200)), int(rng.integers(1, 80))
    shape = (int(rng.integers(1, 6)), 2 * int(rng.integers(1, 9)))
    xy = shape[0] * shape[1]
    conjA, conjB = ROLES[int(rng.integers(0, 3))]
    acc = bool(rng.integers(0, 2))
    A = synth.normal(((K, I) if conjA else (I, K)) + shape + (2,), seed=21 + seed).numpy()
    B = synth.normal(((J, K) if conjB else (K, J)) + shape + (2,), seed=22 + seed).numpy()
    C0 = synth.normal((I, J) + shape + (2,), seed=23 + seed).numpy()
    rc, got = mm(A, B, conjA, conjB, 0.25, C0=C0 if acc else None)
    assert rc == F.Success
    want = oracle.transpose_mm(A.reshape(A.shape[0], A.shape[1], xy, 2),
                               B.reshape(B.shape[0], B.shape[1], xy, 2), conjA, conjB, 0.25,
                               C=C0.reshape(I, J, xy, 2) if acc else None)
    assert rel(got.reshape(I, J, xy, 2), want) < TOL_FFT, (I, J, K, shape, conjA, conjB, acc)


def test_conv_fprop_batch_beyond_a_16_bit_grid_index(oracle):
    """70000 images with 40 output planes keep the batch on the slow index of the product,
    so the inverse transform's launch counts more than 65535 images: every image is
    reached (whole tensor finite) and seeded pixels, the last images included, match."""
    d = dev()
    B, Cin, Cout, H, k, N = 70000, 2, 40, 8, 3, 8
    x = synth.normal((B, Cin, H, H), seed=60, device=d)
    w = synth.normal((Cout, Cin, k, k), seed=61, std=0.1, device=d)
    out = torch.full((B, Cout, H - k + 1, H - k + 1), float("nan"), device=d)
    assert F.conv_fprop(x, w, out, N, workspace(0, B, Cin, Cout, N)) == F.Success
    torch.cuda.synchronize()
    assert bool(torch.isfinite(out).all())
    rng = np.random.default_rng(62)
    coords = np.stack([rng.integers(0, B, 2048), rng.integers(0, Cout, 2048),
                       rng.integers(0, H - k + 1, 2048), rng.integers(0, H - k + 1, 2048)],
                      axis=1).astype(np.int32)
    coords[:4, 0] = [0, 65535, 65536, B - 1]
    want = oracle.corr2d_valid_at(x.cpu().numpy(), w.cpu().numpy(), coords)
    oh = out.cpu().numpy()
    assert rel(oh[coords[:, 0], coords[:, 1], coords[:, 2], coords[:, 3]], want) < TOL_CONV
