"""Shared helpers of the GPU parity tests: they call the product through its C ABI
(fbcuda_amd -> libfbfft_amd.so) and check it against the CPU oracle."""
import numpy as np
import torch

import fbcuda_amd as F

TOL_FFT = 1e-5    # rel-L2 per transform (vs the fp32 transcription and vs the fp64 DFT)
TOL_CONV = 1e-4   # rel-L2 per full convolution


def dev():
    return torch.device("cuda:0")


def c(a):
    a = np.asarray(a)
    return a[..., 0] + 1j * a[..., 1]


def rel(a, b):
    a, b = np.asarray(a), np.asarray(b)
    wide = np.complex128 if (np.iscomplexobj(a) or np.iscomplexobj(b)) else np.float64
    a, b = a.astype(wide).ravel(), b.astype(wide).ravel()
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-300))


def check(label, got, want, tol):
    """Asserts rel-L2(got, want) < tol and prints the observed figure (`pytest -s` shows it:
    the parity numbers quoted in the documents come from these lines)."""
    e = rel(got, want)
    print("parity %-58s rel-L2 %.2e (bar %.0e)" % (label, e, tol))
    assert e < tol, "%s: rel-L2 %.3e >= %.0e" % (label, e, tol)
    return e


def fft2d(x, N, padL=0, padU=0):
    """numpy real [B][h][w] -> numpy [B][N/2+1][N][2] through the C ABI."""
    xd = torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to(dev())
    out = torch.full((x.shape[0], N // 2 + 1, N, 2), float("nan"), device=dev())
    rc = F.fbfft2D(xd, out, padL, padU)
    torch.cuda.synchronize()
    return rc, out.cpu().numpy()


def ifft2d(spec, h, w, padL=0, padU=0, fill=float("nan")):
    sd = torch.from_numpy(np.ascontiguousarray(spec, dtype=np.float32)).to(dev())
    out = torch.full((spec.shape[0], h, w), fill, device=dev())
    rc = F.fbifft2D(sd, out, padL, padU)
    torch.cuda.synchronize()
    return rc, out.cpu().numpy()
