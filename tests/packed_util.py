"""The packed spectrum format of the N <= 32 transforms, restated from its definition
with numpy (independently of the oracle's C++ and of the kernels): a real N x N plane
has real rows 0 and N/2 along the halved (vertical-frequency) axis, so their
horizontal spectra F0 and FH are Hermitian in kx and fit one complex row
P[kx] = F0[kx] + i FH[kx]; rows 1 .. N/2-1 are stored as they are."""
import numpy as np


def pack(U):
    """[..., N/2+1, N] complex -> [..., N/2, N] complex."""
    H = U.shape[-2] - 1
    P = np.array(U[..., :H, :], dtype=np.complex128)
    P[..., 0, :] = U[..., 0, :] + 1j * U[..., H, :]
    return P


def unpack(P):
    """[..., N/2, N] complex -> [..., N/2+1, N] complex; inverse of pack for spectra of
    real planes (and a bijection onto Hermitian row pairs for any P)."""
    H, N = P.shape[-2], P.shape[-1]
    p0 = P[..., 0, :]
    mirror = np.conj(p0[..., (-np.arange(N)) % N])
    U = np.zeros(P.shape[:-2] + (H + 1, N), np.complex128)
    U[..., :H, :] = P
    U[..., 0, :] = 0.5 * (p0 + mirror)
    U[..., H, :] = (p0 - mirror) / 2j
    return U


def as_float(Z):
    return np.stack([Z.real, Z.imag], axis=-1).astype(np.float32)
