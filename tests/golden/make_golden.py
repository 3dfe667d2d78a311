#!/usr/bin/env python3
"""Writes tests/golden/fft_vectors.npz: small seeded inputs and their transforms
as computed by numpy.fft (a third-party library, not the reference; the
reference holds no vectors for this path) in float64, stored in the reference's
output layouts:

  1D            cplx[b][k]          k  = 0..N/2
  2D, N = 8, 16, 32      cplx[b][ky][kx]     ky = 0..N/2   (fft2(X)[:N/2+1, :])
  2D, N = 2, 4, 64, 128  cplx[b][kx][ky]     kx = 0..N/2   (rfft2(X) transposed)

Run from the repository root:  python tests/golden/make_golden.py
"""
import os

import numpy as np

out = {}
rng = np.random.default_rng(20240607)
for N in (8, 32, 256):
    x = rng.uniform(-1, 1, (3, N)).astype(np.float32)
    out["x1d_%d" % N] = x
    out["f1d_%d" % N] = np.fft.rfft(x.astype(np.float64), axis=1)
for N, h, w, padL, padU in ((8, 8, 8, 0, 0), (16, 11, 9, 2, 3), (32, 27, 27, 0, 0),
                            (32, 5, 5, 0, 0), (64, 64, 64, 0, 0), (128, 100, 90, 5, 7),
                            (4, 4, 4, 0, 0), (4, 3, 3, 1, 0), (2, 2, 2, 0, 0)):
    nb = 2 if N <= 32 else 1
    x = rng.standard_normal((nb, h, w)).astype(np.float32)
    X = np.zeros((nb, N, N))
    X[:, padU:padU + h, padL:padL + w] = x
    F = np.fft.fft2(X)
    if N >= 64 or N < 8:
        F = np.transpose(F, (0, 2, 1))
    key = "%d_%d_%d_%d_%d" % (N, h, w, padL, padU)
    out["x2d_" + key] = x
    out["f2d_" + key] = F[:, :N // 2 + 1, :]
np.savez_compressed(os.path.join(os.path.dirname(os.path.abspath(__file__)), "fft_vectors.npz"), **out)
print("wrote", len(out), "arrays")
