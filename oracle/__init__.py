"""ctypes front-end of the CPU oracle (test infrastructure only).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import this
module.  It loads oracle/liboracle.so (built from fbfft_oracle.cpp by
oracle/Makefile) and wraps every exported function with numpy arrays.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None

_f32p = ctypes.POINTER(ctypes.c_float)
_f64p = ctypes.POINTER(ctypes.c_double)
_i32p = ctypes.POINTER(ctypes.c_int)


def build():
    subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"])


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.orc_num_threads.restype = ctypes.c_int
    return _lib


def use_library(path):
    """Load the oracle from another build of fbfft_oracle.cpp (bench.py's cpu_baseline
    compiles one for the machine it runs on)."""
    global _lib
    _lib = ctypes.CDLL(path)
    _lib.orc_num_threads.restype = ctypes.c_int
    return _lib


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _p(a):
    if a.dtype == np.float32:
        return a.ctypes.data_as(_f32p)
    if a.dtype == np.float64:
        return a.ctypes.data_as(_f64p)
    if a.dtype == np.int32:
        return a.ctypes.data_as(_i32p)
    raise TypeError(a.dtype)


def num_threads():
    return lib().orc_num_threads()


def set_num_threads(n):
    lib().orc_set_num_threads(int(n))


def twiddle_table():
    out = np.empty(256, np.float32)
    lib().orc_twiddle_table(_p(out))
    return out.reshape(128, 2)


def fbfft1d(real, padL=0):
    real = _f32(real)
    B, N = real.shape
    out = np.zeros((B, N // 2 + 1, 2), np.float32)
    rc = lib().orc_fbfft1d(_p(real), B, N, padL, _p(out))
    return rc, out


def fbifft1d(cplx, padL=0, out=None):
    cplx = _f32(cplx)
    B, nc, _ = cplx.shape
    N = 2 * (nc - 1)
    if out is None:
        out = np.zeros((B, N), np.float32)
    rc = lib().orc_fbifft1d(_p(cplx), B, N, padL, _p(out))
    return rc, out


def fbfft2d(real, N, padL=0, padU=0):
    real = _f32(real)
    B, h, w = real.shape
    out = np.zeros((B, N // 2 + 1, N, 2), np.float32)
    rc = lib().orc_fbfft2d(_p(real), B, h, w, N, padL, padU, _p(out))
    return rc, out


def fbifft2d(cplx, h, w, padL=0, padU=0, out=None):
    cplx = _f32(cplx)
    B, nc, N, _ = cplx.shape
    if out is None:
        out = np.zeros((B, h, w), np.float32)
    rc = lib().orc_fbifft2d(_p(cplx), B, N, h, w, padL, padU, _p(out))
    return rc, out


def fbfft2d_packed(real, N, padL=0, padU=0):
    """Packed spectrum format [B][N/2][N][2] (Unpack = false, FFT2D32.cuh:421-427)."""
    real = _f32(real)
    B, h, w = real.shape
    out = np.zeros((B, N // 2, N, 2), np.float32)
    rc = lib().orc_fbfft2d_packed(_p(real), B, h, w, N, padL, padU, _p(out))
    return rc, out


def fbifft2d_packed(cplx, h, w, padL=0, padU=0):
    cplx = _f32(cplx)
    B, nr, N, _ = cplx.shape
    assert nr == N // 2
    out = np.zeros((B, h, w), np.float32)
    rc = lib().orc_fbifft2d_packed(_p(cplx), B, N, h, w, padL, padU, _p(out))
    return rc, out


def transpose_mm_packed(A, B, conjA, conjB, invNorm, C=None):
    """A, B packed spectra [..][..][N/2][N][2]; returns C [I][J][N/2][N][2]."""
    A, B = _f32(A), _f32(B)
    N = A.shape[3]
    assert A.shape[2] == N // 2 and B.shape[2:] == A.shape[2:]
    if conjA:
        K, I = A.shape[:2]
    else:
        I, K = A.shape[:2]
    J = B.shape[0] if conjB else B.shape[1]
    accumulate = C is not None
    C = np.zeros((I, J, N // 2, N, 2), np.float32) if C is None else _f32(C).copy()
    lib().orc_transpose_mm_packed(_p(A), _p(B), _p(C), I, J, K, N, int(conjA), int(conjB),
                                  int(accumulate), ctypes.c_float(invNorm))
    return C


def transpose_mm(A, B, conjA, conjB, invNorm, C=None):
    """A, B complex-as-float [..][..][XY][2]; returns C [I][J][XY][2]."""
    A, B = _f32(A), _f32(B)
    XY = A.shape[2]
    if conjA:
        K, I = A.shape[:2]
    else:
        I, K = A.shape[:2]
    J = B.shape[0] if conjB else B.shape[1]
    accumulate = C is not None
    if C is None:
        C = np.zeros((I, J, XY, 2), np.float32)
    else:
        C = _f32(C).copy()
    lib().orc_transpose_mm(_p(A), _p(B), _p(C), I, J, K, XY, int(conjA), int(conjB),
                           int(accumulate), ctypes.c_float(invNorm))
    return C


class TileDesc(ctypes.Structure):
    """TiledDeviceTensor<float,4> (FFTIteratedConvolution.cuh:71-88)."""
    _fields_ = [("padL", ctypes.c_int), ("padU", ctypes.c_int), ("data", ctypes.c_void_p),
                ("stride", ctypes.c_int * 4), ("size", ctypes.c_int * 4)]


assert ctypes.sizeof(TileDesc) == 48


def make_tiles(arr, views):
    """views: list of (y0, x0, h, w, padL, padU) windows into the 4-d float32 array arr."""
    n = len(views)
    descs = (TileDesc * n)()
    st = [s // 4 for s in arr.strides]
    for i, (y0, x0, h, w, padL, padU) in enumerate(views):
        descs[i].padL = padL
        descs[i].padU = padU
        descs[i].data = arr.ctypes.data + 4 * (y0 * st[2] + x0 * st[3])
        descs[i].stride[:] = st
        descs[i].size[:] = [arr.shape[0], arr.shape[1], h, w]
    return descs


def iterated_conv(N, in_arr, in_views, out_arr, out_views, weight, pass_, scale=1.0):
    """Runs the fused tiled convolution in place on host arrays (float32, C-contiguous)."""
    assert in_arr.dtype == np.float32 and out_arr.dtype == np.float32
    assert weight.dtype == np.float32 and weight.flags.c_contiguous
    ins = make_tiles(in_arr, in_views)
    outs = make_tiles(out_arr, out_views)
    wsz = (ctypes.c_int * 4)(*weight.shape)
    wst = (ctypes.c_int * 4)(*[s // 4 for s in weight.strides])
    return lib().orc_iterated_conv(N, ins, outs, _p(weight), wsz, wst, int(pass_),
                                   ctypes.c_float(scale), in_arr.shape[0], len(in_views))


# ------------------------------ double precision ------------------------------

def dft1d_r2c(real):
    real = _f32(real)
    B, N = real.shape
    out = np.zeros((B, N // 2 + 1, 2), np.float64)
    lib().ref64_dft1d_r2c(_p(real), B, N, _p(out))
    return out


def idft1d_c2r(cplx):
    cplx = _f32(cplx)
    B, nc, _ = cplx.shape
    N = 2 * (nc - 1)
    out = np.zeros((B, N), np.float64)
    lib().ref64_idft1d_c2r(_p(cplx), B, N, _p(out))
    return out


def layout_of(N):
    """0: [ky half][kx] (N in 8, 16, 32), 1: [kx half][ky] (N in 2, 4 and N >= 64)."""
    return 0 if 8 <= N <= 32 else 1


def dft2d_r2c(real, N, padL=0, padU=0, layout=None):
    real = _f32(real)
    B, h, w = real.shape
    if layout is None:
        layout = layout_of(N)
    out = np.zeros((B, N // 2 + 1, N, 2), np.float64)
    lib().ref64_dft2d_r2c(_p(real), B, h, w, N, padL, padU, layout, _p(out))
    return out


def corr2d_valid(inp, w):
    inp, w = _f32(inp), _f32(w)
    Nb, Cin, H, W = inp.shape
    Cout, _, kH, kW = w.shape
    out = np.zeros((Nb, Cout, H - kH + 1, W - kW + 1), np.float64)
    lib().ref64_corr2d_valid(_p(inp), _p(w), Nb, Cin, H, W, Cout, kH, kW, _p(out))
    return out


def corr2d_valid_at(inp, w, coords):
    inp, w = _f32(inp), _f32(w)
    _, Cin, H, W = inp.shape
    _, _, kH, kW = w.shape
    coords = np.ascontiguousarray(coords, dtype=np.int32)
    out = np.zeros(len(coords), np.float64)
    lib().ref64_corr2d_valid_at(_p(inp), _p(w), Cin, H, W, kH, kW, _p(coords), len(coords), _p(out))
    return out


def corr2d_grad_input(gout, w, H, W):
    gout, w = _f32(gout), _f32(w)
    Nb, Cout = gout.shape[:2]
    _, Cin, kH, kW = w.shape
    gin = np.zeros((Nb, Cin, H, W), np.float64)
    lib().ref64_corr2d_grad_input(_p(gout), _p(w), Nb, Cin, H, W, Cout, kH, kW, _p(gin))
    return gin


def corr2d_grad_weight(inp, gout, kH, kW):
    inp, gout = _f32(inp), _f32(gout)
    Nb, Cin, H, W = inp.shape
    Cout = gout.shape[1]
    gw = np.zeros((Cout, Cin, kH, kW), np.float64)
    lib().ref64_corr2d_grad_weight(_p(inp), _p(gout), Nb, Cin, H, W, Cout, kH, kW, _p(gw))
    return gw


def corr2d_grad_input_at(gout, w, H, W, coords):
    """fp64 gradInput of the valid correlation at the listed (n, c, y, x)."""
    gout, w = _f32(gout), _f32(w)
    Cout, Cin, kH, kW = w.shape
    coords = np.ascontiguousarray(coords, dtype=np.int32)
    out = np.zeros(len(coords), np.float64)
    lib().ref64_corr2d_grad_input_at(_p(gout), _p(w), Cin, H, W, Cout, kH, kW, _p(coords),
                                     len(coords), _p(out))
    return out


def corr2d_grad_weight_at(inp, gout, kH, kW, coords):
    """fp64 gradWeight of the valid correlation at the listed (f, c, u, v)."""
    inp, gout = _f32(inp), _f32(gout)
    Nb, Cin, H, W = inp.shape
    Cout = gout.shape[1]
    coords = np.ascontiguousarray(coords, dtype=np.int32)
    out = np.zeros(len(coords), np.float64)
    lib().ref64_corr2d_grad_weight_at(_p(inp), _p(gout), Nb, Cin, H, W, Cout, kH, kW, _p(coords),
                                      len(coords), _p(out))
    return out


def transpose_mm64(A, B, conjA, conjB, invNorm):
    A, B = _f32(A), _f32(B)
    XY = A.shape[2]
    if conjA:
        K, I = A.shape[:2]
    else:
        I, K = A.shape[:2]
    J = B.shape[0] if conjB else B.shape[1]
    C = np.zeros((I, J, XY, 2), np.float64)
    lib().ref64_transpose_mm(_p(A), _p(B), _p(C), I, J, K, XY, int(conjA), int(conjB),
                             ctypes.c_double(invNorm))
    return C


def rel_l2(a, b):
    """||a - b||_2 / ||b||_2 over all elements (b is the trusted side)."""
    a = np.asarray(a, dtype=np.float64).ravel()
    b = np.asarray(b, dtype=np.float64).ravel()
    den = np.linalg.norm(b)
    return float(np.linalg.norm(a - b) / den) if den > 0 else float(np.linalg.norm(a - b))
