"""Host-side mirror of fbcuda's fbfft interface on top of the gfx950 C ABI.

The functions keep the reference's names and argument meaning
(fbfft/FBFFT.cuh:11-56, MM.cuh:11-17, fbfft/FFTIteratedConvolution.cuh:624) and
return its FBFFTParameters::ErrorCode values.  Operands are torch tensors that
already live on the GPU; torch is used only to own device memory and to name the
current stream.  Everything is computed by libfbfft_amd.so (hand-written HIP
kernels); there is no CPU or torch fallback, and importing a compute entry point
without the built library raises.
"""
import ctypes
import os

from .params import FBFFTParameters, numHermitian  # noqa: F401

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libfbfft_amd.so")
MAX_DIM = 5

Success = 0
UnsupportedSize = 1
UnsupportedDimension = 2
HipError = 3

FFT_UpdateOutput = 0
FFT_UpdateGradInput = 1
FFT_AccGradParameters = 2


class Tensor(ctypes.Structure):
    """fbfft_tensor of include/fbfft_amd.h."""
    _fields_ = [("data", ctypes.c_void_p), ("stride", ctypes.c_int * MAX_DIM),
                ("size", ctypes.c_int * MAX_DIM), ("dim", ctypes.c_int)]


class Tile(ctypes.Structure):
    """fbfft_tile of include/fbfft_amd.h (TiledDeviceTensor<float, 4>)."""
    _fields_ = [("padL", ctypes.c_int), ("padU", ctypes.c_int), ("data", ctypes.c_void_p),
                ("stride", ctypes.c_int * 4), ("size", ctypes.c_int * 4)]


assert ctypes.sizeof(Tile) == 48

_lib = None

# every symbol include/fbfft_amd.h declares
EXPORTS = (
    "fbfft_r2c_1d", "fbfft_c2r_1d", "fbfft_r2c_2d", "fbfft_c2c_2d_pass2", "fbfft_c2r_2d",
    "fbfft_c2c_2d_inverse_pass1", "fbfft_transpose_mm", "fbfft_transpose_mm_packed", "fbfft_iterated_conv", "fbfft_iterated_conv_ex",
    "fbfft_iterated_conv_workspace", "fbfft_iterated_conv_ws",
    "fbfft_make_tiles",
    "fbfft_make_tiles_for_pass",
    "fbfft_conv_choose_fft_size", "fbfft_conv_workspace", "fbfft_conv_workspace_image", "fbfft_conv_fprop_workspace", "fbfft_conv_fprop", "fbfft_conv_bprop",
    "fbfft_conv_accgrad", "fbfft_conv_fprop_static", "fbfft_bench_copy", "fbfft_error_string",
    "fbfft_twiddle_table",
)


def lib():
    """Loads the HIP library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "%s is missing: build it with `make -C fbcuda_amd/csrc` (or "
                "__graft_entry__.build()); there is no fallback path" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        tp = ctypes.POINTER(Tensor)
        vp = ctypes.c_void_p
        L.fbfft_r2c_1d.argtypes = [tp, tp, ctypes.c_int, vp]
        L.fbfft_c2r_1d.argtypes = [tp, tp, ctypes.c_int, vp]
        L.fbfft_r2c_2d.argtypes = [tp, tp, ctypes.c_int, ctypes.c_int, vp]
        L.fbfft_c2r_2d.argtypes = [tp, tp, ctypes.c_int, ctypes.c_int, vp]
        L.fbfft_c2c_2d_pass2.argtypes = [tp, tp, vp]
        L.fbfft_c2c_2d_inverse_pass1.argtypes = [tp, tp, vp]
        L.fbfft_transpose_mm.argtypes = [tp, tp, tp, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                         ctypes.c_float, vp]
        L.fbfft_transpose_mm_packed.argtypes = L.fbfft_transpose_mm.argtypes
        L.fbfft_iterated_conv.argtypes = [ctypes.c_int, vp, vp, tp, ctypes.c_int, ctypes.c_float,
                                          ctypes.c_int, ctypes.c_size_t, vp]
        L.fbfft_iterated_conv_ex.argtypes = [ctypes.c_int, vp, vp, tp, ctypes.c_int, ctypes.c_float,
                                             ctypes.c_int, ctypes.c_size_t, ctypes.c_uint, vp]
        L.fbfft_iterated_conv_workspace.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                                    ctypes.c_size_t, ctypes.c_int, ctypes.c_int]
        L.fbfft_iterated_conv_workspace.restype = ctypes.c_size_t
        L.fbfft_iterated_conv_ws.argtypes = [ctypes.c_int, vp, vp, tp, ctypes.c_int, ctypes.c_float,
                                             ctypes.c_int, ctypes.c_size_t, vp, ctypes.c_size_t, vp]
        L.fbfft_make_tiles.argtypes = [tp, tp, ctypes.c_int, ctypes.c_int, ctypes.c_int, vp, vp,
                                       ctypes.c_size_t]
        L.fbfft_make_tiles.restype = ctypes.c_size_t
        L.fbfft_make_tiles_for_pass.argtypes = [ctypes.c_int, tp, tp, ctypes.c_int, ctypes.c_int,
                                                ctypes.c_int, vp, vp, ctypes.c_size_t]
        L.fbfft_make_tiles_for_pass.restype = ctypes.c_size_t
        L.fbfft_conv_fprop_workspace.argtypes = [ctypes.c_int] * 4
        L.fbfft_conv_fprop_workspace.restype = ctypes.c_size_t
        L.fbfft_conv_fprop.argtypes = [tp, tp, tp, ctypes.c_int, vp, ctypes.c_size_t, vp]
        L.fbfft_conv_workspace.argtypes = [ctypes.c_int] * 5
        L.fbfft_conv_workspace.restype = ctypes.c_size_t
        L.fbfft_conv_choose_fft_size.argtypes = [ctypes.c_int] * 8
        L.fbfft_conv_workspace_image.argtypes = [ctypes.c_int] * 9
        L.fbfft_conv_workspace_image.restype = ctypes.c_size_t
        L.fbfft_conv_bprop.argtypes = [tp, tp, tp, ctypes.c_int, vp, ctypes.c_size_t, vp]
        L.fbfft_conv_accgrad.argtypes = [tp, tp, tp, ctypes.c_int, ctypes.c_float, ctypes.c_int, vp,
                                         ctypes.c_size_t, vp]
        L.fbfft_conv_fprop_static.argtypes = [tp, tp, tp, ctypes.c_int, vp]
        L.fbfft_bench_copy.argtypes = [vp, vp, ctypes.c_size_t, vp]
        L.fbfft_error_string.argtypes = [ctypes.c_int]
        L.fbfft_error_string.restype = ctypes.c_char_p
        L.fbfft_twiddle_table.argtypes = [ctypes.POINTER(ctypes.c_float)]
        L.fbfft_twiddle_table.restype = None
        _lib = L
    return _lib


def error_string(code):
    return lib().fbfft_error_string(int(code)).decode()


def view(t):
    """fbfft_tensor describing a float32 torch tensor (strides in elements)."""
    import torch
    if t.dtype != torch.float32:
        raise TypeError("fbfft operands are float32 (complex as trailing [2])")
    if t.dim() > MAX_DIM:
        raise ValueError("rank > %d" % MAX_DIM)
    d = Tensor()
    d.data = t.data_ptr()
    d.dim = t.dim()
    for i in range(t.dim()):
        # the descriptor holds 32-bit ints like DeviceTensor (DeviceTensor.cuh:241-245)
        if not (0 <= t.size(i) < 2 ** 31 and -2 ** 31 <= t.stride(i) < 2 ** 31):
            raise ValueError("size or stride of dimension %d does not fit a 32-bit int" % i)
        d.size[i] = t.size(i)
        d.stride[i] = t.stride(i)
    return d


def _stream(stream):
    import torch
    if stream is None:
        return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    if isinstance(stream, int):
        return ctypes.c_void_p(stream)
    return ctypes.c_void_p(stream.cuda_stream)


def _on_gpu(*ts):
    for t in ts:
        if not t.is_cuda:
            raise ValueError("operands must be GPU tensors; this library has no CPU path")


def fbfft1D(real, complex, padL=0, stream=None):
    """fbfft1D<1>: real [B][N] -> complex [B][N/2+1][2] (fbfft/FBFFT.cuh:11-16)."""
    _on_gpu(real, complex)
    return lib().fbfft_r2c_1d(view(real), view(complex), padL, _stream(stream))


def fbifft1D(real, complex, padL=0, stream=None):
    """fbifft1D<1>: complex [B][N/2+1][2] -> real [B][N], gain N (fbfft/FBFFT.cuh:18-23)."""
    _on_gpu(real, complex)
    return lib().fbfft_c2r_1d(view(real), view(complex), padL, _stream(stream))


def fbfft2D(real, complex, padL=0, padU=0, stream=None):
    """fbfft2D<1>(real, complexAsFloat, padL, padU) (fbfft/FBFFT.cuh:30-36)."""
    _on_gpu(real, complex)
    return lib().fbfft_r2c_2d(view(real), view(complex), padL, padU, _stream(stream))


def fbfft2D_pass2(src, dst, stream=None):
    """fbfft2D<1>(Complex src, Complex dst): second pass for N >= 64 (fbfft/FBFFT.cuh:39-43)."""
    _on_gpu(src, dst)
    return lib().fbfft_c2c_2d_pass2(view(src), view(dst), _stream(stream))


def fbifft2D(complex, real, padL=0, padU=0, stream=None):
    """fbifft2D<1>(complexSrc, realDst, padL, padU), gain N*N (fbfft/FBFFT.cuh:50-56)."""
    _on_gpu(real, complex)
    return lib().fbfft_c2r_2d(view(complex), view(real), padL, padU, _stream(stream))


def fbifft2D_pass1(src, dst, stream=None):
    """fbifft2D<1>(float src, float dst): first inverse pass for N >= 64 (fbfft/FBFFT.cuh:45-49)."""
    _on_gpu(src, dst)
    return lib().fbfft_c2c_2d_inverse_pass1(view(src), view(dst), _stream(stream))


def transposeMM(A, B, C, invNorm, conjugateTransposeA=False, conjugateTransposeB=False,
                accumulate=False, stream=None, packed=False):
    """transposeMM<Dim, ConjugateTransposeA, ConjugateTransposeB, Accumulate> (MM.cuh:11-17).

    packed: operands are [d0][d1][N/2][N][2] spectra in the packed format of
    fbfft2D (Unpack = false, fbfft/FFT2D32.cuh:421-427); row 0 is multiplied by the
    unpack / multiply / re-pack rule of fbfft/FFTIteratedConvolution.cuh:161-186."""
    _on_gpu(A, B, C)
    fn = lib().fbfft_transpose_mm_packed if packed else lib().fbfft_transpose_mm
    return fn(view(A), view(B), view(C), int(conjugateTransposeA), int(conjugateTransposeB),
              int(accumulate), float(invNorm), _stream(stream))


def make_tiles(t, windows):
    """Device array of tile descriptors over the 4-d GPU tensor t.

    windows: iterable of (y0, x0, h, w, padL, padU).  Returns (device uint8 tensor
    holding the descriptors, count); the tensor must outlive the launch.  This is
    the work the reference leaves to its external caller
    (fbfft/FFTIteratedConvolution.cuh:71-88, :113-114).
    """
    import torch
    windows = list(windows)
    arr = (Tile * len(windows))()
    st = [t.stride(i) for i in range(4)]
    for i, (y0, x0, h, w, padL, padU) in enumerate(windows):
        arr[i].padL, arr[i].padU = padL, padU
        arr[i].data = t.data_ptr() + 4 * (y0 * st[2] + x0 * st[3])
        arr[i].stride[:] = st
        arr[i].size[:] = [t.size(0), t.size(1), h, w]
    host = torch.frombuffer(bytearray(bytes(arr)), dtype=torch.uint8)
    return host.to(t.device), len(windows)


def make_tile_grid(input, output, kH, kW, fftSize, pass_=FFT_UpdateOutput):
    """The tiling of a whole layer for one pass (fbfft_make_tiles_for_pass): device
    descriptor arrays (ins, outs) for `input` [B][Cin][H][W] and `output`
    [B][Cout][H-kH+1][W-kW+1], and the tile count.  FFT_UpdateGradInput has its own
    grid (disjoint gradInput windows); the other two passes share one.  Raises on
    unsupported arguments."""
    import torch
    vi, vo = view(input), view(output)
    n = lib().fbfft_make_tiles_for_pass(int(pass_), vi, vo, kH, kW, fftSize, None, None, 0)
    if n == 0:
        raise ValueError("fbfft_make_tiles_for_pass: unsupported arguments")
    a, b = (Tile * n)(), (Tile * n)()
    got = lib().fbfft_make_tiles_for_pass(int(pass_), vi, vo, kH, kW, fftSize,
                                          ctypes.cast(a, ctypes.c_void_p),
                                          ctypes.cast(b, ctypes.c_void_p), n)
    assert got == n
    up = lambda arr: torch.frombuffer(bytearray(bytes(arr)), dtype=torch.uint8).to(input.device)
    return up(a), up(b), n


DETERMINISTIC = 1


def FFTIteratedConvolution(fftSize, ins, outs, weight, pass_, scale, batchSize, numTiles,
                           stream=None, deterministic=False):
    """detail::FFTIteratedConvolution<fftSize> (fbfft/FFTIteratedConvolution.cuh:624-755).

    ins / outs: device uint8 tensors from make_tiles.  Returns True if launched.
    deterministic: FFT_AccGradParameters reduces in the reference's fixed order (one
    workgroup per plane group, no atomic adds): reproducible bit for bit, much slower.
    """
    _on_gpu(ins, outs, weight)
    rc = lib().fbfft_iterated_conv_ex(fftSize, ctypes.c_void_p(ins.data_ptr()),
                                      ctypes.c_void_p(outs.data_ptr()), view(weight), int(pass_),
                                      float(scale), int(batchSize), int(numTiles),
                                      DETERMINISTIC if deterministic else 0, _stream(stream))
    if rc < 0:
        raise RuntimeError("fbfft_iterated_conv: %s" % error_string(-rc))
    return rc == 1


def iterated_conv_workspace(fftSize, pass_, batchSize, numTiles, cin, cout):
    """Workspace bytes of FFTIteratedConvolution(..., workspace=...) for that pass."""
    return lib().fbfft_iterated_conv_workspace(fftSize, int(pass_), int(batchSize), int(numTiles),
                                               cin, cout)


def FFTIteratedConvolutionWS(fftSize, ins, outs, weight, pass_, scale, batchSize, numTiles,
                             workspace, stream=None):
    """FFTIteratedConvolution on the same tile descriptors through a caller-owned workspace
    (fbfft_iterated_conv_ws): the three kernels of the layer entry points instead of the
    fused kernel.  Returns True if launched."""
    _on_gpu(ins, outs, weight, workspace)
    rc = lib().fbfft_iterated_conv_ws(fftSize, ctypes.c_void_p(ins.data_ptr()),
                                      ctypes.c_void_p(outs.data_ptr()), view(weight), int(pass_),
                                      float(scale), int(batchSize), int(numTiles),
                                      ctypes.c_void_p(workspace.data_ptr()),
                                      workspace.numel() * workspace.element_size(), _stream(stream))
    if rc < 0:
        raise RuntimeError("fbfft_iterated_conv_ws: %s" % error_string(-rc))
    return rc == 1


def conv_fprop_workspace(batch, cin, cout, fftSize):
    return lib().fbfft_conv_fprop_workspace(batch, cin, cout, fftSize)


def conv_fprop(input, weight, output, fftSize, workspace, stream=None):
    """FFT -> per-frequency contraction -> IFFT forward convolution (valid cross-correlation)."""
    _on_gpu(input, weight, output, workspace)
    return lib().fbfft_conv_fprop(view(input), view(weight), view(output), fftSize,
                                  ctypes.c_void_p(workspace.data_ptr()),
                                  workspace.numel() * workspace.element_size(), _stream(stream))


STATIC_SCRATCH_BYTES = 32 << 20


def conv_fprop_static(input, weight, output, fftSize, stream=None):
    """conv_fprop through the library's own fixed scratch array (fbfft_conv_fprop_static):
    no workspace argument, no allocation; layers needing more than STATIC_SCRATCH_BYTES of
    workspace return UnsupportedSize."""
    _on_gpu(input, weight, output)
    return lib().fbfft_conv_fprop_static(view(input), view(weight), view(output), fftSize,
                                         _stream(stream))


def conv_workspace(pass_, batch, cin, cout, fftSize):
    """Workspace bytes of pass 0 (conv_fprop), 1 (conv_bprop) or 2 (conv_accgrad)."""
    return lib().fbfft_conv_workspace(int(pass_), batch, cin, cout, fftSize)


def conv_choose_fft_size(pass_, batch, cin, cout, H, W, kH, kW):
    """The transform size that fftSize = 0 stands for in the conv_* call of that pass
    (8, 16 or 32; 0 if no size fits the filter)."""
    return lib().fbfft_conv_choose_fft_size(int(pass_), batch, cin, cout, H, W, kH, kW)


def conv_workspace_image(pass_, batch, cin, cout, H, W, kH, kW, fftSize):
    """Workspace bytes of a pass for input extents H x W (images larger than the transform
    are overlap-tiled when fftSize <= 32; fftSize 0: the library's choice)."""
    return lib().fbfft_conv_workspace_image(int(pass_), batch, cin, cout, H, W, kH, kW, fftSize)


def conv_bprop(gradOutput, weight, gradInput, fftSize, workspace, stream=None):
    """updateGradInput: gradInput[b][c] = sum_f fullconv(gradOutput[b][f], weight[f][c])."""
    _on_gpu(gradOutput, weight, gradInput, workspace)
    return lib().fbfft_conv_bprop(view(gradOutput), view(weight), view(gradInput), fftSize,
                                  ctypes.c_void_p(workspace.data_ptr()),
                                  workspace.numel() * workspace.element_size(), _stream(stream))


def conv_accgrad(input, gradOutput, gradWeight, fftSize, workspace, scale=1.0, accumulate=False,
                 stream=None):
    """accGradParameters: gradWeight[f][c] (+)= scale * sum_b corr(input[b][c], gradOutput[b][f])."""
    _on_gpu(input, gradOutput, gradWeight, workspace)
    return lib().fbfft_conv_accgrad(view(input), view(gradOutput), view(gradWeight), fftSize,
                                    ctypes.c_float(scale), int(bool(accumulate)),
                                    ctypes.c_void_p(workspace.data_ptr()),
                                    workspace.numel() * workspace.element_size(), _stream(stream))
