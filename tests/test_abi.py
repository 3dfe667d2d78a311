"""CPU-only checks of the boundary: the shared library loads and exports every
symbol include/fbfft_amd.h declares, the structs have the reference's layout,
and the host-side mirror behaves like the reference's parameter class."""
import ctypes
import os
import re

import numpy as np
import pytest

import fbcuda_amd as F

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    src = open(os.path.join(ROOT, "include", "fbfft_amd.h")).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(fbfft_[a-z0-9_]+)\s*\(", src)))


def test_header_and_python_agree():
    assert declared_symbols() == sorted(F.EXPORTS)


def test_library_exports_every_declared_symbol():
    if not os.path.exists(F.LIB_PATH):
        import __graft_entry__
        __graft_entry__.build()
    L = ctypes.CDLL(F.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(L, name), name


def test_struct_layouts():
    # fbfft_tensor: pointer, 5 strides, 5 sizes, rank
    assert F.Tensor.data.offset == 0 and F.Tensor.stride.offset == 8
    assert F.Tensor.size.offset == 28 and F.Tensor.dim.offset == 48
    # TiledDeviceTensor<float,4>: {int padL; int padU; {float* data; int stride[4]; int size[4];}}
    assert ctypes.sizeof(F.Tile) == 48
    assert (F.Tile.padL.offset, F.Tile.padU.offset, F.Tile.data.offset) == (0, 4, 8)
    assert (F.Tile.stride.offset, F.Tile.size.offset) == (16, 32)


def test_error_strings_and_twiddles():
    assert F.error_string(0) == "Success"
    assert F.error_string(1) == "UnsupportedSize"
    assert F.error_string(2) == "UnsupportedDimension"
    assert F.error_string(3) == "HipError"
    out = (ctypes.c_float * 256)()
    F.lib().fbfft_twiddle_table(out)
    tw = np.frombuffer(out, dtype=np.float32).reshape(128, 2)
    k = np.arange(128)
    assert np.array_equal(tw[:, 1], np.sin(np.pi * k / 128).astype(np.float32))
    assert tw[64, 0] == 0.0 and tw[0, 0] == 1.0


def test_parameters_mirror():
    p = F.FBFFTParameters()
    assert p.forwardFFT() and not p.inverseFFT() and not p.normalizeFFT()
    assert p.padLeft() == 0 and p.padUp() == 0
    q = p.inverse().normalize(True).withPadLeft(3).withPadUp(4)
    assert q is p and p.inverseFFT() and p.normalizeFFT() and (p.padLeft(), p.padUp()) == (3, 4)
    assert p.forward().forwardFFT()
    assert (p.Success, p.UnsupportedSize, p.UnsupportedDimension, p.CudaError) == (0, 1, 2, 3)
    assert [F.numHermitian(n) for n in (2, 8, 32, 256)] == [2, 5, 17, 129]


def test_cpu_tensors_are_rejected():
    import torch
    with pytest.raises(ValueError):
        F.fbfft2D(torch.zeros(1, 8, 8), torch.zeros(1, 5, 8, 2))


def test_synth_is_deterministic():
    from fbcuda_amd import synth
    a = synth.normal((4, 8), seed=3)
    b = synth.normal((4, 8), seed=3)
    assert a.dtype.is_floating_point and bool((a == b).all())
    assert not bool((a == synth.normal((4, 8), seed=4)).all())
    u = synth.uniform((1000,), seed=0)
    assert float(u.min()) >= -1.0 and float(u.max()) < 1.0


def test_cpp_facade_compiles_against_reference_include_paths():
    """Host code that includes cuda/fbfft/FBFFT.cuh, cuda/MM.cuh and
    cuda/fbfft/FFTIteratedConvolution.cuh and uses the reference's names builds and links."""
    import subprocess
    if not os.path.exists(F.LIB_PATH):
        import __graft_entry__
        __graft_entry__.build()
    subprocess.check_call(["make", "-C", os.path.join(ROOT, "tests", "cpp"), "-B"],
                          stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    assert os.path.exists(os.path.join(ROOT, "tests", "cpp", "facade_check"))


def test_cpp_device_tensor_and_complex_host_arithmetic():
    """tests/cpp/tensor_check.cpp: sizes / strides of downcast, upcast, transpose, permute,
    view and cast, and Complex's operators, against hand-written expectations (host only)."""
    import subprocess
    subprocess.check_call(["make", "-C", os.path.join(ROOT, "tests", "cpp"), "-B", "tensor_check"],
                          stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    out = subprocess.run([os.path.join(ROOT, "tests", "cpp", "tensor_check")], capture_output=True,
                         text=True)
    assert out.returncode == 0 and out.stdout.strip() == "OK", out.stdout


def test_cpp_in_register_transforms_on_the_host():
    """tests/cpp/regs_check.cpp: the butterfly and real-fix-up templates the kernels
    instantiate (fbcuda_amd/csrc/fft_regs.h), compiled for the host and compared with a
    naive fp64 DFT for 2 ... 128 complex points, both directions, and 4 ... 128 real points."""
    import subprocess
    subprocess.check_call(["make", "-C", os.path.join(ROOT, "tests", "cpp"), "-B", "regs_check"],
                          stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    out = subprocess.run([os.path.join(ROOT, "tests", "cpp", "regs_check")], capture_output=True,
                         text=True)
    assert out.returncode == 0 and out.stdout.strip() == "OK", out.stdout


def _fake_tensor(shape, base=0x10000000):
    """fbfft_tensor over memory that is never touched: the tile builder only does
    address arithmetic."""
    t = F.Tensor()
    t.data = base
    t.dim = len(shape)
    stride = 1
    for i in reversed(range(len(shape))):
        t.size[i] = shape[i]
        t.stride[i] = stride
        stride *= shape[i]
    return t


@pytest.mark.parametrize("H,W,kH,kW,N", [
    (256, 256, 9, 9, 32),    # configs[4]: 11 x 11 tiles, the last 16 wide in, 8 wide out
    (32, 32, 5, 5, 32), (40, 56, 9, 3, 32), (14, 17, 3, 3, 8), (30, 25, 5, 1, 16), (9, 9, 1, 1, 8)])
def test_make_tiles_grid(H, W, kH, kW, N):
    Bn, Cin, Cout = 3, 2, 5
    oH, oW = H - kH + 1, W - kW + 1
    ti, to = _fake_tensor((Bn, Cin, H, W)), _fake_tensor((Bn, Cout, oH, oW), 0x20000000)
    L = F.lib()
    n = L.fbfft_make_tiles(ti, to, kH, kW, N, None, None, 0)
    sy, sx = N - kH + 1, N - kW + 1
    ys, xs = list(range(0, oH, sy)), list(range(0, oW, sx))
    assert n == len(ys) * len(xs)
    a, b = (F.Tile * n)(), (F.Tile * n)()
    assert L.fbfft_make_tiles(ti, to, kH, kW, N, ctypes.cast(a, ctypes.c_void_p),
                              ctypes.cast(b, ctypes.c_void_p), n) == n
    covered = np.zeros((oH, oW), np.int32)
    for t, (y0, x0) in enumerate((y, x) for y in ys for x in xs):
        assert (a[t].padL, a[t].padU, b[t].padL, b[t].padU) == (0, 0, 0, 0)
        assert a[t].data == 0x10000000 + 4 * (y0 * W + x0)
        assert b[t].data == 0x20000000 + 4 * (y0 * oW + x0)
        assert list(a[t].stride) == [Cin * H * W, H * W, W, 1]
        assert list(b[t].stride) == [Cout * oH * oW, oH * oW, oW, 1]
        assert list(a[t].size) == [Bn, Cin, min(N, H - y0), min(N, W - x0)]
        assert list(b[t].size) == [Bn, Cout, min(sy, oH - y0), min(sx, oW - x0)]
        # the input window holds every sample the output window needs
        assert a[t].size[2] >= b[t].size[2] + kH - 1 and a[t].size[3] >= b[t].size[3] + kW - 1
        covered[y0:y0 + b[t].size[2], x0:x0 + b[t].size[3]] += 1
    assert (covered == 1).all()   # output windows partition the output plane
    if (H, N) == (256, 32):
        assert n == 121 and a[n - 1].size[2] == 16 and b[n - 1].size[2] == 8


def test_make_tiles_capacity_and_rejects():
    ti, to = _fake_tensor((1, 1, 40, 40)), _fake_tensor((1, 1, 36, 36))
    L = F.lib()
    a, b = (F.Tile * 2)(), (F.Tile * 2)()
    pa, pb = ctypes.cast(a, ctypes.c_void_p), ctypes.cast(b, ctypes.c_void_p)
    assert L.fbfft_make_tiles(ti, to, 5, 5, 16, pa, pb, 2) == 9    # 3 x 3 grid, two written
    assert a[1].data == 0x10000000 + 4 * 12
    assert L.fbfft_make_tiles(ti, to, 5, 5, 64, None, None, 0) == 0    # FFT size
    assert L.fbfft_make_tiles(ti, to, 3, 3, 16, None, None, 0) == 0    # output shape mismatch
    assert L.fbfft_make_tiles(ti, to, 5, 17, 16, None, None, 0) == 0   # kernel wider than the FFT
    assert F.lib().fbfft_conv_workspace(0, 128, 64, 192, 32) == \
        F.lib().fbfft_conv_fprop_workspace(128, 64, 192, 32) > 0
    for p in (0, 1, 2):
        assert F.lib().fbfft_conv_workspace(p, 4, 5, 6, 16) % 8 == 0
    # 64 / 128: plane-major half spectra of both operands and the result
    assert F.lib().fbfft_conv_workspace(0, 4, 5, 6, 64) == (20 + 30 + 24) * 33 * 64 * 8
    assert F.lib().fbfft_conv_workspace(2, 4, 5, 6, 128) == (20 + 30 + 24) * 65 * 128 * 8 + 30 * 128 * 128 * 4
    assert F.lib().fbfft_conv_workspace(0, 4, 5, 6, 256) == 0


def _descriptor_views(tiles, base_ptr, strides):
    """(y0, x0, h, w, padL, padU) of each descriptor, recovered from its address."""
    out = []
    for t in tiles:
        off = (t.data - base_ptr) // 4
        assert (t.data - base_ptr) % 4 == 0 and off >= 0
        y0, x0 = off // strides[2], off % strides[2]
        out.append((y0, x0, t.size[2], t.size[3], t.padL, t.padU))
    return out


@pytest.mark.parametrize("N,kH,kW,H,W", [(8, 3, 3, 14, 17), (16, 5, 3, 30, 41), (32, 9, 9, 70, 56),
                                         (8, 1, 1, 9, 9), (16, 16, 16, 16, 16), (8, 3, 2, 8, 6)])
def test_grad_input_tile_grid_partitions_and_reproduces_gradient(oracle, N, kH, kW, H, W):
    """fbfft_make_tiles_for_pass(FFT_UpdateGradInput) is host code: its gradInput windows
    tile the tensor exactly once, and the CPU transcription of the tiled pass run over its
    descriptors gives the fp64 input gradient (multi-tile, seams included)."""
    import torch
    from fbcuda_amd import synth
    Nb, Cin, Cout = 2, 3, 2
    gin = np.full((Nb, Cin, H, W), 7.0, np.float32)
    g = synth.normal((Nb, Cout, H - kH + 1, W - kW + 1), seed=60).numpy()
    w = synth.normal((Cout, Cin, kH, kW), seed=61, std=0.05).numpy()
    vi, vo = F.view(torch.from_numpy(gin)), F.view(torch.from_numpy(g))
    n = F.lib().fbfft_make_tiles_for_pass(1, vi, vo, kH, kW, N, None, None, 0)
    stepY, stepX = N - kH + 1, N - kW + 1
    assert n == -(-H // stepY) * -(-W // stepX)
    a, b = (F.Tile * n)(), (F.Tile * n)()
    assert F.lib().fbfft_make_tiles_for_pass(1, vi, vo, kH, kW, N, ctypes.cast(a, ctypes.c_void_p),
                                             ctypes.cast(b, ctypes.c_void_p), n) == n
    iv = _descriptor_views(a, gin.ctypes.data, [s // 4 for s in gin.strides])
    ov = _descriptor_views(b, g.ctypes.data, [s // 4 for s in g.strides])
    cover = np.zeros((H, W), np.int32)
    for (y0, x0, h, wd, padL, padU), (gy, gx, gh, gw, gpl, gpu) in zip(iv, ov):
        cover[y0:y0 + h, x0:x0 + wd] += 1
        assert (padU, padL) == (kH - 1, kW - 1) and h >= 1 and wd >= 1
        assert gh >= 1 and gw >= 1 and gpu + gh <= N and gpl + gw <= N
        assert gy - gpu == y0 - (kH - 1) and gx - gpl == x0 - (kW - 1)
    assert (cover == 1).all()
    assert oracle.iterated_conv(N, gin, iv, g.copy(), ov, w, 1) == 1
    from oracle import rel_l2
    assert rel_l2(gin, oracle.corr2d_grad_input(g, w, H, W)) < 1e-4
    # passes 0 and 2 share the grid of fbfft_make_tiles
    assert F.lib().fbfft_make_tiles_for_pass(2, vi, vo, kH, kW, N, None, None, 0) == \
        F.lib().fbfft_make_tiles(vi, vo, kH, kW, N, None, None, 0)
    assert F.lib().fbfft_make_tiles_for_pass(3, vi, vo, kH, kW, N, None, None, 0) == 0


def test_view_rejects_strides_beyond_32_bits():
    import torch
    t = torch.empty(4).as_strided((1, 2), (2 ** 31, 1))
    with pytest.raises(ValueError):
        F.view(t)
    assert F.view(torch.empty(4).as_strided((1, 2), (2 ** 31 - 1, 1))).stride[0] == 2 ** 31 - 1


def test_iterated_conv_refuses_filters_larger_than_the_transform():
    """Validated on the host before anything is launched: returns 0 (not launched)."""
    import torch
    w = torch.zeros((1, 1, 9, 3))
    ins, outs = (F.Tile * 1)(), (F.Tile * 1)()
    rc = F.lib().fbfft_iterated_conv(8, ctypes.cast(ins, ctypes.c_void_p),
                                     ctypes.cast(outs, ctypes.c_void_p), F.view(w), 0,
                                     ctypes.c_float(1.0), 1, 1, None)
    assert rc == 0


def test_conv_choose_fft_size():
    """fftSize = 0 of the layer entry points: the choices recorded next to the measurements
    they came from (forward pass / input gradient / weight gradient, us per pass at
    fftSize 8, 16, 32 on one MI355X), and the properties every choice has."""
    L = F.lib()
    measured = [
        # batch, cin, cout, H, k: chosen size per pass
        ((128, 64, 192, 27, 5), (16, 32, 16)),    # configs[3]: 196/92/102, 236/184/99, 226/104/104
        ((16, 32, 32, 256, 9), (32, 32, 32)),     # configs[4]: -/499/285, -/506/283, -/549/310
        ((32, 32, 64, 60, 5), (32, 16, 32)),      # 68/45/36, 81/55/76, 123/76/55
        ((128, 96, 256, 13, 3), (8, 16, 16)),     # 46/50/168, 94/56/181, 58/53/186
        ((128, 256, 256, 13, 3), (8, 16, 16)),    # 87/92/351, 161/92/356, 97/91/365
        ((32, 64, 64, 56, 3), (16, 16, 32)),      # 51/43/50, 60/43/50, 82/60/56
    ]
    for (B, cin, cout, H, k), want in measured:
        got = tuple(L.fbfft_conv_choose_fft_size(p, B, cin, cout, H, H, k, k) for p in range(3))
        assert got == want, ((B, cin, cout, H, k), got)
    for (H, W, kH, kW) in [(27, 27, 5, 5), (8, 8, 3, 3), (12, 40, 3, 5), (16, 16, 1, 1),
                           (100, 7, 7, 7), (33, 33, 17, 2), (9, 9, 9, 9), (500, 300, 32, 32)]:
        for p in range(3):
            N = L.fbfft_conv_choose_fft_size(p, 4, 3, 5, H, W, kH, kW)
            assert N in (8, 16, 32) and N >= max(kH, kW), (p, H, W, kH, kW, N)
            # the workspace of size 0 is the workspace of the chosen size
            assert L.fbfft_conv_workspace_image(p, 4, 3, 5, H, W, kH, kW, 0) == \
                L.fbfft_conv_workspace_image(p, 4, 3, 5, H, W, kH, kW, N) > 0
    # an image that fits one 32-point window is one window for the input gradient too (its
    # 30..32 rows are more than the 28 a window advances by, but there is nothing to advance to)
    for H in (29, 30, 31, 32):
        assert L.fbfft_conv_choose_fft_size(1, 128, 64, 192, H, H, 5, 5) == 32, H
    # no size holds the filter, the filter is larger than the image, bad pass or counts
    assert L.fbfft_conv_choose_fft_size(0, 4, 3, 5, 64, 64, 33, 3) == 0
    assert L.fbfft_conv_choose_fft_size(0, 4, 3, 5, 4, 4, 5, 5) == 0
    assert L.fbfft_conv_choose_fft_size(3, 4, 3, 5, 27, 27, 5, 5) == 0
    assert L.fbfft_conv_choose_fft_size(0, 0, 3, 5, 27, 27, 5, 5) == 0
    assert L.fbfft_conv_workspace_image(0, 4, 3, 5, 64, 64, 33, 3, 0) == 0
