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
