"""The library's plain copy kernel (the yardstick bench.py times beside the transforms)
copies what it is given and refuses what it cannot move in 16-byte words."""
import ctypes

import pytest
import torch

import fbcuda_amd as F
from gpu_util import dev

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("words", [1, 63, 1024, 1025, 66 * 65536 + 7])
def test_copy_is_exact(words):
    d = dev()
    src = torch.randn(4 * words + 8, device=d)
    dst = torch.full_like(src, 7.0)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = F.lib().fbfft_bench_copy(ctypes.c_void_p(src.data_ptr()), ctypes.c_void_p(dst.data_ptr()),
                                  16 * words, stream)
    torch.cuda.synchronize()
    assert rc == F.Success
    assert torch.equal(dst[:4 * words], src[:4 * words])
    assert bool((dst[4 * words:] == 7.0).all())      # nothing past the end


def test_copy_argument_checks():
    d = dev()
    a, b = torch.zeros(64, device=d), torch.zeros(64, device=d)
    L = F.lib()
    pa, pb = a.data_ptr(), b.data_ptr()
    assert L.fbfft_bench_copy(ctypes.c_void_p(pa), ctypes.c_void_p(pb), 0, None) == F.Success
    assert L.fbfft_bench_copy(ctypes.c_void_p(pa), ctypes.c_void_p(pb), 24, None) == F.UnsupportedDimension
    assert L.fbfft_bench_copy(ctypes.c_void_p(pa + 4), ctypes.c_void_p(pb), 16, None) == F.UnsupportedDimension
    assert L.fbfft_bench_copy(None, ctypes.c_void_p(pb), 16, None) == F.UnsupportedDimension
    torch.cuda.synchronize()
