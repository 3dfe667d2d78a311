"""The library keeps no mutable state and enqueues only on the caller's stream:
calls issued from several host threads on several streams at once give the same
results as the same calls made one after the other."""
import threading

import pytest
import torch

import fbcuda_amd as F
from fbcuda_amd import synth
from gpu_util import dev

pytestmark = pytest.mark.gpu


def work(seed, stream, out):
    d = dev()
    with torch.cuda.stream(stream):
        planes = synth.normal((700, 32, 32), seed=seed, device=d)
        rows = synth.uniform((5000, 128), seed=seed + 1, device=d)
        x = synth.normal((6, 5, 27, 27), seed=seed + 2, device=d)
        w = synth.normal((7, 5, 5, 5), seed=seed + 3, std=0.05, device=d)
        spec = torch.empty((700, 17, 32, 2), device=d)
        spec1 = torch.empty((5000, 65, 2), device=d)
        y = torch.empty((6, 7, 23, 23), device=d)
        ws = torch.empty(F.conv_workspace(0, 6, 5, 7, 32), dtype=torch.uint8, device=d)
        for _ in range(20):
            assert F.fbfft2D(planes, spec, stream=stream) == F.Success
            assert F.fbfft1D(rows, spec1, stream=stream) == F.Success
            assert F.conv_fprop(x, w, y, 32, ws, stream=stream) == F.Success
        stream.synchronize()
        out[seed] = [t.cpu() for t in (spec, spec1, y)]


def test_concurrent_streams_and_threads():
    seeds = [100, 200, 300, 400]
    serial, parallel = {}, {}
    for s in seeds:
        work(s, torch.cuda.Stream(), serial)
    threads = [threading.Thread(target=work, args=(s, torch.cuda.Stream(), parallel)) for s in seeds]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    for s in seeds:
        assert s in parallel
        for a, b in zip(serial[s], parallel[s]):
            assert torch.equal(a, b)
