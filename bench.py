#!/usr/bin/env python3
"""Benchmark of the fbfft hot path on one MI355X.

A step is one fbfft2D real-to-complex pass over the whole batch of
BASELINE.json configs[1] (16384 planes of 32x32 fp32, N(0,1)), inputs resident
in HBM - and served from HBM: consecutive steps run on eight different sets of
operand buffers (1.1 GB in all), because one set (132 MB) would sit in the 256 MiB
last-level cache from one launch to the next.  Prints ONE JSON line:

  value / unit   algorithmic GB/s of the timed region (8448 bytes per plane:
                 4096 read + 4352 written), the metric BASELINE.json names
  roofline       the R2C kernel against the 8 TB/s HBM peak, duration from HIP
                 events recorded on the launch stream around the timed region
  roofline_llc   the same launch on the same buffers every time (operands in
                 the last-level cache), roofline_4x one launch over a 4x batch,
                 copy_ceiling plain copies of the same bytes under the same
                 rotation of buffers
  cpu_baseline   the CPU oracle (host transcription of the reference's
                 algorithm, OpenMP over planes) on the same workload, timed on
                 this machine's cores for a bounded number of passes
  extra          other measured configurations (C2R, other sizes, the FFT
                 convolution of configs[3] with its own CPU baseline) -
                 informative, not the metric
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0


def plane_bytes(N):
    return 4 * N * N + 8 * N * (N // 2 + 1)


def timed(fn, steps, warmup, torch):
    """(seconds per step by host clock with sync on both sides, seconds per launch by HIP events)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    return (t1 - t0) / steps, e0.elapsed_time(e1) * 1e-3 / steps


def spread(fn, steps, torch, chunks=20):
    """Median and minimum seconds per launch over `chunks` consecutive groups of at least
    five launches, each group bracketed by its own pair of HIP events (a separate pass
    after the timed region, so that the extra events do not sit inside it; an event
    around every single launch would add 2-3 us to a 22 us kernel)."""
    n = chunks
    per = max(5, steps // n)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(n + 1)]
    ev[0].record()
    for c in range(n):
        for _ in range(per):
            fn()
        ev[c + 1].record()
    torch.cuda.synchronize()
    ts = sorted(ev[c].elapsed_time(ev[c + 1]) * 1e-3 / per for c in range(n))
    mid = ts[n // 2] if n % 2 else 0.5 * (ts[n // 2 - 1] + ts[n // 2])
    return mid, ts[0]


def prepared(fn_name, F, *tensors_then_ints):
    """Bind a C-ABI call once: descriptors are built outside the timed region."""
    import torch
    L = F.lib()
    cfn = getattr(L, fn_name)
    args = []
    keep = []
    for a in tensors_then_ints:
        if isinstance(a, torch.Tensor):
            v = F.view(a)
            keep.append(v)
            args.append(ctypes.byref(v))
        else:
            args.append(a)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    args.append(stream)

    def call():
        rc = cfn(*args)
        if rc != 0:
            raise RuntimeError("%s failed: %s" % (fn_name, F.error_string(rc)))
    call.keep = keep
    return call


NATIVE_FLAGS = ["-O3", "-march=native", "-std=c++17", "-fPIC", "-fopenmp", "-ffp-contract=off",
                "-fno-fast-math"]


def native_oracle():
    """The CPU oracle compiled for THIS machine's cores (-O3 -march=native, contraction
    off) into a temporary directory; the in-tree library is built on another machine with
    a portable -march and is what is used when no compiler is at hand.  Returns
    (module, flags string)."""
    import shutil
    import subprocess
    import tempfile

    import oracle as O
    cxx = shutil.which("g++")
    src = os.path.join(ROOT, "oracle", "fbfft_oracle.cpp")
    if cxx and os.path.exists(src):
        out = os.path.join(tempfile.mkdtemp(prefix="fbfft_oracle_"), "liboracle_native.so")
        try:
            subprocess.check_call([cxx] + NATIVE_FLAGS + ["-shared", "-o", out, src],
                                  stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL, timeout=120)
            O.use_library(out)
            return O, " ".join(NATIVE_FLAGS[:2]) + " -ffp-contract=off, built on this machine"
        except (subprocess.SubprocessError, OSError):
            pass
    O.lib()
    return O, "in-tree build (oracle/Makefile flags)"


def cpu_baseline(x_host, N, budget_s=12.0):
    """Times the CPU oracle (kind "port") on the same planes; bounded to ~budget_s."""
    O, flags = native_oracle()
    threads = O.num_threads()
    O.fbfft2d(x_host[:64], N)  # warm
    t0 = time.perf_counter()
    O.fbfft2d(x_host, N)
    one = time.perf_counter() - t0
    reps = max(1, min(5000, int(budget_s / max(one, 1e-4))))
    t0 = time.perf_counter()
    for _ in range(reps):
        O.fbfft2d(x_host, N)
    dt = (time.perf_counter() - t0) / reps
    gbs = x_host.shape[0] * plane_bytes(N) / dt / 1e9
    # one thread, a few passes, for scale
    O.set_num_threads(1)
    t0 = time.perf_counter()
    for _ in range(3):
        O.fbfft2d(x_host, N)
    dt1 = (time.perf_counter() - t0) / 3
    O.set_num_threads(threads)
    return {"value": round(gbs, 3), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": "%d passes of the full %d-plane %dx%d R2C batch, OpenMP over planes, "
                      "%.3f s per pass" % (reps, x_host.shape[0], N, N, dt),
            "flags": flags,
            "single_thread_GBps": round(x_host.shape[0] * plane_bytes(N) / dt1 / 1e9, 3)}


def conv_cpu_baseline(budget_s=12.0):
    """The reference's composition for configs[3] on the CPU oracle (kind "port"): fbfft2D of
    the images and of the filters (FBFFT2D-inl.cuh:450-623), transposeMM with the filters
    conjugate-transposed (MM-inl.cuh:515-814), fbifft2D with crop (FBIFFT2D-inl.cuh:567-742),
    OpenMP over planes / (image, output plane) pairs.  Timed on a slice of the batch sized to
    the budget; the filter transforms are charged once, the rest scales with the images."""
    import numpy as np

    from fbcuda_amd import synth
    O, flags = native_oracle()
    threads = O.num_threads()
    cin, cout, N = 64, 192, 32
    w = synth.normal((cout, cin, 5, 5), seed=31, std=0.02).numpy()

    def run(x):
        nb = x.shape[0]
        t0 = time.perf_counter()
        _, W = O.fbfft2d(w.reshape(-1, 5, 5), N)
        t1 = time.perf_counter()
        _, X = O.fbfft2d(x.reshape(-1, 27, 27), N)
        C = O.transpose_mm(X.reshape(nb, cin, -1, 2), W.reshape(cout, cin, -1, 2), False, True,
                           1.0 / (N * N))
        _, out = O.fbifft2d(C.reshape(nb * cout, N // 2 + 1, N, 2), 23, 23)
        t2 = time.perf_counter()
        return t1 - t0, t2 - t1, out

    x = synth.normal((128, cin, 27, 27), seed=30).numpy()
    run(x[:1])                                    # warm
    tw, tx, _ = run(x[:2])
    nb = int(max(2, min(128, budget_s / max(tx / 2, 1e-4))))
    tw, tx, out = run(x[:nb])
    reps = 1
    if nb == 128:   # the whole layer fits the budget several times over: average a few passes
        reps = int(max(1, min(500, budget_s / max(tw + tx, 1e-3))))
        acc = [run(x)[:2] for _ in range(reps)]
        tw, tx = sum(a[0] for a in acc) / reps, sum(a[1] for a in acc) / reps
    # sanity: one output pixel against its definition
    ref = float(np.sum(x[0].astype(np.float64) [:, 3:8, 4:9] * w[5].astype(np.float64)))
    got = float(out.reshape(nb, cout, 23, 23)[0, 5, 3, 4])
    ms = (tw + tx * 128.0 / nb) * 1e3
    # one thread, a slice of the batch, for scale
    O.set_num_threads(1)
    n1 = max(1, min(nb, 8))
    tw1, tx1, _ = run(x[:n1])
    O.set_num_threads(threads)
    ms1 = (tw1 + tx1 * 128.0 / n1) * 1e3
    return {"value": round(ms, 1), "unit": "ms/iter", "cores": threads, "kind": "port",
            "single_thread_ms_per_iter": round(ms1, 1),
            "sample": "%d pass(es) over %d of the 128 images of configs[3] with all 192x64 filters "
                      "(%.2f s for the image-dependent part, %.3f s for the filter transforms per "
                      "pass), scaled to 128 images" % (reps, nb, tx, tw),
            "flags": flags, "check_abs_err": abs(got - ref)}


CSRC = os.path.join(ROOT, "fbcuda_amd", "csrc")
# the kernel sources each committed counter summary was measured on
PROFILE_SOURCES = {
    "fft2dSmallForward32_configs1.md": ("fft2d_small.hip", "fft2d_core.h", "fft_regs.h", "common.h"),
    "conv_pipeline_configs3.md": ("conv_pipeline.hip", "fft2d_core.h", "fft_regs.h", "common.h"),
    "conv_pipeline_configs4.md": ("conv_pipeline.hip", "fft2d_core.h", "fft_regs.h", "common.h"),
}


def source_sha16(files):
    """First 16 hex digits of the SHA-256 over the named kernel sources, in order."""
    import hashlib
    h = hashlib.sha256()
    for f in files:
        with open(os.path.join(CSRC, f), "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]


def profile_traffic(name, key):
    """(HBM bytes, where the figure comes from) read from a committed rocprofv3 counter
    summary under profiles/.  The summary records the hash of the kernel sources it was
    measured on (`kernel_source_sha16: ...`); when the sources have changed since, the
    figure is withheld: (None, reason)."""
    value = recorded = None
    try:
        for line in open(os.path.join(ROOT, "profiles", name)):
            if line.startswith(key + ":"):
                value = int(line.split(":")[1])
            elif line.startswith("kernel_source_sha16:"):
                recorded = line.split(":")[1].split()[0]
    except (OSError, ValueError, IndexError):
        return None, "profiles/%s unreadable" % name
    try:
        current = source_sha16(PROFILE_SOURCES[name])
    except OSError:
        current = None
    if value is None:
        return None, "profiles/%s holds no %s" % (name, key)
    if recorded is None or recorded != current:
        return None, "profiles/%s was measured on other kernel sources (%s, now %s)" % (
            name, recorded, current)
    return value, "profiles/%s, rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE on sources %s" % (
        name, recorded)


MFMA_FP32_PEAK = 157.3e12
CONV3_FLOP = 544 * 128 * 192 * 64 * 8.0          # 8 flop per complex multiply-add
CONV3_FLOP_ISSUED = 544 * 128 * 192 * 64 * 6.0   # three real products per complex product


def conv_extras(F, synth, torch, dev, extra):
    """configs[3] FFT convolution forward (ms/iter) and its contraction; configs[4] tiled conv."""
    x = synth.normal((128, 64, 27, 27), seed=30, device=dev)
    w = synth.normal((192, 64, 5, 5), seed=31, std=0.02, device=dev)
    out = torch.empty((128, 192, 23, 23), device=dev)
    ws = torch.empty(F.conv_fprop_workspace(128, 64, 192, 32), dtype=torch.uint8, device=dev)
    L = F.lib()
    vx, vw, vo = F.view(x), F.view(w), F.view(out)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    wsp, wsb = ctypes.c_void_p(ws.data_ptr()), ws.numel()

    def conv():
        rc = L.fbfft_conv_fprop(ctypes.byref(vx), ctypes.byref(vw), ctypes.byref(vo), 32, wsp, wsb,
                                stream)
        if rc != 0:
            raise RuntimeError(F.error_string(rc))
    _, t = timed(conv, 200, 200, torch)
    mid, low = spread(conv, 200, torch)
    extra["fft_conv_configs3_ms_per_iter"] = round(t * 1e3, 4)
    extra["fft_conv_configs3_ms_per_iter_median"] = round(mid * 1e3, 4)
    extra["fft_conv_configs3_ms_per_iter_min"] = round(low * 1e3, 4)
    extra["fft_conv_configs3_direct_equiv_TFLOPs"] = round(41.6e9 / t / 1e12, 1)
    extra["fft_conv_configs3_fp32_peak_direct_ms"] = round(41.6e9 / 157.3e12 * 1e3, 4)
    # the second half of the metric against its roofline: the whole iteration (forward
    # transforms, contraction, inverse transform) is charged to the contraction's matrix
    # work, 8 flop per complex multiply-add; frac_issued counts the 6 flop the kernels issue
    tr3, tr3_src = profile_traffic("conv_pipeline_configs3.md", "traffic_bytes_per_iteration")
    extra["fft_conv_roofline"] = {
        "bound": "mfma", "achieved": round(CONV3_FLOP / t / 1e12, 2), "peak": MFMA_FP32_PEAK / 1e12,
        "unit": "TFLOP/s", "frac": round(CONV3_FLOP / t / MFMA_FP32_PEAK, 4),
        "frac_issued": round(CONV3_FLOP_ISSUED / t / MFMA_FP32_PEAK, 4),
        "floor_us": round(CONV3_FLOP / MFMA_FP32_PEAK * 1e6, 1), "iter_us": round(t * 1e6, 1),
        "traffic": tr3, "traffic_source": tr3_src,
        "algorithmic_bytes": 77119488,
        "workload": "configs[3]: 128x64x27x27 * 192x64x5x5 -> 128x192x23x23, 32-point FFTs"}
    # the same pass with the transform size left to the library (fftSize 0): configs[3]
    # names 32-point transforms, so this is an extra, not the metric
    auto = L.fbfft_conv_choose_fft_size(0, 128, 64, 192, 27, 27, 5, 5)
    wsa = torch.empty(F.conv_workspace_image(0, 128, 64, 192, 27, 27, 5, 5, 0), dtype=torch.uint8,
                      device=dev)
    wspa, wsba = ctypes.c_void_p(wsa.data_ptr()), wsa.numel()

    def conv_auto():
        if L.fbfft_conv_fprop(ctypes.byref(vx), ctypes.byref(vw), ctypes.byref(vo), 0, wspa, wsba,
                              stream) != 0:
            raise RuntimeError("fbfft_conv_fprop failed")
    _, t = timed(conv_auto, 200, 200, torch)
    extra["fft_conv_configs3_library_choice_ms_per_iter"] = round(t * 1e3, 4)
    extra["fft_conv_configs3_library_choice_fft_size"] = auto
    del wsa
    # the other two passes of the same layer
    g = synth.normal((128, 192, 23, 23), seed=32, device=dev)
    gi, gw = torch.empty_like(x), torch.empty_like(w)
    vg, vgi, vgw = F.view(g), F.view(gi), F.view(gw)
    ws2 = torch.empty(max(F.conv_workspace(1, 128, 64, 192, 32), F.conv_workspace(2, 128, 64, 192, 32)),
                      dtype=torch.uint8, device=dev)
    wsp2, wsb2 = ctypes.c_void_p(ws2.data_ptr()), ws2.numel()

    def bprop():
        if L.fbfft_conv_bprop(ctypes.byref(vg), ctypes.byref(vw), ctypes.byref(vgi), 32, wsp2, wsb2,
                              stream) != 0:
            raise RuntimeError("fbfft_conv_bprop failed")

    def accgrad():
        if L.fbfft_conv_accgrad(ctypes.byref(vx), ctypes.byref(vg), ctypes.byref(vgw), 32,
                                ctypes.c_float(1.0), 0, wsp2, wsb2, stream) != 0:
            raise RuntimeError("fbfft_conv_accgrad failed")
    _, t = timed(bprop, 200, 200, torch)
    extra["fft_conv_configs3_bprop_ms_per_iter"] = round(t * 1e3, 4)
    _, t = timed(accgrad, 200, 200, torch)
    extra["fft_conv_configs3_accgrad_ms_per_iter"] = round(t * 1e3, 4)
    del g, gi, gw, ws2
    A = synth.normal((128, 64, 17, 32, 2), seed=30, device=dev)
    Bm = synth.normal((192, 64, 17, 32, 2), seed=31, device=dev)
    C = torch.empty((128, 192, 17, 32, 2), device=dev)
    mm = prepared("fbfft_transpose_mm", F, A, Bm, C, 0, 1, 0, ctypes.c_float(1.0 / 1024))
    _, t = timed(mm, 200, 200, torch)
    extra["transposeMM_configs3_us"] = round(t * 1e6, 1)
    extra["transposeMM_configs3_TFLOPs"] = round(6.845e9 / t / 1e12, 1)
    extra["transposeMM_configs3_frac_of_fp32_mfma_peak"] = round(6.845e9 / t / 157.3e12, 4)
    # the kernel issues three real products per complex one: 6 flop per multiply-add
    extra["transposeMM_configs3_frac_issued"] = round(6.845e9 * 0.75 / t / 157.3e12, 4)
    del A, Bm, C
    # the same contraction on packed spectra (16 rows per plane instead of 17)
    Ap = synth.normal((128, 64, 16, 32, 2), seed=30, device=dev)
    Bp = synth.normal((192, 64, 16, 32, 2), seed=31, device=dev)
    Cp = torch.empty((128, 192, 16, 32, 2), device=dev)
    mmp = prepared("fbfft_transpose_mm_packed", F, Ap, Bp, Cp, 0, 1, 0, ctypes.c_float(1.0 / 1024))
    _, t = timed(mmp, 200, 200, torch)
    extra["transposeMM_packed_configs3_us"] = round(t * 1e6, 1)
    del Ap, Bp, Cp, x, w, out, ws
    # a 64-point layer (plane-major spectra through transposeMM): 32x32x60x60 * 64x32x5x5
    x6 = synth.normal((32, 32, 60, 60), seed=50, device=dev)
    w6 = synth.normal((64, 32, 5, 5), seed=51, std=0.02, device=dev)
    o6 = torch.empty((32, 64, 56, 56), device=dev)
    ws6 = torch.empty(F.conv_workspace(0, 32, 32, 64, 64), dtype=torch.uint8, device=dev)
    v6 = (F.view(x6), F.view(w6), F.view(o6))

    def conv64():
        if L.fbfft_conv_fprop(ctypes.byref(v6[0]), ctypes.byref(v6[1]), ctypes.byref(v6[2]), 64,
                              ctypes.c_void_p(ws6.data_ptr()), ws6.numel(), stream) != 0:
            raise RuntimeError("fbfft_conv_fprop (64) failed")
    _, t = timed(conv64, 200, 200, torch)
    flop64 = 2.0 * 32 * 64 * 56 * 56 * 32 * 25
    extra["fft_conv_64pt_32x32x60x60_k5_f64_ms_per_iter"] = round(t * 1e3, 4)
    extra["fft_conv_64pt_direct_equiv_TFLOPs"] = round(flop64 / t / 1e12, 1)
    del x6, w6, o6, ws6
    # configs[4]
    x4 = synth.uniform((16, 32, 256, 256), seed=40, device=dev)
    w4 = synth.normal((32, 32, 9, 9), seed=41, std=0.05, device=dev)
    o4 = torch.empty((16, 32, 248, 248), device=dev)
    ins, outs, n = F.make_tile_grid(x4, o4, 9, 9, 32)   # 11 x 11 tiles of stride 24
    vw4 = F.view(w4)

    def tiled():
        rc = L.fbfft_iterated_conv(32, ctypes.c_void_p(ins.data_ptr()),
                                   ctypes.c_void_p(outs.data_ptr()), ctypes.byref(vw4), 0,
                                   ctypes.c_float(1.0), 16, n, stream)
        if rc != 1:
            raise RuntimeError("fbfft_iterated_conv returned %d" % rc)
    _, t = timed(tiled, 30, 20, torch)
    extra["iterated_conv_configs4_ms_per_iter"] = round(t * 1e3, 4)
    extra["iterated_conv_configs4_direct_equiv_TFLOPs"] = round(163.3e9 / t / 1e12, 1)
    # the same descriptors through a caller-owned workspace (fbfft_iterated_conv_ws)
    wsd = torch.empty(F.iterated_conv_workspace(32, 0, 16, n, 32, 32), dtype=torch.uint8, device=dev)
    wsdp, wsdb = ctypes.c_void_p(wsd.data_ptr()), wsd.numel()

    def tiled_ws():
        rc = L.fbfft_iterated_conv_ws(32, ctypes.c_void_p(ins.data_ptr()),
                                      ctypes.c_void_p(outs.data_ptr()), ctypes.byref(vw4), 0,
                                      ctypes.c_float(1.0), 16, n, wsdp, wsdb, stream)
        if rc != 1:
            raise RuntimeError("fbfft_iterated_conv_ws returned %d" % rc)
    _, t = timed(tiled_ws, 60, 30, torch)
    extra["iterated_conv_ws_configs4_ms_per_iter"] = round(t * 1e3, 4)
    extra["iterated_conv_ws_configs4_direct_equiv_TFLOPs"] = round(163.3e9 / t / 1e12, 1)
    del wsd
    # the same layer through the convolution-layer entry point: the 121 windows per image
    # ride through the bin-major pipeline (spectra in a workspace) instead of the fused kernel
    ws4 = torch.empty(F.conv_workspace_image(0, 16, 32, 32, 256, 256, 9, 9, 32), dtype=torch.uint8,
                      device=dev)
    v4 = (F.view(x4), F.view(w4), F.view(o4))

    def layer4():
        if L.fbfft_conv_fprop(ctypes.byref(v4[0]), ctypes.byref(v4[1]), ctypes.byref(v4[2]), 32,
                              ctypes.c_void_p(ws4.data_ptr()), ws4.numel(), stream) != 0:
            raise RuntimeError("fbfft_conv_fprop (tiled) failed")
    _, t = timed(layer4, 60, 40, torch)
    mid, low = spread(layer4, 60, torch)
    extra["conv_layer_configs4_ms_per_iter"] = round(t * 1e3, 4)
    extra["conv_layer_configs4_ms_per_iter_median"] = round(mid * 1e3, 4)
    extra["conv_layer_configs4_ms_per_iter_min"] = round(low * 1e3, 4)
    extra["conv_layer_configs4_direct_equiv_TFLOPs"] = round(163.3e9 / t / 1e12, 1)
    # 260.5 MB of algorithmic traffic (input + filters + output) against the HBM peak
    tr4, tr4_src = profile_traffic("conv_pipeline_configs4.md", "traffic_bytes_per_iteration")
    extra["conv_layer_configs4_roofline"] = {
        "bound": "hbm", "achieved": round(260.5e6 / t / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": round(260.5e6 / t / 1e9 / HBM_PEAK_GBS, 4), "algorithmic_bytes": 260500000,
        "traffic": tr4, "traffic_source": tr4_src,
        "workload": "configs[4]: 16x32x256x256 * 32x32x9x9 -> 16x32x248x248, 32-point windows"}
    # the layer's other two passes on the same tiled image
    gi4, gw4 = torch.empty_like(x4), torch.empty_like(w4)
    vgi4, vgw4 = F.view(gi4), F.view(gw4)
    wsb = torch.empty(max(F.conv_workspace_image(1, 16, 32, 32, 256, 256, 9, 9, 32),
                          F.conv_workspace_image(2, 16, 32, 32, 256, 256, 9, 9, 32)),
                      dtype=torch.uint8, device=dev)

    def layer4_bprop():
        if L.fbfft_conv_bprop(ctypes.byref(v4[2]), ctypes.byref(v4[1]), ctypes.byref(vgi4), 32,
                              ctypes.c_void_p(wsb.data_ptr()), wsb.numel(), stream) != 0:
            raise RuntimeError("fbfft_conv_bprop (tiled) failed")

    def layer4_accgrad():
        if L.fbfft_conv_accgrad(ctypes.byref(v4[0]), ctypes.byref(v4[2]), ctypes.byref(vgw4), 32,
                                ctypes.c_float(1.0), 0, ctypes.c_void_p(wsb.data_ptr()), wsb.numel(),
                                stream) != 0:
            raise RuntimeError("fbfft_conv_accgrad (tiled) failed")
    _, t = timed(layer4_bprop, 40, 20, torch)
    extra["conv_layer_configs4_bprop_ms_per_iter"] = round(t * 1e3, 4)
    _, t = timed(layer4_accgrad, 40, 20, torch)
    extra["conv_layer_configs4_accgrad_ms_per_iter"] = round(t * 1e3, 4)
    del ws4, wsb, gi4, gw4
    # the other two passes (o4 as gradOutput): accGradParameters on the same descriptors,
    # updateGradInput on its own grid of disjoint gradInput windows
    bins, bouts, nbp = F.make_tile_grid(x4, o4, 9, 9, 32, F.FFT_UpdateGradInput)
    for pass_, key, ti, to, nt in ((1, "bprop", bins, bouts, nbp), (2, "accgrad", ins, outs, n)):
        def other():
            rc = L.fbfft_iterated_conv(32, ctypes.c_void_p(ti.data_ptr()),
                                       ctypes.c_void_p(to.data_ptr()), ctypes.byref(vw4), pass_,
                                       ctypes.c_float(1.0), 16, nt, stream)
            if rc != 1:
                raise RuntimeError("fbfft_iterated_conv returned %d" % rc)
        _, t = timed(other, 30, 20, torch)
        extra["iterated_conv_configs4_%s_ms_per_iter" % key] = round(t * 1e3, 4)


def run_only(name, steps, warmup, F, synth, torch, dev):
    """One workload in a tight loop, for profiling."""
    import re
    m2 = re.fullmatch(r"(r2c|c2r)(8|16|32|64|128)", name)
    if m2:
        # one 2D size on one set of buffers: configs[2]'s batches (256 MiB of input, far beyond
        # the last-level cache) and configs[1]'s 16384 planes at 32 x 32 (which stay in it:
        # r2c32hbm / c2r32hbm are the forms that read from HBM)
        n = int(m2.group(2))
        b = int(os.environ.get("FBFFT_BENCH_B", {8: 1 << 20, 16: 1 << 18, 32: 16384, 64: 16384,
                                                 128: 4096}[n]))
        x = synth.normal((b, n, n), seed=1, device=dev)
        spec = torch.empty((b, n // 2 + 1, n, 2), device=dev)
        fwd = prepared("fbfft_r2c_2d", F, x, spec, 0, 0)
        fwd()
        fn = fwd if name.startswith("r2c") else prepared("fbfft_c2r_2d", F, spec, x, 0, 0)
        _, t = timed(fn, steps, warmup, torch)
        return {"only": name, "planes": b, "us": round(t * 1e6, 2),
                "GBps": round(b * plane_bytes(n) / t / 1e9, 1)}
    if name in ("r2c32hbm", "c2r32hbm"):
        # configs[1] with operands served from HBM: eight sets of buffers in turn
        n, b, sets = 32, 16384, 8
        xs = [synth.normal((b, n, n), seed=1 + i, device=dev) for i in range(sets)]
        ss = [torch.empty((b, n // 2 + 1, n, 2), device=dev) for _ in range(sets)]
        fw = [prepared("fbfft_r2c_2d", F, xs[i], ss[i], 0, 0) for i in range(sets)]
        for f in fw:
            f()
        cs = fw if name == "r2c32hbm" else [prepared("fbfft_c2r_2d", F, ss[i], xs[i], 0, 0)
                                            for i in range(sets)]
        turn = [0]

        def step():
            cs[turn[0] % sets]()
            turn[0] += 1
        _, t = timed(step, steps, warmup, torch)
        return {"only": name, "us": round(t * 1e6, 2), "GBps": round(b * plane_bytes(n) / t / 1e9, 1)}
    m1 = re.fullmatch(r"(r2c|c2r)1d(32|64|128|256)?", name)
    if m1:
        # 1D: configs[0] (32 points, 4096 rows) or 256 MiB of input at the larger sizes
        n = int(m1.group(2) or 256)
        b = 4096 if n == 32 else (1 << 26) // n
        x = synth.uniform((b, n), seed=0, device=dev)
        spec = torch.empty((b, n // 2 + 1, 2), device=dev)
        fwd = prepared("fbfft_r2c_1d", F, x, spec, 0)
        fwd()
        fn = fwd if m1.group(1) == "r2c" else prepared("fbfft_c2r_1d", F, x, spec, 0)
        _, t = timed(fn, steps, warmup, torch)
        return {"only": name, "rows": b, "us": round(t * 1e6, 2),
                "GBps": round(b * (4 * n + 8 * (n // 2 + 1)) / t / 1e9, 1)}
    extra = {}
    if name in ("iter4", "iter4ws"):
        # configs[4] updateOutput through the fused tiled kernel only
        x4 = synth.uniform((16, 32, 256, 256), seed=40, device=dev)
        w4 = synth.normal((32, 32, 9, 9), seed=41, std=0.05, device=dev)
        o4 = torch.empty((16, 32, 248, 248), device=dev)
        ins, outs, n = F.make_tile_grid(x4, o4, 9, 9, 32)
        vw4 = F.view(w4)
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

        def tiled():
            rc = F.lib().fbfft_iterated_conv(32, ctypes.c_void_p(ins.data_ptr()),
                                             ctypes.c_void_p(outs.data_ptr()), ctypes.byref(vw4), 0,
                                             ctypes.c_float(1.0), 16, n, stream)
            assert rc == 1
        if name == "iter4ws":
            # the same descriptors through a caller-owned workspace
            wsd = torch.empty(F.iterated_conv_workspace(32, 0, 16, n, 32, 32), dtype=torch.uint8,
                              device=dev)

            def tiled():  # noqa: F811
                rc = F.lib().fbfft_iterated_conv_ws(32, ctypes.c_void_p(ins.data_ptr()),
                                                    ctypes.c_void_p(outs.data_ptr()),
                                                    ctypes.byref(vw4), 0, ctypes.c_float(1.0), 16, n,
                                                    ctypes.c_void_p(wsd.data_ptr()), wsd.numel(),
                                                    stream)
                assert rc == 1
        _, t = timed(tiled, steps, warmup, torch)
        return {"only": name, "us": round(t * 1e6, 2)}
    if name == "mm":
        A = synth.normal((128, 64, 17, 32, 2), seed=30, device=dev)
        Bm = synth.normal((192, 64, 17, 32, 2), seed=31, device=dev)
        C = torch.empty((128, 192, 17, 32, 2), device=dev)
        mm = prepared("fbfft_transpose_mm", F, A, Bm, C, 0, 1, 0, ctypes.c_float(1.0 / 1024))
        _, t = timed(mm, steps, warmup, torch)
        return {"only": name, "us": round(t * 1e6, 2), "TFLOPs": round(6.845e9 / t / 1e12, 2)}
    if name in ("conv", "conv_bprop", "conv_accgrad", "conv4", "conv4_bprop", "conv4_accgrad"):
        # one pass of the convolution layer at configs[3] / configs[4] shapes
        big = name.startswith("conv4")
        pass_ = 1 if name.endswith("bprop") else 2 if name.endswith("accgrad") else 0
        if big:
            nb, cin, cout, hw, k = 16, 32, 32, 256, 9
            x = synth.uniform((nb, cin, hw, hw), seed=40, device=dev)
            w = synth.normal((cout, cin, k, k), seed=41, std=0.05, device=dev)
        else:
            nb = int(os.environ.get("FBFFT_BENCH_CONV_B", "128"))  # profiling aid: other batch sizes
            cin, cout, k = 64, 192, 5
            hw = int(os.environ.get("FBFFT_BENCH_CONV_HW", "27"))  # profiling aid: other image sizes
            x = synth.normal((nb, cin, hw, hw), seed=30, device=dev)
            w = synth.normal((cout, cin, k, k), seed=31, std=0.02, device=dev)
        o = synth.normal((nb, cout, hw - k + 1, hw - k + 1), seed=32, device=dev)
        fft = int(os.environ.get("FBFFT_BENCH_CONV_N", "32"))  # profiling aid: other transform sizes
        ws = torch.empty(F.conv_workspace_image(pass_, nb, cin, cout, hw, hw, k, k, fft),
                         dtype=torch.uint8, device=dev)
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        vx, vw, vo = F.view(x), F.view(w), F.view(o)
        wsp, wsn = ctypes.c_void_p(ws.data_ptr()), ws.numel()
        L = F.lib()

        def layer():
            if pass_ == 0:
                rc = L.fbfft_conv_fprop(ctypes.byref(vx), ctypes.byref(vw), ctypes.byref(vo), fft,
                                        wsp, wsn, stream)
            elif pass_ == 1:
                rc = L.fbfft_conv_bprop(ctypes.byref(vo), ctypes.byref(vw), ctypes.byref(vx), fft,
                                        wsp, wsn, stream)
            else:
                rc = L.fbfft_conv_accgrad(ctypes.byref(vx), ctypes.byref(vo), ctypes.byref(vw), fft,
                                          ctypes.c_float(1.0), 0, wsp, wsn, stream)
            assert rc == 0
        _, t = timed(layer, steps, warmup, torch)
        return {"only": name, "us": round(t * 1e6, 2)}
    conv_extras(F, synth, torch, dev, extra)
    return {"only": name, **extra}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=800)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the informative extra configs")
    ap.add_argument("--only", default=None,
                    choices=["r2c32hbm", "c2r32hbm"] +
                            [d + n for d in ("r2c", "c2r") for n in ("8", "16", "32", "64", "128")] +
                            [d + "1d" + n for d in ("r2c", "c2r") for n in ("", "32", "64", "128", "256")] +
                            ["mm", "conv", "conv_bprop", "conv_accgrad", "iterconv", "iter4", "iter4ws",
                             "conv4", "conv4_bprop", "conv4_accgrad"],
                    help="run just this workload --steps times (for rocprofv3) and print its timing")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="only run a plain 256 MiB device-to-device copy 20 times: the known-size "
                         "kernel that FETCH_SIZE / WRITE_SIZE counter readings are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on exactly one GPU (no sharding or collectives "
                 "are part of the fbfft path); run with --gpus 1")

    import torch

    import fbcuda_amd as F
    from fbcuda_amd import synth

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    dev = torch.device("cuda:0")
    F.lib()

    if args.calibrate_copy:
        a = torch.zeros(64 * 1024 * 1024, device=dev)
        c = torch.empty_like(a)
        for _ in range(20):
            c.copy_(a)
        torch.cuda.synchronize()
        print(json.dumps({"calibrate_copy_bytes_read": a.numel() * 4,
                          "calibrate_copy_bytes_written": a.numel() * 4, "launches": 20}))
        return

    if args.only:
        print(json.dumps(run_only(args.only, args.steps, args.warmup, F, synth, torch, dev)))
        return

    N, B, SETS = 32, 16384, 8
    nbytes = B * plane_bytes(N)
    # Eight sets of operands (8 x 132 MB): a step runs on the set after the previous step's,
    # so no launch finds its planes in the 256 MiB last-level cache, as in a pipeline that
    # streams batches through the transform.  Set 0 is configs[1]'s own tensor (seed 1).
    xs = [synth.normal((B, N, N), seed=1 + i, device=dev) for i in range(SETS)]
    specs = [torch.empty((B, N // 2 + 1, N, 2), device=dev) for _ in range(SETS)]
    x, spec = xs[0], specs[0]
    back = torch.empty_like(x)
    calls = [prepared("fbfft_r2c_2d", F, a, b, 0, 0) for a, b in zip(xs, specs)]
    fwd = calls[0]
    inv = prepared("fbfft_c2r_2d", F, spec, back, 0, 0)
    turn = [0]

    def step():
        calls[turn[0] % SETS]()
        turn[0] += 1

    step_s, launch_s = timed(step, args.steps, args.warmup, torch)
    launch_mid, launch_min = spread(step, args.steps, torch)
    value = nbytes / step_s / 1e9

    def hbm_roofline(nb, t, mid, low, note):
        return {"bound": "hbm", "achieved": round(nb / t / 1e9, 1), "peak": HBM_PEAK_GBS,
                "unit": "GB/s", "frac": round(nb / t / 1e9 / HBM_PEAK_GBS, 4),
                "frac_median": round(nb / mid / 1e9 / HBM_PEAK_GBS, 4),
                "frac_best": round(nb / low / 1e9 / HBM_PEAK_GBS, 4),
                "kernel": "fft2dSmallForward<32>", "bytes_per_launch": nb,
                "launch_us": round(t * 1e6, 2), "launch_us_median": round(mid * 1e6, 2),
                "launch_us_min": round(low * 1e6, 2), "residency": note}

    traffic, traffic_src = profile_traffic("fft2dSmallForward32_configs1.md",
                                           "traffic_bytes_per_launch")
    roofline = dict(hbm_roofline(nbytes, launch_s, launch_mid, launch_min,
                                 "hbm: consecutive launches run on %d different sets of operands, "
                                 "%d MB in all" % (SETS, SETS * nbytes // 1000000)),
                    traffic=traffic, traffic_source=traffic_src)

    # What moving the same bytes costs with no arithmetic, under the same rotation: the
    # runtime's device-to-device copy and the library's own copy kernel, 66 MiB -> 66 MiB
    # (configs[1] reads 64 MiB and writes 68 MiB).
    half = nbytes // 2
    csrc = [t.view(-1)[:half // 4] for t in specs]          # contents do not matter
    cdst = [torch.empty(half // 4, device=dev) for _ in range(SETS)]
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    L = F.lib()

    cargs = [(ctypes.c_void_p(a.data_ptr()), ctypes.c_void_p(b.data_ptr()), half, stream)
             for a, b in zip(csrc, cdst)]

    def copy_runtime():
        i = turn[0] % SETS
        turn[0] += 1
        cdst[i].copy_(csrc[i])

    def copy_kernel():
        i = turn[0] % SETS
        turn[0] += 1
        if L.fbfft_bench_copy(*cargs[i]) != 0:
            raise RuntimeError("fbfft_bench_copy failed")
    n_aux, w_aux = max(args.steps, 40), max(args.warmup, 8)
    _, t_rt = timed(copy_runtime, n_aux, w_aux, torch)
    _, t_ck = timed(copy_kernel, n_aux, w_aux, torch)
    copy_ceiling = {
        "bytes_per_launch": 2 * half, "residency": roofline["residency"],
        "runtime_copy_us": round(t_rt * 1e6, 2), "runtime_copy_GBps": round(2 * half / t_rt / 1e9, 1),
        "copy_kernel_us": round(t_ck * 1e6, 2), "copy_kernel_GBps": round(2 * half / t_ck / 1e9, 1),
        "transform_over_copy_kernel": round(launch_s / t_ck, 3)}
    del csrc, cdst, cargs

    # the same launch on the same buffers over and over: operands in the last-level cache
    _, llc_s = timed(fwd, max(args.steps, 200), max(args.warmup, 200), torch)
    llc_mid, llc_min = spread(fwd, max(args.steps, 200), torch)
    roofline_llc = hbm_roofline(nbytes, llc_s, llc_mid, llc_min,
                                "last-level cache: the same 132 MB of operands every launch "
                                "(not an HBM figure)")
    x4 = synth.normal((4 * B, N, N), seed=6, device=dev)
    s4 = torch.empty((4 * B, N // 2 + 1, N, 2), device=dev)
    f4 = prepared("fbfft_r2c_2d", F, x4, s4, 0, 0)
    _, l4 = timed(f4, max(20, args.steps // 4), max(args.warmup // 4, 5), torch)
    m4, b4 = spread(f4, max(20, args.steps // 4), torch)
    roofline_4x = hbm_roofline(4 * nbytes, l4, m4, b4, "hbm: one launch over 65536 planes, 554 MB")
    del x4, s4, f4

    extra = {}
    if not args.no_extra:
        # C2R and the packed-format pair, operands from HBM like the headline (the inverse of
        # set i overwrites its own planes for i > 0; set 0 returns into `back`)
        def rotate(cs):
            def f():
                cs[turn[0] % SETS]()
                turn[0] += 1
            return f
        backs = [back] + xs[1:]
        invs = [prepared("fbfft_c2r_2d", F, specs[i], backs[i], 0, 0) for i in range(SETS)]
        _, l = timed(rotate(invs), n_aux, w_aux, torch)
        extra["c2r_32x32_b16384_us"] = round(l * 1e6, 2)
        extra["c2r_32x32_b16384_GBps"] = round(nbytes / l / 1e9, 1)
        # round-trip sanity on the benchmark tensors themselves
        err = float((back / (N * N) - x).double().norm() / x.double().norm())
        extra["roundtrip_rel_l2"] = err
        # packed spectra of configs[1]: [B][16][32][2], 8192 bytes per plane
        sps = [t.view(-1)[:B * (N // 2) * N * 2].view(B, N // 2, N, 2) for t in specs]
        pf = [prepared("fbfft_r2c_2d", F, backs[i] if i else x, sps[i], 0, 0) for i in range(SETS)]
        pi = [prepared("fbfft_c2r_2d", F, sps[i], backs[i], 0, 0) for i in range(SETS)]
        _, lp = timed(rotate(pf), n_aux, w_aux, torch)
        _, lq = timed(rotate(pi), n_aux, w_aux, torch)
        extra["r2c_32x32_packed_b16384_GBps"] = round(B * 8192 / lp / 1e9, 1)
        extra["c2r_32x32_packed_b16384_GBps"] = round(B * 8192 / lq / 1e9, 1)
        del sps, pf, pi, invs, backs
        del xs[1:], specs[1:], calls
        for n2, b2 in ((16, 262144), (8, 1048576), (64, 16384), (128, 4096)):
            x2 = synth.normal((b2, n2, n2), seed=2 + n2.bit_length() - 1, device=dev)
            s2 = torch.empty((b2, n2 // 2 + 1, n2, 2), device=dev)
            f2 = prepared("fbfft_r2c_2d", F, x2, s2, 0, 0)
            i2 = prepared("fbfft_c2r_2d", F, s2, x2, 0, 0)
            try:
                # the first hundred or so launches on fresh buffers run slower: past them
                _, lf = timed(f2, 50, 100, torch)
                _, li = timed(i2, 50, 100, torch)
            except RuntimeError:
                continue
            nb = b2 * plane_bytes(n2)
            extra["r2c_%dx%d_b%d_GBps" % (n2, n2, b2)] = round(nb / lf / 1e9, 1)
            extra["c2r_%dx%d_b%d_GBps" % (n2, n2, b2)] = round(nb / li / 1e9, 1)
            del x2, s2
        # configs[0] (1D, 32 points, 4096 rows: launch-bound) and the 1D sizes above one wave
        for n1, b1 in ((32, 4096), (64, 1 << 20), (128, 1 << 19), (256, 1 << 18)):
            x1 = synth.uniform((b1, n1), seed=0, device=dev)
            s1 = torch.empty((b1, n1 // 2 + 1, 2), device=dev)
            _, lf = timed(prepared("fbfft_r2c_1d", F, x1, s1, 0), 50, 100, torch)
            _, li = timed(prepared("fbfft_c2r_1d", F, x1, s1, 0), 50, 100, torch)
            nb = b1 * (4 * n1 + 8 * (n1 // 2 + 1))
            extra["r2c_1d_%d_b%d_us" % (n1, b1)] = round(lf * 1e6, 2)
            extra["c2r_1d_%d_b%d_us" % (n1, b1)] = round(li * 1e6, 2)
            extra["r2c_1d_%d_b%d_GBps" % (n1, b1)] = round(nb / lf / 1e9, 1)
            del x1, s1
        conv_extras(F, synth, torch, dev, extra)

    out = {
        "metric": "fbfft2D 32x32 R2C GB/s (% HBM peak); FFT-conv ms/iter at configs[3]",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "configs[1]: fbfft2D R2C, 16384 planes of 32x32 fp32 N(0,1), output "
                               "[16384][17][32][2]; 8448 algorithmic bytes per plane; operands "
                               "served from HBM (8 sets of buffers in turn, set 0 = seed 1)"},
        "roofline": roofline,
        "copy_ceiling": copy_ceiling,
        "roofline_llc": roofline_llc,
        "roofline_4x": roofline_4x,
        "extra": extra,
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(x.cpu().numpy(), N)
        if not args.no_extra:
            extra["fft_conv_cpu_baseline"] = conv_cpu_baseline()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
