"""What this GPU gives, measured: streaming bandwidth of HBM and the rate of its matrix and vector
units, by the engine's own micro-benchmark kernels (csrc/kernels/peaks.hip). The benchmark prints a
step's achieved figures against these beside the published peaks, as the reference plots its
roofline from peaks it measured itself
(/root/reference/benchmarks/roofline/plot_roofline_only.py:9-10)."""
from __future__ import annotations

import ctypes
from typing import Dict

import torch

from ..build import load_library
from .ops import KernelError, _p, _stream

NOMINAL = {"hbm_GBps": 8000.0, "mfma_bf16_TFLOPs": 2500.0, "mfma_f32_TFLOPs": 157.3}


def _timed(fn, reps: int) -> float:
    """Seconds per launch: `fn(reps)` queues that many launches; the first call warms up."""
    fn(2)
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    fn(reps)
    b.record()
    b.synchronize()
    return a.elapsed_time(b) * 1e-3 / reps


def measure_peaks(device="cuda:0", buffer_bytes: int = 2 << 30) -> Dict[str, float]:
    """Best of a few grid shapes each: HBM read and copy in GB/s (the buffer is far larger than every
    cache), bf16 and f32 MFMA loops and an f32 FMA loop in TFLOP/s."""
    dev = torch.device(device)
    if dev.type != "cuda":
        raise KernelError("peaks are measured on the GPU")
    lib = load_library("peaks")
    with torch.cuda.device(dev):
        src = torch.empty(buffer_bytes // 4, dtype=torch.int32, device=dev).fill_(1)
        dst = torch.empty_like(src)
        sink = torch.zeros(64, dtype=torch.float32, device=dev)
        n = ctypes.c_size_t(buffer_bytes)
        out: Dict[str, float] = {}

        def check(rc):
            if rc != 0:
                raise KernelError(f"peak kernel failed (code {rc})")

        best = 0.0
        for wgs in (2048, 4096, 8192, 16384):
            t = _timed(lambda r: check(lib.mllm_peak_stream_read(_p(src), n, _p(sink), wgs, r, _stream())), 5)
            best = max(best, buffer_bytes / t)
        out["hbm_read_GBps"] = round(best / 1e9, 1)
        best = 0.0
        for wgs in (2048, 4096, 8192, 16384):
            t = _timed(lambda r: check(lib.mllm_peak_stream_copy(_p(src), _p(dst), n, wgs, r, _stream())), 5)
            best = max(best, 2.0 * buffer_bytes / t)
        out["hbm_copy_GBps"] = round(best / 1e9, 1)
        flops = ctypes.c_double(0.0)
        for kind, key, iters in ((0, "mfma_bf16_TFLOPs", 4000), (1, "mfma_f32_TFLOPs", 4000), (2, "fma_f32_TFLOPs", 20000)):
            best = 0.0
            for wgs in (256 * 2, 256 * 4, 256 * 8):
                t = _timed(lambda r: check(lib.mllm_peak_math_loop(kind, wgs, iters, _p(sink), r, ctypes.byref(flops),
                                                                   _stream())), 3)
                best = max(best, flops.value / t)
            out[key] = round(best / 1e12, 1)
        del src, dst
        torch.cuda.empty_cache()
    return out
