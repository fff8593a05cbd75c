"""Measured peaks of the GPU at hand, for the benchmark's report: what a read stream and what the bfloat16
matrix cores reach on this machine under this package's own kernels (``csrc/peaks.hip``)."""
from __future__ import annotations

import ctypes
from typing import Tuple

import torch

from . import library
from .kernels import KernelError, _check, _ptr, _stream


def _timed(launch, reps: int) -> float:
    """The shortest of ``reps`` launches in seconds (a peak is what the machine can do, not what it did on average),
    timed with events on the current stream."""
    launch()
    torch.cuda.synchronize()
    times = []
    for _ in range(reps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        launch()
        e1.record()
        e1.synchronize()
        times.append(e0.elapsed_time(e1) * 1e-3)
    return min(times)


def read_bandwidth(num_bytes: int = 2 << 30, reps: int = 11, device: str = "cuda:0") -> float:
    """Bytes a second of a read-only stream over ``num_bytes`` of device memory (far more than the caches hold),
    eight workgroups a compute unit."""
    if not torch.cuda.is_available():
        raise KernelError("the peaks are measured on the GPU")
    lib = library.peaks()
    buf = torch.empty(num_bytes // 4, dtype=torch.int32, device=device)
    buf.fill_(1)
    blocks = 8 * torch.cuda.get_device_properties(device).multi_processor_count
    sink = torch.empty(blocks, dtype=torch.int32, device=device)
    sec = _timed(lambda: _check(lib, lib.pico_peak_read(_ptr(buf), ctypes.c_longlong(buf.numel() * 4), _ptr(sink), blocks,
                                                        _stream())), reps)
    return buf.numel() * 4 / sec


def mfma_peak(reps: int = 5, iters: int = 20000, device: str = "cuda:0") -> Tuple[float, float]:
    """(flops a second, seconds of one run) of back-to-back bfloat16 32x32x16 products, two workgroups of four
    waves on every compute unit; a run lasts some milliseconds, so the clock is the one the chip holds under load."""
    if not torch.cuda.is_available():
        raise KernelError("the peaks are measured on the GPU")
    lib = library.peaks()
    lib.pico_peak_mfma_flops.restype = ctypes.c_longlong
    blocks = 2 * torch.cuda.get_device_properties(device).multi_processor_count
    sink = torch.zeros(4, dtype=torch.float32, device=device)
    sec = _timed(lambda: _check(lib, lib.pico_peak_mfma(blocks, iters, _ptr(sink), _stream())), reps)
    return lib.pico_peak_mfma_flops(blocks, iters) / sec, sec
