"""What this GPU delivers to a kernel that does nothing else, measured: memory bandwidth for a kernel
that only reads, and the rate of back-to-back matrix-core instructions.  The published peaks (8 TB/s,
2.5 PFLOP/s dense bfloat16) are what the benchmark's fractions are stated against; these are what a
kernel on this machine can come to, and the benchmark programs state their results against both.
The matrix cores' rate depends on their operands: the chip lowers its clock with the power that toggling
operands draw, so it is measured twice -- on normally distributed values, like the benchmark's weights and
activations (about 1.8 PFLOP/s), and on ones (about 2.3)."""
from __future__ import annotations

from typing import Dict

import torch

from . import library
from .ops import _stream

_cache: Dict[int, Dict[str, float]] = {}


def _timed(fn, runs: int) -> float:
    """Milliseconds of the fastest of `runs` calls (each alone between two events)."""
    best = float("inf")
    for _ in range(runs):
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        fn()
        end.record()
        end.synchronize()
        best = min(best, start.elapsed_time(end))
    return best


def measured_peaks(device="cuda:0", read_bytes: int = 4 << 30, runs: int = 5) -> Dict[str, float]:
    """{"hbm_gbs": GB/s a read-only kernel reaches over a buffer far larger than the caches,
    "bf16_tflops": TFLOP/s of nothing but 32x32x16 bfloat16 MFMAs on normally distributed operands,
    "bf16_tflops_ones": the same on ones} -- measured once per process and device."""
    dev = torch.device(device)
    index = dev.index if dev.index is not None else torch.cuda.current_device()
    if index in _cache:
        return _cache[index]
    with torch.cuda.device(index):
        props = torch.cuda.get_device_properties(index)
        cus = props.multi_processor_count
        free, _ = torch.cuda.mem_get_info(index)
        read_bytes = int(min(read_bytes, max(64 << 20, free // 4))) // 4096 * 4096
        buf = torch.ones(read_bytes // 4, dtype=torch.int32, device=dev)
        sink = torch.zeros(cus * 16 * 256, dtype=torch.float32, device=dev)
        read = lambda: library.call("bc4g_probe_read", buf.data_ptr(), read_bytes, sink.data_ptr(), cus * 16, _stream())
        read()
        hbm = read_bytes / (_timed(read, runs) * 1e-3) / 1e9
        del buf
        iters, groups = 20000, cus                          # a workgroup of four waves a CU: a wave a SIMD
        flops = groups * 4 * iters * 16 * 2.0 * 32 * 32 * 16
        rates = {}
        for name, operands in (("bf16_tflops", torch.randn(12 * 256 * 8, device=dev).bfloat16()),
                               ("bf16_tflops_ones", torch.ones(12 * 256 * 8, device=dev).bfloat16())):
            mfma = lambda: library.call("bc4g_probe_mfma", operands.data_ptr(), iters, sink.data_ptr(), groups, _stream())
            library.call("bc4g_probe_mfma", operands.data_ptr(), 100, sink.data_ptr(), groups, _stream())
            rates[name] = round(flops / (_timed(mfma, max(2, runs // 2)) * 1e-3) / 1e12, 1)
    _cache[index] = {"hbm_gbs": round(hbm, 1), **rates}
    return _cache[index]
