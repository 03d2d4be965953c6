"""What the GPU at hand gives to the simplest kernels: the bandwidth of its memory and the rate of its bf16
matrix instructions, measured (``csrc/peaks.hip``).

    python -m infernum_amd.peaks            one JSON line

The published peaks of an MI355X are 8 TB/s and 2.5 PFLOP/s (dense bf16); the benchmark's fractions are against
those.  Beside them it reports what simple kernels reach on the device it runs on, as a reading aid and not as a
bound: memory three ways (a pass of 16-byte loads with all workgroups side by side, the same with every workgroup
on a stretch of its own, and copies, by a kernel of this package and by the runtime's own, counted as two bytes
moved per byte copied), the best of which is the figure; the matrix rate as the median of several long runs (the
clock moves with the load, a short run measures the moment).  (The reference measures the bandwidth it prices its
kernels against, docs/performance.md:9-41.)
"""
from __future__ import annotations

import ctypes
import json
from typing import Dict

import torch

from .kernels.api import KernelError, _ok, _p, _stream, load_library

READ_BYTES = 4 << 30            # far beyond the 256 MB memory-side cache and the L2s


def _times_ms(fn, repeats: int) -> list:
    out = []
    for _ in range(repeats):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        b.synchronize()
        out.append(a.elapsed_time(b))
    return out


def _time_ms(fn, repeats: int) -> float:
    """The fastest of ``repeats`` runs, in milliseconds, by the device's own clock."""
    return min(_times_ms(fn, repeats))


def read_bandwidth(device: str = "cuda:0", nbytes: int = READ_BYTES, repeats: int = 5) -> Dict[str, float]:
    """GB/s of memory traffic by the simplest kernels over ``nbytes``: one pass of 16-byte loads with the workgroups
    side by side ("strided") and with each on a stretch of its own ("blocks"), for several numbers of workgroups;
    a copy by a kernel of this package and one by the runtime (``Tensor.copy_``), as bytes read plus bytes written.
    "best" is the largest of all of them."""
    if not torch.cuda.is_available():
        raise KernelError("no GPU is visible")
    lib = load_library("core")
    dev = torch.device(device)
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    buf = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    buf.view(torch.int32).fill_(0x3C003C00)
    out: Dict[str, float] = {}
    with torch.cuda.device(dev):
        for per_cu in (4, 8, 16, 32):
            wgs = cus * per_cu
            sink = torch.empty(wgs * 256 * 4, dtype=torch.int32, device=dev)
            run = lambda: _ok(lib.ia_peak_read(_p(buf), ctypes.c_size_t(nbytes), _p(sink), wgs, _stream()), "peak_read")  # noqa: E731
            run()
            out[f"{per_cu}_workgroups_per_cu"] = round(nbytes / (_time_ms(run, repeats) * 1e-3) / 1e9, 1)
            blocks = lambda: _ok(lib.ia_peak_read_blocks(_p(buf), ctypes.c_size_t(nbytes), _p(sink), wgs, _stream()),  # noqa: E731
                                 "peak_read_blocks")
            blocks()
            out[f"blocks_{per_cu}_workgroups_per_cu"] = round(nbytes / (_time_ms(blocks, repeats) * 1e-3) / 1e9, 1)
        half = nbytes // 2 // 16 * 16
        src, dst = buf[:half], buf[half:2 * half]
        for per_cu in (8, 32):
            copy = lambda: _ok(lib.ia_peak_copy(_p(src), _p(dst), ctypes.c_size_t(half), cus * per_cu, _stream()),  # noqa: E731
                               "peak_copy")
            copy()
            out[f"copy_{per_cu}_workgroups_per_cu"] = round(2 * half / (_time_ms(copy, repeats) * 1e-3) / 1e9, 1)
        runtime_copy = lambda: dst.copy_(src)  # noqa: E731
        runtime_copy()
        out["copy_by_the_runtime"] = round(2 * half / (_time_ms(runtime_copy, repeats) * 1e-3) / 1e9, 1)
    out["best"] = max(out.values())
    return out


def mfma_rate(device: str = "cuda:0", rounds: int = 20000, repeats: int = 7) -> Dict[str, float]:
    """TFLOP/s of chains of ``v_mfma_f32_32x32x16_bf16`` on registers, one and two workgroups of four waves a
    compute unit: the median of several runs of some ten milliseconds each (the clock settles under the load; the
    fastest of a few short runs measured 2.05 to 2.37 PFLOP/s from one process to the next); the better grid."""
    if not torch.cuda.is_available():
        raise KernelError("no GPU is visible")
    lib = load_library("core")
    dev = torch.device(device)
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    out: Dict[str, float] = {}
    with torch.cuda.device(dev):
        for per_cu in (1, 2):
            wgs = cus * per_cu
            sink = torch.empty(wgs * 256, dtype=torch.float32, device=dev)
            flops = ctypes.c_double(0.0)
            run = lambda: _ok(lib.ia_peak_mfma(rounds, wgs, _p(sink), ctypes.byref(flops), _stream()), "peak_mfma")  # noqa: E731
            run()
            run()
            times = sorted(_times_ms(run, repeats))
            out[f"{per_cu}_workgroups_per_cu"] = round(flops.value / (times[len(times) // 2] * 1e-3) / 1e12, 1)
    out["best"] = max(out.values())
    return out


def measure(device: str = "cuda:0") -> Dict[str, object]:
    """{"hbm_read_gbs": best GB/s of a pass of loads, "hbm_gbs": best GB/s of loads and copies, "bf16_mfma_tflops":
    TFLOP/s, and the single figures}; about three seconds."""
    props = torch.cuda.get_device_properties(torch.device(device))
    read = read_bandwidth(device)
    mfma = mfma_rate(device)
    return {"device": props.name, "compute_units": props.multi_processor_count,
            "hbm_read_gbs": max(v for k, v in read.items() if not k.startswith("copy") and k != "best"),
            "hbm_gbs": read["best"], "bf16_mfma_tflops": mfma["best"],
            "read_gbs_by_grid": {k: v for k, v in read.items() if k != "best"},
            "mfma_tflops_by_grid": {k: v for k, v in mfma.items() if k != "best"},
            "read_bytes": READ_BYTES}


if __name__ == "__main__":
    print(json.dumps(measure()))
