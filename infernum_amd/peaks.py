"""What the GPU at hand gives to the simplest kernels: streaming read bandwidth of its memory and the rate of
its bf16 matrix instructions, measured (``csrc/peaks.hip``).

    python -m infernum_amd.peaks            one JSON line

The published peaks of an MI355X are 8 TB/s and 2.5 PFLOP/s (dense bf16).  A kernel cannot be asked to beat what
a bare stream of loads or a bare chain of matrix instructions reaches on the device it runs on, so the
benchmark reports its fractions against both.  (The reference measures the bandwidth it prices its kernels
against in the same way, docs/performance.md:9-41.)
"""
from __future__ import annotations

import ctypes
import json
from typing import Dict

import torch

from .kernels.api import KernelError, _ok, _p, _stream, load_library

READ_BYTES = 4 << 30            # far beyond the 256 MB memory-side cache and the L2s


def _time_ms(fn, repeats: int) -> float:
    """The fastest of ``repeats`` runs, in milliseconds, by the device's own clock."""
    best = float("inf")
    for _ in range(repeats):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        b.synchronize()
        best = min(best, a.elapsed_time(b))
    return best


def read_bandwidth(device: str = "cuda:0", nbytes: int = READ_BYTES, repeats: int = 5) -> Dict[str, float]:
    """GB/s of one pass of 16-byte loads over ``nbytes``, for several numbers of workgroups; the best of them."""
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
    out["best"] = max(out.values())
    return out


def mfma_rate(device: str = "cuda:0", rounds: int = 4000, repeats: int = 4) -> Dict[str, float]:
    """TFLOP/s of chains of ``v_mfma_f32_32x32x16_bf16`` on registers, one and two workgroups of four waves a
    compute unit; the best of them."""
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
            out[f"{per_cu}_workgroups_per_cu"] = round(flops.value / (_time_ms(run, repeats) * 1e-3) / 1e12, 1)
    out["best"] = max(out.values())
    return out


def measure(device: str = "cuda:0") -> Dict[str, object]:
    """{"hbm_read_gbs": best GB/s, "bf16_mfma_tflops": best TFLOP/s, and the single figures}; about two seconds."""
    props = torch.cuda.get_device_properties(torch.device(device))
    read = read_bandwidth(device)
    mfma = mfma_rate(device)
    return {"device": props.name, "compute_units": props.multi_processor_count,
            "hbm_read_gbs": read["best"], "bf16_mfma_tflops": mfma["best"],
            "read_gbs_by_grid": {k: v for k, v in read.items() if k != "best"},
            "mfma_tflops_by_grid": {k: v for k, v in mfma.items() if k != "best"},
            "read_bytes": READ_BYTES}


if __name__ == "__main__":
    print(json.dumps(measure()))
