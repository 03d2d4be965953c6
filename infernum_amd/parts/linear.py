"""The matrix product of every projection: y[M, N] = x[M, K] @ W[N, K]^T.

Weights stay in the layout of the file ([out, in]: rows contiguous in K, which
is what a product that streams the weight once wants); the reference transposes
them on the host instead (infernum-cuda/src/inner/weights/generic_impl.rs:107-131)
and calls cuBLAS (infernum-cuda/src/inner/cuda/ops/matmul.rs:68-117).

fp32: the hand-written fp32 kernel, always (no reduced-precision matrix mode).
bf16: up to 128 rows the hand-written MFMA kernel that streams the weight once or the library's
product, whichever was measured faster for the weight's shape (up to 16 rows always the former; without a
measurement up to 64 rows the former, to 128 for weights that are not wide); above that the library product (hipBLASLt, called directly with its choice of
an algorithm kept per shape), as the reference uses its library there; an fp32
result of many rows comes 128 rows at a time from the hand-written kernel.
``set_prefill_gemm("mfma")`` (or INFERNUM_PREFILL_GEMM=mfma in the environment)
sends the many-row bf16 products to the hand-written LDS-tiled MFMA kernel
instead, where it takes the size (K in steps of 64); it is correct at every size
but slower than the library so far, hence not the default.  ``"torch"`` sends
them to the same library through ``torch.mm``, which costs more on the host.

``epilogue="swiglu"`` returns silu(y[:, :N/2]) * y[:, N/2:]; the decode kernel
does it while it joins its partial sums, the other paths in a kernel of its own.
``keep_split`` lets the decode kernel hand its partial sums on as a
:class:`SplitSum`, for a norm or the rotary kernel to join.
"""
from __future__ import annotations

import os
from typing import Optional, Union

import torch

from ..kernels import api as K
from ..kernels.api import SplitSum


# The weight-streaming kernel takes up to 128 rows.  Up to 64 rows it is the faster one for every weight; from 65
# to 128 rows for weights of fewer than 16,384 rows (8B shapes at 128 rows: 23 against 25 us for QKV, 15 against
# 25 for the output projection, 38 against 75 for down), while the library is ahead on wider ones (gate+up 60
# against 76 us).
SKINNY_ROWS_ANY_WIDTH = 64
SKINNY_WIDE = 16384

# Which of the two the rows from 17 to 128 really go to is measured, once per shape of a weight and use
# (``measure_route``): the rule above stands where nothing was measured.  The library's kernels are ahead for
# some shapes already at 32 rows (Llama-2-13B's QKV and gate+up products at 64 rows: 35 against 52 and 61 against
# 82 us) and behind for others (the 8B shape's down projection: 38 against 34), and no rule of sizes tells which.
ROUTES = ("measured", "static")
_route = os.environ.get("INFERNUM_GEMM_ROUTE", "measured")
if _route not in ROUTES:
    raise ValueError(f"INFERNUM_GEMM_ROUTE={_route!r}: one of {ROUTES}")
_library_rows: dict = {}         # (N, K, epilogue, keep_split) -> bit b set: 16 b + 1 .. 16 b + 16 rows go to the library


def set_gemm_route(name: str) -> str:
    """"measured": engines made from now on time both products for their weights' shapes; "static": the rule
    of sizes.  Returns the previous choice."""
    global _route
    if name not in ROUTES:
        raise ValueError(f"gemm route {name!r}: one of {ROUTES}")
    previous, _route = _route, name
    return previous


def library_rows(N: int, K_: int, epilogue: Optional[str], keep_split: bool) -> int:
    """The measured choice for a weight [N, K_] in this use as a mask over blocks of 16 rows (bit b: 16 b + 1 to
    16 b + 16 rows go to the library), or -1 where nothing was measured."""
    return _library_rows.get((N, K_, epilogue, bool(keep_split)), -1) if _route == "measured" else -1


def _skinny_rows(M: int, N: int, Kdim: int, out_dtype: torch.dtype, epilogue: Optional[str], keep_split: bool) -> bool:
    """Whether a bf16 product of M rows goes to the weight-streaming kernel (sizes it takes assumed)."""
    if out_dtype != torch.bfloat16:
        return True
    mask = library_rows(N, Kdim, epilogue, keep_split)
    if mask >= 0:
        return not (mask >> ((M - 1) // 16)) & 1
    return M <= SKINNY_ROWS_ANY_WIDTH or N < SKINNY_WIDE


def measure_routes_for(rt, uses) -> None:
    """``uses``: (weight, epilogue, keep_split) of a part that has just been loaded.  On a GPU, in bfloat16 with the
    fast kernels, and with the measured route switched on, each use's shape is measured (once a process)."""
    if _route == "measured" and rt.device.type == "cuda" and rt.dtype == torch.bfloat16 and rt.kernels == "auto":
        for w, epilogue, keep_split in uses:
            measure_route(w, epilogue, keep_split)


def measure_route(w: torch.Tensor, epilogue: Optional[str], keep_split: bool, margin: float = 0.95) -> int:
    """Times, for 32 to 128 rows in steps of 16, the weight-streaming product as this use launches it (its
    partial sums left for the next kernel with ``keep_split``, the activation in its epilogue) against the
    library's (followed by the activation's kernel), on the weight itself, and keeps which is faster (the
    library must win by 5 %: a tie stays with the kernel whose sums do not depend on a library's version).
    Once per shape and use in a process.  Returns the mask of :func:`library_rows`."""
    N, Kdim = w.shape
    key = (N, Kdim, epilogue, bool(keep_split))
    if key in _library_rows:
        return _library_rows[key]
    mask = 0
    if w.is_cuda and w.dtype == torch.bfloat16 and K.gemm_skinny_supported(1, N, Kdim) and _prefill_gemm == "library":
        def timed(fn) -> float:
            best = float("inf")
            for _ in range(3):
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                for _ in range(4):
                    fn()
                b.record()
                b.synchronize()
                best = min(best, a.elapsed_time(b))
            return best
        try:
            for block in range(1, K.SKINNY_MAX_M // 16):
                M = 16 * (block + 1)
                x = torch.zeros((M, Kdim), dtype=torch.bfloat16, device=w.device)
                y = torch.empty((M, N), dtype=torch.bfloat16, device=w.device)
                act = torch.empty((M, N // 2), dtype=torch.bfloat16, device=w.device) if epilogue == "swiglu" else None

                def own():
                    K.gemm_skinny(x, w, epilogue=epilogue, keep_split=keep_split)

                def library():
                    K.gemm_library(x, w, out=y)
                    if act is not None:
                        K.swiglu(y, act)
                own(), library()                      # the first call of a shape asks the library for its plan
                if timed(library) < margin * timed(own):
                    mask |= 1 << block
        except K.KernelError:
            mask = 0                                  # a shape that one of them refuses: the rule of sizes
            _library_rows[key] = -1
            return -1
    _library_rows[key] = mask
    return mask

PREFILL_GEMMS = ("library", "mfma", "torch")
_prefill_gemm = os.environ.get("INFERNUM_PREFILL_GEMM", "library")
if _prefill_gemm not in PREFILL_GEMMS:
    raise ValueError(f"INFERNUM_PREFILL_GEMM={_prefill_gemm!r}: one of {PREFILL_GEMMS}")


def set_prefill_gemm(name: str) -> str:
    """Chooses the bf16 product for more than 64 rows; returns the previous choice."""
    global _prefill_gemm
    if name not in PREFILL_GEMMS:
        raise ValueError(f"prefill gemm {name!r}: one of {PREFILL_GEMMS}")
    previous, _prefill_gemm = _prefill_gemm, name
    return previous


def prefill_gemm() -> str:
    return _prefill_gemm


def linear(x: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
           epilogue: Optional[str] = None, keep_split: bool = False,
           kernels: str = "auto") -> Union[torch.Tensor, SplitSum]:
    """``kernels="generic"``: the plain product (fp32 multiply-adds in a fixed order) for every size and type."""
    M, Kdim = x.shape
    N = w.shape[0]
    out_dtype = out_dtype or x.dtype
    n_out = N // 2 if epilogue == "swiglu" else N
    if M == 0:
        return torch.empty((0, n_out), dtype=out_dtype, device=x.device)
    if kernels == "generic":
        if x.dtype not in (torch.float32, torch.bfloat16):
            raise K.KernelError(f"linear: dtype {x.dtype} is not supported")
        y = K.gemm_generic(x, w, torch.empty((M, N), dtype=out_dtype, device=x.device))
    elif x.dtype == torch.bfloat16 and K.gemm_skinny_supported(M, N, Kdim) and x.is_contiguous() and \
            _skinny_rows(M, N, Kdim, out_dtype, epilogue, keep_split):
        return K.gemm_skinny(x, w, epilogue=epilogue, keep_split=keep_split, out_dtype=out_dtype)
    elif x.dtype == torch.float32:
        y = K.gemm_generic(x, w, torch.empty((M, N), dtype=out_dtype, device=x.device))
    elif x.dtype != torch.bfloat16:
        raise K.KernelError(f"linear: dtype {x.dtype} is not supported")
    elif out_dtype == torch.bfloat16:
        if _prefill_gemm == "mfma" and x.is_contiguous() and K.gemm_mfma_supported(M, N, Kdim):
            y = K.gemm_mfma(x, w)
        elif _prefill_gemm == "torch" or not x.is_contiguous():
            y = torch.mm(x, w.t())                  # library product, fp32 accumulation
        else:
            try:
                y = K.gemm_library(x, w)
            except K.KernelUnsupported:             # the library has no algorithm for this shape
                y = K.gemm_mfma(x, w) if K.gemm_mfma_supported(M, N, Kdim) else \
                    K.gemm_generic(x, w, torch.empty((M, N), dtype=out_dtype, device=x.device))
    elif K.gemm_skinny_supported(1, N, Kdim) and x.is_contiguous():
        # fp32 result from bf16 operands, many rows: 128 rows at a time through the skinny kernel
        y = torch.empty((M, N), dtype=out_dtype, device=x.device)
        for m0 in range(0, M, K.SKINNY_MAX_M):
            m1 = min(M, m0 + K.SKINNY_MAX_M)
            K.gemm_skinny(x[m0:m1], w, out=y[m0:m1])
    else:
        y = K.gemm_generic(x, w, torch.empty((M, N), dtype=out_dtype, device=x.device))
    if epilogue == "swiglu":
        return K.swiglu(y, torch.empty((M, n_out), dtype=y.dtype, device=y.device))
    if epilogue is not None:
        raise K.KernelError(f"linear: unknown epilogue {epilogue!r}")
    return y
