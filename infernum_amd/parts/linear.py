"""The matrix product of every projection: y[M, N] = x[M, K] @ W[N, K]^T.

Weights stay in the layout of the file ([out, in]: rows contiguous in K, which
is what a product that streams the weight once wants); the reference transposes
them on the host instead (infernum-cuda/src/inner/weights/generic_impl.rs:107-131)
and calls cuBLAS (infernum-cuda/src/inner/cuda/ops/matmul.rs:68-117).

Which kernel a product goes to is decided in ONE place, :func:`plan`: a short list of routes, each for some
blocks of sixteen rows.  :func:`linear` runs the route of the rows at hand; :func:`emit_linear` writes every
route into a step's program with its condition, so both make the same launches.

fp32: the hand-written fp32 kernel, always (no reduced-precision matrix mode).
bf16: up to 128 rows the hand-written MFMA kernel that streams the weight once, or the library's product
(hipBLASLt, called directly with its choice of an algorithm kept per shape) where that is known to be faster for
the weight's shape (:data:`KNOWN_ROUTES`, a table that is part of the source, so that two runs of one model make
the same launches; ``INFERNUM_GEMM_ROUTE=measured`` times both when a model loads instead, ``static`` keeps to
the rule of sizes); for the bands of rows of :data:`KNOWN_MID_ROWS` (up to a few hundred rows) the LDS-tiled MFMA
kernel with K split over workgroups, for products whose partial sums the next kernel takes (the library's kernels
for so few rows leave most of the GPU idle, and from some tens of rows on the tiled kernel streams a weight faster
than the weight-streaming one); above that the library, as the reference uses its library there; an fp32 result of more
than 128 rows comes from the LDS-tiled kernel's fp32 sums (128 rows at a time from the weight-streaming kernel where
the tiled one does not take the size).  ``set_prefill_gemm("mfma")`` (or
INFERNUM_PREFILL_GEMM=mfma) sends the many-row bf16 products to the hand-written LDS-tiled MFMA kernel instead,
where it takes the size (K in steps of 64).

``epilogue="swiglu"`` returns silu(y[:, :N/2]) * y[:, N/2:]; the decode kernel
does it while it joins its partial sums, the other paths in a kernel of its own.
``keep_split`` lets the decode kernel hand its partial sums on as a
:class:`SplitSum`, for a norm or the rotary kernel to join.
"""
from __future__ import annotations

import os
from dataclasses import dataclass
from typing import Any, Dict, List, Optional, Tuple, Union

import torch

from ..kernels import api as K
from ..kernels.api import SplitSum

ALL_BLOCKS = 0x1FF          # bit b < 8: 16 b + 1 .. 16 b + 16 rows; bit 8: more than 128 rows
_UP_TO_128 = 0xFF

# The weight-streaming kernel takes up to 128 rows.  Up to 64 rows it is the faster one for most weights; from 65
# to 128 rows for weights of fewer than 16,384 rows (8B shapes at 128 rows: 23 against 25 us for QKV, 15 against
# 25 for the output projection, 38 against 75 for down), while the library is ahead on wider ones (gate+up 60
# against 76 us).  This rule stands for shapes that the table below does not hold.
SKINNY_ROWS_ANY_WIDTH = 64
SKINNY_WIDE = 16384

# (N, K, epilogue, keep_split) of a weight and its use -> the blocks of sixteen rows (bit b: 16 b + 1 .. 16 b + 16)
# that go to the library, for 17 to 128 rows.  Measured with ``measure_route`` on an MI355X, three times over, a
# bit kept where most runs agreed; the shapes are those of the Llama 1B, 8B, 13B and 70B layers.  The library's
# kernels are ahead for some shapes already at 32 rows and behind for others at 128, and no rule of sizes tells.
KNOWN_ROUTES: Dict[Tuple[int, int, Optional[str], bool], int] = {
    (3072, 2048, None, True): 0, (2048, 2048, None, True): 0, (16384, 2048, "swiglu", False): 0b11110010,
    (2048, 8192, None, True): 0,
    (6144, 4096, None, True): 0, (4096, 4096, None, True): 0, (28672, 4096, "swiglu", False): 0b11110000,
    (4096, 14336, None, True): 0,
    (15360, 5120, None, True): 0b11111110, (5120, 5120, None, True): 0,
    (27648, 5120, "swiglu", False): 0b11111010, (5120, 13824, None, True): 0,
    (10240, 8192, None, True): 0, (8192, 8192, None, True): 0,
    (57344, 8192, "swiglu", False): 0b11111110, (8192, 28672, None, True): 0,
}

# (N, K) of a weight whose product leaves partial sums for the next kernel -> bands (first row, last row, parts): for
# these numbers of rows the LDS-tiled MFMA kernel takes the product with K split into so many parts (tiles of
# 128 x 128 of the result: the parts bring the workgroups to about one a compute unit, which is what was fastest
# for nearly every shape).  Measured on an MI355X with cold weights, in microseconds.
# Above 128 rows, against the library's product, at 129 / 192 / 256 rows: the 8B shape's down projection 37 / 41 / 45
# against 58 / 104 / 63, its output projection 17 / 18 / 19 against 22 / 34 / 23, its QKV product 23 / 24 / 26 against
# 40 / 35 / 42 (the rotary kernel then adds the two parts); the 13B shape's down projection 43 / 47 / 53 against
# 54 / 100 / 120, the 70B shape's 165 / 155 / 163 against 298 / 231 / 312, the 1B shape's 16 / 17 / 18 against 27 / 27 /
# 27.  At 384 rows: the 8B shape's down projection 73 against 79, the 13B shape's 72 against 91, the 1B shape's 22
# against 34.  The 8B shape's decode step at 160 / 192 / 256 requests: 19.8k / 21.4k / 24.3k tokens/s against 15.7k /
# 16.3k / 21.7k with the library's products.
# Up to 128 rows, against the weight-streaming kernel (or the library where KNOWN_ROUTES has it), at 32 / 64 / 128
# rows: the 8B shape's down projection 25 / 26 / 30 against 29 / 32 / 40, its QKV product 13 / 14 / 17 against 15 / 17 /
# 24, its output projection 10.5 / 11.5 / 14 against 10 / 12 / 15.5; the 13B shape's down projection 28 / 30 / 34
# against 33 / 37 / 46, its output projection 14 / 16 / 19 against 16 / 19 / 23; the 70B shape's down projection 84 /
# 90 / 105 against 94 / 111 / 139, its QKV product 36 / 35 / 39 against 38 / 41 / 52.  The 8B shape's decode step at 32 / 64 / 128 requests: 7.34k / 11.93k / 17.84k tokens/s
# against 7.08k / 11.52k / 17.03k.  A band begins where the tiled kernel was ahead; a shape whose product came out
# even stays where it was (an entry without bands).
KNOWN_MID_ROWS: Dict[Tuple[int, int], Tuple[Tuple[int, int, int], ...]] = {
    (2048, 8192): ((17, 128, 16), (129, 256, 8), (257, 384, 5), (385, 512, 4)),
    (3072, 2048): (), (2048, 2048): (),
    (4096, 14336): ((17, 128, 8), (129, 256, 4), (257, 384, 2)), (4096, 4096): ((49, 128, 8), (129, 256, 4)),
    (6144, 4096): ((17, 128, 5), (129, 256, 2)),
    (5120, 13824): ((17, 128, 6), (129, 256, 3), (257, 384, 2)), (5120, 5120): ((1, 128, 6), (129, 256, 3), (257, 384, 2)),
    (15360, 5120): ((1, 16, 2), (97, 128, 2)),
    (8192, 28672): ((17, 128, 4), (129, 256, 2)), (8192, 8192): ((25, 128, 4), (129, 256, 2)),
    (10240, 8192): ((33, 128, 3),),
}

# (N, K) of a gate+up weight -> bands (first row, last row) in which the LDS-tiled kernel with the activation in
# its epilogue takes the product (the 8B shape's at 32 / 64 / 128 rows: 43 / 45 / 51 us against the weight-streaming
# kernel's 47 / 56 / 73 and the library's with the activation's launch 54 / 54 / 57).  No rule of sizes stands behind
# this table: 22,016 x 4,096 gains as the 8B shape does (38 / 42 / 48 us against 45 / 53 / 71 and 46 / 48 / 50), while for
# 16,384 x 3,072 and 37,888 x 3,584 the library's product with the activation's launch is ahead from 32 rows on.
KNOWN_GLU_ROWS: Dict[Tuple[int, int], Tuple[Tuple[int, int], ...]] = {
    (28672, 4096): ((17, 128),), (27648, 5120): ((33, 128),), (57344, 8192): ((17, 128),), (16384, 2048): ((129, 256),),
    (22016, 4096): ((17, 128),),
}

ROUTES = ("table", "measured", "static")
_route = os.environ.get("INFERNUM_GEMM_ROUTE", "table")
if _route not in ROUTES:
    raise ValueError(f"INFERNUM_GEMM_ROUTE={_route!r}: one of {ROUTES}")
_measured: Dict[Tuple[int, int, Optional[str], bool], int] = {}


def set_gemm_route(name: str) -> str:
    """"table": the routes that are part of the source, then the rule of sizes; "measured": parts loaded from now
    on time both products for their weights' shapes (once a process); "static": the rule of sizes alone.  Engines
    that are built already keep the launches they were built with.  Returns the previous choice."""
    global _route
    if name not in ROUTES:
        raise ValueError(f"gemm route {name!r}: one of {ROUTES}")
    previous, _route = _route, name
    return previous


def gemm_routes() -> Dict[str, Any]:
    """What decides the routes now, for a benchmark's record: the mode and, when measured, the outcomes."""
    return {"route": _route, "measured": {f"{n}x{k}{'+' + e if e else ''}{'/split' if s else ''}": m
                                          for (n, k, e, s), m in sorted(_measured.items(), key=str)}}


def library_rows(N: int, K_: int, epilogue: Optional[str], keep_split: bool) -> int:
    """The blocks of sixteen rows (bit b: 16 b + 1 to 16 b + 16, b = 1 .. 7) of a bf16 product with this weight
    and use that go to the library rather than to the weight-streaming kernel."""
    key = (N, K_, epilogue, bool(keep_split))
    mask = -1
    if _route == "measured":
        mask = _measured.get(key, -1)
    elif _route == "table":
        mask = KNOWN_ROUTES.get(key, -1)
    if mask < 0:
        mask = 0 if N < SKINNY_WIDE else 0xFF & ~((1 << (SKINNY_ROWS_ANY_WIDTH // 16)) - 1)
    return mask & 0xFE             # up to 16 rows the weight-streaming kernel, always


MID_ROWS_WORKGROUPS = 256      # the MI355X's compute units: the workgroups a launch of the split tiled kernel aims at
MID_ROWS_MOST_PARTS = 8        # as far as measured


def _mid_rows_by_size(N: int, K_: int) -> Tuple[Tuple[int, int, int], ...]:
    """For shapes the table does not hold: per band of rows (33 to 128, 129 to 256, 257 to 384: one, two and three
    tiles of 128 rows) as many parts as bring the tiles of 128 x 128 to one workgroup a compute unit, while those are
    at least two (with one part the library was as fast or faster for every shape measured) and a part keeps at
    least 8 steps of K.  Measured beside the table's shapes on those of other models of the family (4,096 x 11,008,
    12,288 x 4,096, 3,072 x 8,192, 5,120 x 3,072, 3,584 x 18,944, ...): ahead of the weight-streaming kernel and of the
    library, or even with the better of them, from 32 rows on."""
    bands = []
    tiles_n = -(-N // 128)
    for tiles_m in (1, 2, 3):
        parts = min(MID_ROWS_WORKGROUPS // (tiles_m * tiles_n), K_ // 64 // 8, MID_ROWS_MOST_PARTS)
        if parts < 2:
            break
        bands.append((33 if tiles_m == 1 else 128 * (tiles_m - 1) + 1, 128 * tiles_m, parts))
    return tuple(bands)


def mid_rows(N: int, K_: int, keep_split: bool) -> Tuple[Tuple[int, int, int], ...]:
    """(first row, last row, parts) for which the LDS-tiled kernel, K split into ``parts``, takes the product with
    this weight; none where the library takes every number of rows above 128.  By the table, then by the rule of
    sizes ("static": by the rule alone)."""
    if not keep_split or _prefill_gemm != "library" or K_ % 64:
        return ()
    bands = KNOWN_MID_ROWS.get((N, K_)) if _route == "table" else None
    if bands is None:
        bands = _mid_rows_by_size(N, K_)
    return tuple((lo, hi, parts) for lo, hi, parts in bands
                 if 1 <= lo <= hi and K.gemm_mfma_supported(hi, N, K_) and 1 <= parts <= K_ // 64)


def tiled_copy(w: torch.Tensor, epilogue: Optional[str]) -> Optional[torch.Tensor]:
    """The copy of the weight laid out for the weight-streaming kernel in this use, if the part that owns the weight
    had one made (``prepare_weights``)."""
    made = getattr(w, "_infernum_tiled", None)
    return made.get(epilogue) if made else None


COPIES_LEAVE_FREE = 0.15      # of the device's memory: second copies are made only while this much stays free


def _room_for_copy(w: torch.Tensor) -> bool:
    """Whether a second copy of ``w`` still leaves COPIES_LEAVE_FREE of the device's memory free (for the cache and
    the steps' intermediates): a model that fills the memory keeps the file's layout for the rest of its weights
    (the same bits, a few per cent slower), where copies of all would leave no room for the cache."""
    free, total = torch.cuda.mem_get_info(w.device)
    # what the allocator holds without using it counts as free: it hands that out again before it asks for more
    free += torch.cuda.memory_reserved(w.device) - torch.cuda.memory_allocated(w.device)
    return free - w.numel() * w.element_size() >= COPIES_LEAVE_FREE * total


def prepare_weights(rt, uses) -> None:
    """``uses``: (weight, epilogue, keep_split) of a part that has just been loaded.  On a GPU, in bfloat16 with the
    fast kernels: a weight with so many rows that the weight-streaming kernel gives every workgroup all of K (no
    split: the gate+up matrix) gets a second copy laid out for that kernel, in which a workgroup's 64 rows x 256
    values of a chunk are consecutive, so that the workgroup reads one stretch of memory front to back
    (``kernels.api.tile_weight``; the same bits).  Rows of the matrix as the file holds it lie K values apart, and a
    workgroup that walks 64 of them side by side gets less out of the memory: measured on an MI355X, the 8B shape's
    gate+up product at 8 rows 41.8 against 43.4 us, the 13B shape's 53.2 against 57.5, the 70B shape's 168 against 175
    (before the kernel's tiles of rows walked K from starts of their own the gap was twice that, and the head, which
    is even now and gets no copy any more, gained 9 %), for 7.5 GB more memory (the 70B shape: 75 GB beside 141 GB of
    weights; copies are made while COPIES_LEAVE_FREE of the device's memory stays free); weights whose K is split over
    workgroups gain nothing.  The copy in the file's layout stays: the products for more rows read it.  With the
    measured route switched on, each use's shape is timed as well (once a process)."""
    if not (rt.device.type == "cuda" and rt.dtype == torch.bfloat16 and rt.kernels == "auto"):
        return
    for w, epilogue, keep_split in uses:
        N, Kdim = w.shape
        if K.gemm_skinny_supported(1, N, Kdim) and w.is_contiguous() and K.gemm_skinny_splits(N, Kdim) == 1:
            made = getattr(w, "_infernum_tiled", None)
            if made is None:
                made = w._infernum_tiled = {}
            if epilogue not in made and _room_for_copy(w):
                made[epilogue] = K.tile_weight(w, epilogue)
        if _route == "measured":
            measure_route(w, epilogue, keep_split)


def measure_route(w: torch.Tensor, epilogue: Optional[str], keep_split: bool, margin: float = 0.95) -> int:
    """Times, for 32 to 128 rows in steps of 16, the weight-streaming product as this use launches it (its
    partial sums left for the next kernel with ``keep_split``, the activation in its epilogue) against the
    library's (followed by the activation's kernel), on the weight itself, and keeps which is faster (the
    library must win by 5 %: a tie stays with the kernel whose sums do not depend on a library's version).
    Once per shape and use in a process.  Returns the mask of :func:`library_rows`."""
    N, Kdim = w.shape
    key = (N, Kdim, epilogue, bool(keep_split))
    if key in _measured:
        return _measured[key]
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
            mask = -1                                 # a shape that one of them refuses: the rule of sizes
    _measured[key] = mask
    return mask


PREFILL_GEMMS = ("library", "mfma")
_prefill_gemm = os.environ.get("INFERNUM_PREFILL_GEMM", "library")
if _prefill_gemm not in PREFILL_GEMMS:
    raise ValueError(f"INFERNUM_PREFILL_GEMM={_prefill_gemm!r}: one of {PREFILL_GEMMS}")


def set_prefill_gemm(name: str) -> str:
    """Chooses the bf16 product for more than 128 rows; returns the previous choice."""
    global _prefill_gemm
    if name not in PREFILL_GEMMS:
        raise ValueError(f"prefill gemm {name!r}: one of {PREFILL_GEMMS}")
    previous, _prefill_gemm = _prefill_gemm, name
    return previous


def prefill_gemm() -> str:
    return _prefill_gemm


# ------------------------------------------------------------------------------ the one place that decides
@dataclass(frozen=True)
class Route:
    """Rows (a mask over blocks of sixteen, see ALL_BLOCKS) -> the kernel that takes them.  Kinds: "generic"
    (fp32 multiply-adds in a fixed order), "skinny" (the weight-streaming kernel, its parts joined, the
    activation in its epilogue), "skinny_split" (the same with its partial sums left for the next kernel),
    "skinny_rows" (128 rows at a time), "library" (hipBLASLt; ``fallback`` names the kernel for a shape it
    refuses), "mfma" (the LDS-tiled kernel), "mfma_split" (the same with K split into ``parts``, its partial
    sums left for the next kernel), "mfma_f32" (the same in one part: an fp32 result from bf16 operands), "mfma_swiglu" (the tiled kernel with the
    activation in its epilogue).  A route
    with ``rows`` (first, last) takes those numbers of rows only, and takes them from the routes without that stand
    behind it."""

    blocks: int
    kind: str
    fallback: Optional[str] = None
    rows: Optional[Tuple[int, int]] = None
    parts: int = 0


FP32_TILED_FROM_ROWS = (49, 81)     # an fp32 result goes to the tiled kernel from so many rows on: K >= 4,096; shorter K
_MANY_ROWS = 65536         # the LDS-tiled kernel addresses rows with 32 bits: its fitness is judged at this many


def plan(N: int, Kdim: int, dtype: torch.dtype, out_dtype: torch.dtype, epilogue: Optional[str], keep_split: bool,
         kernels: str = "auto") -> List[Route]:
    """The routes of x [M, Kdim] (``dtype``) times a weight [N, Kdim] for every M >= 1, in the order they are tried."""
    if epilogue not in (None, "swiglu"):
        raise K.KernelError(f"linear: unknown epilogue {epilogue!r}")
    if dtype not in (torch.float32, torch.bfloat16):
        raise K.KernelError(f"linear: dtype {dtype} is not supported")
    if kernels == "generic" or dtype == torch.float32:
        return [Route(ALL_BLOCKS, "generic")]
    tiled_fits = K.gemm_mfma_supported(_MANY_ROWS, N, Kdim)
    many = Route(0, "mfma") if (_prefill_gemm == "mfma" and tiled_fits) else \
        Route(0, "library", fallback="mfma" if tiled_fits else "generic")
    if not K.gemm_skinny_supported(1, N, Kdim):
        return [Route(ALL_BLOCKS, many.kind, many.fallback)] if out_dtype == torch.bfloat16 else [Route(ALL_BLOCKS, "generic")]
    own = "skinny_split" if (keep_split and epilogue is None and K.gemm_skinny_splits(N, Kdim) > 1) else "skinny"
    if out_dtype != torch.bfloat16:
        if epilogue is not None:
            raise K.KernelError("linear: an fp32 result from bf16 operands has no activation here")
        # many rows (the head of a step that wants the logits of many places): the LDS-tiled kernel leaving its fp32
        # sums (one part), which reads the weight once per 128 x 128 tile of the result where the weight-streaming
        # kernel reads all of it for every 128 rows (the head of 128,256 x 4,096 on an MI355X: 371 against 649 us at
        # 256 rows, 2.6 against 4.9 ms at 2,048) and all of X for every 64 rows of the weight (201 against 229 us at
        # 64 rows, 226 against 314 at 128; with K of 2,048 even at 64 rows, 150 against 181 at 128).  The same bits.
        routes = [Route(_UP_TO_128, own), Route(ALL_BLOCKS & ~_UP_TO_128, "skinny_rows")]
        if tiled_fits:
            first = FP32_TILED_FROM_ROWS[0] if Kdim >= 4096 else FP32_TILED_FROM_ROWS[1]
            routes.insert(0, Route(ALL_BLOCKS, "mfma_f32", rows=(first, (2 ** 32 - 1) // (2 * Kdim) - 1)))
        return routes
    to_library = library_rows(N, Kdim, epilogue, keep_split) if _prefill_gemm == "library" else \
        (0 if N < SKINNY_WIDE else 0xFF & ~((1 << (SKINNY_ROWS_ANY_WIDTH // 16)) - 1))
    # the bands of rows of the split tiled kernel stand first: they take their rows from the routes behind them
    routes = [Route(ALL_BLOCKS, "mfma_split", rows=(lo, hi), parts=parts)
              for lo, hi, parts in mid_rows(N, Kdim, keep_split and epilogue is None)]
    if epilogue == "swiglu" and _route == "table" and _prefill_gemm == "library" and tiled_fits:
        routes += [Route(ALL_BLOCKS, "mfma_swiglu", rows=(lo, hi)) for lo, hi in KNOWN_GLU_ROWS.get((N, Kdim), ())]
    routes.append(Route(_UP_TO_128 & ~to_library, own))
    routes.append(Route((ALL_BLOCKS & ~_UP_TO_128) | to_library, many.kind, many.fallback))
    return [r for r in routes if r.blocks]


def route_of(routes: List[Route], M: int) -> Route:
    bit = 1 << min((M - 1) // 16, 8)
    for r in routes:
        if r.blocks & bit and (r.rows is None or r.rows[0] <= M <= r.rows[1]):
            return r
    raise K.KernelError(f"linear: no route for {M} rows")


def _run(kind: str, x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype, epilogue: Optional[str],
         fallback: Optional[str] = None, parts: int = 0):
    M, N = x.shape[0], w.shape[0]
    if kind == "mfma_split":
        return K.gemm_mfma_split(x, w, parts), True
    if kind == "mfma_f32":
        return K.gemm_mfma_split(x, w, 1).parts[0], True
    if kind == "mfma_swiglu":
        return K.gemm_mfma_swiglu(x, w, tiled=tiled_copy(w, "swiglu")), True
    if kind == "skinny":
        return K.gemm_skinny(x, w, epilogue=epilogue, out_dtype=out_dtype, tiled=tiled_copy(w, epilogue)), True
    if kind == "skinny_split":
        return K.gemm_skinny(x, w, keep_split=True, tiled=tiled_copy(w, None)), True
    if kind == "skinny_rows":
        return K.gemm_skinny_rows(x, w, torch.empty((M, N), dtype=out_dtype, device=x.device), tiled_copy(w, None)), True
    if kind == "generic":
        return K.gemm_generic(x, w, torch.empty((M, N), dtype=out_dtype, device=x.device)), False
    if kind == "mfma":
        return K.gemm_mfma(x, w), False
    if kind == "library":
        try:
            return K.gemm_library(x, w), False
        except K.KernelUnsupported:             # the library has no algorithm for this shape
            return _run(fallback or "generic", x, w, out_dtype, None)
    raise K.KernelError(f"linear: unknown route {kind!r}")


def linear(x: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
           epilogue: Optional[str] = None, keep_split: bool = False,
           kernels: str = "auto") -> Union[torch.Tensor, SplitSum]:
    """``kernels="generic"``: the plain product (fp32 multiply-adds in a fixed order) for every size and type."""
    M, Kdim = x.shape
    N = w.shape[0]
    out_dtype = out_dtype or x.dtype
    if M == 0:
        return torch.empty((0, N // 2 if epilogue == "swiglu" else N), dtype=out_dtype, device=x.device)
    if not x.is_contiguous():
        x = x.contiguous()
    route = route_of(plan(N, Kdim, x.dtype, out_dtype, epilogue, keep_split, kernels), M)
    y, activated = _run(route.kind, x, w, out_dtype, epilogue, route.fallback, route.parts)
    if epilogue == "swiglu" and not activated:
        return K.swiglu(y, torch.empty((M, N // 2), dtype=y.dtype, device=y.device))
    return y


# ------------------------------------------------------------------- the same routes, written into a program
def emit_linear(program, x: Any, M: Any, w: torch.Tensor, out_dtype: torch.dtype, epilogue: Optional[str],
                keep_split: bool, out: Any, key: str, when: Any = None):
    """Writes the launches of :func:`linear` for ``x`` (an address: a Buffer, a tensor, a StepPtr) of ``M`` rows
    (a number of the step) into ``program``, one route after the other, each for its rows.  ``out``: a key (the
    result gets a buffer of that name) or a StepPtr (the step's logits); ``key`` names the scratch memory.
    Returns the ``Value`` that stands for the result."""
    from ..engine import program as P
    rt = program.rt
    when = P.ALWAYS if when is None else when
    N, Kdim = w.shape
    T = program.T
    routes = plan(N, Kdim, rt.dtype, out_dtype, epilogue, keep_split, rt.kernels)
    n_out = N // 2 if epilogue == "swiglu" else N
    out_bytes = 4 if out_dtype == torch.float32 else 2
    splits = K.gemm_skinny_splits(N, Kdim) if any(r.kind.startswith("skinny") for r in routes) else 1
    small = min(T, K.SKINNY_MAX_M)
    if isinstance(out, str):
        size = T * n_out * out_bytes
        if any(r.kind == "skinny_split" for r in routes):
            size = max(size, splits * small * N * 4)
        for r in routes:
            if r.kind == "mfma_split":
                size = max(size, r.parts * min(T, r.rows[1]) * N * 4)
        out = program.buffer(out, size)
    code, in_code = K.DTYPE_CODE[out_dtype], K.DTYPE_CODE[rt.dtype]
    tiled = tiled_copy(w, epilogue)
    skinny, wk = ("ia_gemm_skinny_tiled", tiled) if tiled is not None else ("ia_gemm_skinny", w)
    program.keep(w, tiled)
    alts = []
    taken: List[Tuple[int, int]] = []          # the rows that routes with a range of their own have taken

    def not_taken():
        """Holds for the numbers of rows in none of the ranges taken so far: the gaps between them."""
        g, first = P.NEVER, None
        for lo, hi in sorted(taken) + [(None, None)]:
            last = None if lo is None else lo - 1
            if first is None or last is None or first <= last:
                g = g | P.Guard.between(M, first, last)
            first = None if hi is None else (hi + 1 if first is None else max(first, hi + 1))
        return g

    for r in routes:
        g = when & P.Guard.blocks(M, r.blocks) & not_taken()
        if r.rows is not None:
            g = g & P.Guard.between(M, r.rows[0], r.rows[1])
            taken.append(r.rows)
        if g.never:
            continue
        if r.kind == "mfma_split":
            program.op("core", "ia_gemm_mfma_split", [x, w, out, M, N, Kdim, r.parts, P.STREAM], g)
            alts.append(P.Alt(g, out, r.parts, torch.float32))
            continue
        if r.kind == "mfma_swiglu":
            program.op("core", "ia_gemm_mfma_swiglu", [x, wk, int(tiled is not None), out, M, N, Kdim, P.STREAM], g)
            alts.append(P.Alt(g, out, 0, out_dtype))
            continue
        if r.kind == "mfma_f32":                # one part: the fp32 matrix itself
            program.op("core", "ia_gemm_mfma_split", [x, w, out, M, N, Kdim, 1, P.STREAM], g)
            alts.append(P.Alt(g, out, 0, out_dtype))
            continue
        if r.kind == "skinny_split":
            program.op("core", skinny, [x, wk, None, 0, M, N, Kdim, 0, out, M * (splits * N), P.STREAM], g)
            alts.append(P.Alt(g, out, splits, torch.float32))
            continue
        if r.kind == "skinny":
            ws = program.buffer(key + ".parts", splits * small * N * 4) if splits > 1 else None
            program.op("core", skinny, [x, wk, out, code, M, N, Kdim, K.EPILOGUE[epilogue], ws,
                                        M * (splits * N) if splits > 1 else 0, P.STREAM], g)
        elif r.kind == "skinny_rows":
            ws = program.buffer(key + ".parts", splits * small * N * 4) if splits > 1 else None
            program.op("core", "ia_gemm_skinny_rows", [x, wk, int(tiled is not None), out, code, M, N, Kdim, ws,
                                                        splits * small * N if splits > 1 else 0, P.STREAM], g)
        else:
            # a product that leaves the whole matrix: into scratch first when an activation follows
            y = program.buffer(key + ".product", T * N * out_bytes) if epilogue == "swiglu" else out
            _emit_whole(program, r.kind, x, w, y, M, N, Kdim, in_code, code, g, False)
            if r.fallback:
                _emit_whole(program, r.fallback, x, w, y, M, N, Kdim, in_code, code, g, True)
            if epilogue == "swiglu":
                program.op("core", "ia_swiglu", [y, out, code, M, N // 2, P.STREAM], g)
        alts.append(P.Alt(g, out, 0, out_dtype))
    return P.Value(n_out, alts)


def _emit_whole(program, kind, x, w, y, M, N, Kdim, in_code, out_code, when, if_unsupported) -> None:
    from ..engine import program as P
    if kind == "generic":
        program.op("core", "ia_gemm_generic", [x, w, y, in_code, out_code, M, N, Kdim, Kdim, Kdim, N, P.STREAM],
                   when, if_unsupported)
    elif kind == "mfma":
        program.op("core", "ia_gemm_mfma", [x, w, y, M, N, Kdim, 0, P.STREAM], when, if_unsupported)
    elif kind == "library":
        ws = K.library_workspace(program.rt.device)
        program.op("blaslt", "ia_gemm_lt", [x, w, y, M, N, Kdim, in_code, ws, ws.numel(), P.STREAM], when, if_unsupported)
    else:
        raise K.KernelError(f"linear: {kind!r} does not leave a whole matrix")
