"""Python face of the HIP kernels: shape checks on the host, then one C call.

Every function checks that its operands are what the kernel and its grid assume
(device, dtype, contiguity, sizes) before anything is launched, and launches on
torch's current stream, so that calls order with torch's own work and can be
captured into a HIP graph.  There is no fallback: without a GPU or without the
built library a call raises :class:`KernelError`.
"""
from __future__ import annotations

import atexit
import ctypes
import functools
import math
import os
import sys
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from ..csrc import build as _build


class KernelError(RuntimeError):
    pass


class KernelUnsupported(KernelError):
    """The kernel (or the library) does not take this size; nothing was launched."""


DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1}
_libs: Dict[str, ctypes.CDLL] = {}

_ERRORS = {10001: "bad argument", 10002: "size not supported by this kernel",
           10003: "a call into the GEMM library failed"}


# Into how many parts the weight-streaming product splits the inner dimension of a weight [N, K], where that was
# measured and differs from the rule of sizes (about 512 workgroups): the 13B, 70B and 1B shapes' products on an
# MI355X, with cold weights and the norm that joins the parts behind them, at 1, 8 and 64 rows (13B down projection:
# 35.0 us in six even parts of nine chunks, 42.3 in the rule's seven; 70B QKV: 35.4 us in three parts, 43.5 in four).
# The sums of a product are taken in the order that its number of parts gives: a shape's entry is part of its
# arithmetic, the same in every process.
KNOWN_SPLITS = {
    (15360, 5120): 2, (5120, 5120): 5, (5120, 13824): 6,       # Llama-2-13B: QKV, output and down projection
    (10240, 8192): 3,                                          # Llama-3.1-70B: QKV
    (2048, 8192): 8,                                           # Llama-3.2-1B: down projection
}


def load_library(name: str) -> ctypes.CDLL:
    lib = _libs.get(name)
    if lib is None:
        if not torch.cuda.is_available():
            raise KernelError("no GPU is visible: infernum_amd runs on a gfx950 GPU only (there is no CPU fallback)")
        try:
            path = _build.ensure(name)
            lib = ctypes.CDLL(path)
        except (OSError, _build.BuildError) as e:
            raise KernelError(f"the HIP kernel library '{name}' could not be built or loaded: {e}") from e
        if name == "core":
            for (N, K), parts in KNOWN_SPLITS.items():
                _ok(lib.ia_gemm_skinny_set_splits(N, K, parts), "gemm_skinny_set_splits")
        _libs[name] = lib
    return lib


def _core() -> ctypes.CDLL:
    return load_library("core")


def _p(t: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return ctypes.c_void_p(t.data_ptr() if t is not None else 0)


_fixed_stream: Optional[ctypes.c_void_p] = None


def _stream() -> ctypes.c_void_p:
    if _fixed_stream is not None:
        return _fixed_stream
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


class on_current_stream:
    """Within this block every kernel call launches on the stream that is current at its entry, looked up
    once (the lookup costs as much as several launches).  Enter it anew inside a graph capture: the capture
    has a stream of its own."""

    def __enter__(self):
        global _fixed_stream
        if not torch.cuda.is_available():
            raise KernelError("no GPU is visible: infernum_amd runs on a gfx950 GPU only (there is no CPU fallback)")
        self._before = _fixed_stream
        _fixed_stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        return self

    def __exit__(self, *exc):
        global _fixed_stream
        _fixed_stream = self._before
        return False


def _ok(code: int, what: str) -> None:
    if code != 0:
        why = _ERRORS.get(code, f"HIP error {code}")
        raise (KernelUnsupported if code == 10002 else KernelError)(f"{what}: {why}")


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _dev(*ts: Optional[torch.Tensor]) -> None:
    for t in ts:
        if t is not None:
            _need(t.is_cuda, "operand is not on the GPU")
            _need(t.is_contiguous(), "operand is not contiguous")


def _i32(t: torch.Tensor, n: int, what: str) -> None:
    _need(t.dtype == torch.int32 and t.is_cuda and t.is_contiguous() and t.numel() >= n,
          f"{what}: needs a contiguous int32 GPU tensor of at least {n} elements")


# --------------------------------------------------------------------------- rows
def embed(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[n, :] = float(table[ids[n], :]); out is fp32 [N, H]."""
    _dev(table, ids, out)
    V, H = table.shape
    N = ids.numel()
    _need(table.dtype in DTYPE_CODE, f"embed: table dtype {table.dtype}")
    _i32(ids, N, "embed ids")
    _need(out.dtype == torch.float32 and tuple(out.shape) == (N, H), f"embed: out must be fp32 [{N}, {H}]")
    _ok(_core().ia_embed(_p(table), DTYPE_CODE[table.dtype], _p(ids), _p(out), N, H, V, _stream()), "embed")
    return out


class SplitSum:
    """A matrix [M, N] given as a stack of fp32 partial sums ``parts`` [S, M, N]: what a matrix product
    whose inner dimension was split over workgroups leaves.  The kernels that take the product next
    (residual add + norm, rotary + cache write) add the parts themselves, in the order of their index."""

    __slots__ = ("parts",)

    def __init__(self, parts: torch.Tensor):
        if parts.dim() != 3 or parts.dtype != torch.float32 or not parts.is_contiguous():
            raise KernelError("SplitSum: parts must be a contiguous fp32 [S, M, N] tensor")
        self.parts = parts

    @property
    def shape(self):
        return self.parts.shape[1:]

    def joined(self, dtype: torch.dtype) -> torch.Tensor:
        """The sum as one tensor (a library reduction; for paths that are not hot)."""
        return self.parts.sum(dim=0).to(dtype)


def add_rmsnorm(h: torch.Tensor, delta, weight: torch.Tensor, eps: float,
                out: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """h += delta (fp32, in place); out = h * rsqrt(mean(h^2) + eps) * weight.

    ``delta`` is None, a tensor of h's shape in out's dtype, or a :class:`SplitSum`.
    With ``rows`` the norm is taken of the selected rows only and h stays as it is.
    """
    split = isinstance(delta, SplitSum)
    d = delta.parts if split else delta
    _dev(h, d, weight, out, rows)
    _need(h.dtype == torch.float32 and h.dim() == 2, "add_rmsnorm: h must be fp32 [N, H]")
    H = h.shape[1]
    n_out = rows.numel() if rows is not None else h.shape[0]
    _need(out.dtype in DTYPE_CODE and tuple(out.shape) == (n_out, H), f"add_rmsnorm: out must be [{n_out}, {H}]")
    splits, d_rows, d_code = 1, h.shape[0], DTYPE_CODE[out.dtype]
    if split:
        _need(tuple(d.shape[1:]) == tuple(h.shape), "add_rmsnorm: partial sums must be [S, N, H]")
        splits, d_code = d.shape[0], DTYPE_CODE[torch.float32]
    elif d is not None:
        _need(d.dtype == out.dtype and tuple(d.shape) == tuple(h.shape),
              "add_rmsnorm: delta must have h's shape and out's dtype")
    _need(weight.dtype in DTYPE_CODE and weight.numel() == H, f"add_rmsnorm: weight must hold {H} values")
    if rows is not None:
        _i32(rows, n_out, "add_rmsnorm rows")
    _ok(_core().ia_add_rmsnorm(_p(h), _p(d), d_code, splits, d_rows, DTYPE_CODE[out.dtype], _p(weight),
                               DTYPE_CODE[weight.dtype], _p(out), _p(rows), n_out, H, ctypes.c_float(eps),
                               _stream()), "add_rmsnorm")
    return out


def residual_add(h: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
    _dev(h, delta)
    _need(h.dtype == torch.float32 and h.dim() == 2 and tuple(delta.shape) == tuple(h.shape)
          and delta.dtype in DTYPE_CODE, "residual_add: h fp32 [N, H], delta of the same shape")
    _ok(_core().ia_residual_add(_p(h), _p(delta), DTYPE_CODE[delta.dtype], h.shape[0], h.shape[1], _stream()),
        "residual_add")
    return h


def rope_kv_append(qkv, positions: torch.Tensor, inv_freq: Optional[torch.Tensor], nh: int, nkv: int,
                   d: int, rot: int, slots: Optional[torch.Tensor] = None, k_pages: Optional[torch.Tensor] = None,
                   v_pages: Optional[torch.Tensor] = None, q_out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Rotate q and k, and write k and v to their page slots.  Returns the rotated q, [N, >= nh d].

    qkv is [N, (nh + 2 nkv) d] (or [N, nh d] when no pages are given), a tensor or a :class:`SplitSum`.
    A tensor is rotated in place unless ``q_out`` is given; a SplitSum needs ``q_out`` [N, nh d] (made here
    when absent).  Key pages are [num_pages, nkv, page_size, d], value pages [num_pages, nkv, d, page_size].
    """
    split = isinstance(qkv, SplitSum)
    src = qkv.parts if split else qkv
    write = k_pages is not None
    N, row = (src.shape[1], src.shape[2]) if split else tuple(src.shape)
    act = (k_pages.dtype if write else (q_out.dtype if q_out is not None else None)) if split else src.dtype
    _need(act is not None, "rope: partial sums need pages or q_out to tell the activations' dtype")
    if q_out is None:
        q_out = torch.empty((N, nh * d), dtype=act, device=src.device) if split else src
    _dev(src, positions, inv_freq, slots, k_pages, v_pages)
    _need(q_out.is_cuda and q_out.dim() == 2 and q_out.stride(1) == 1 and q_out.shape[0] == N
          and q_out.shape[1] >= nh * d and q_out.dtype == act, "rope: q_out must be [N, >= nh*d] in the activations' dtype")
    _need(act in DTYPE_CODE and src.dtype in DTYPE_CODE, "rope: dtype")
    _need(row >= (nh + (2 * nkv if write else 0)) * d, "rope: row of qkv is too short for its heads")
    _i32(positions, N, "rope positions")
    if inv_freq is not None:
        _need(inv_freq.dtype in (torch.float32, torch.float64) and inv_freq.numel() == rot // 2 and rot % 2 == 0
              and 0 < rot <= d, "rope: inv_freq must hold rot/2 fp32 or float64 values, rot even and at most the head size")
    page_size = num_pages = 0
    if write:
        _need(v_pages is not None and slots is not None, "rope: k_pages, v_pages and slots go together")
        _need(k_pages.dtype == act and v_pages.dtype == act, "rope: pages must have the activations' dtype")
        num_pages, page_size = k_pages.shape[0], k_pages.shape[2]
        _need(k_pages.dim() == 4 and k_pages.shape[1] == nkv and k_pages.shape[3] == d
              and tuple(v_pages.shape) == (num_pages, nkv, d, page_size),
              "rope: key pages must be [num_pages, nkv, page_size, d], value pages [num_pages, nkv, d, page_size]")
        _i32(slots, N, "rope slots")
    _ok(_core().ia_rope_kv_append(_p(src), DTYPE_CODE[src.dtype], src.shape[0] if split else 1, N, _p(q_out),
                                  q_out.stride(0), DTYPE_CODE[act], _p(positions), _p(slots), _p(inv_freq),
                                  1 if (inv_freq is not None and inv_freq.dtype == torch.float64) else 0,
                                  _p(k_pages), _p(v_pages), N, row, nh, nkv, d, rot if inv_freq is not None else 0,
                                  page_size, num_pages, 1 if write else 0, _stream()), "rope_kv_append")
    return q_out


def swiglu(gate_up: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[n, i] = silu(gate_up[n, i]) * gate_up[n, I + i]."""
    _dev(gate_up, out)
    N, two_i = gate_up.shape
    _need(two_i % 2 == 0 and tuple(out.shape) == (N, two_i // 2) and out.dtype == gate_up.dtype
          and out.dtype in DTYPE_CODE, "swiglu: gate_up [N, 2I] and out [N, I] of one dtype")
    _ok(_core().ia_swiglu(_p(gate_up), _p(out), DTYPE_CODE[out.dtype], N, two_i // 2, _stream()), "swiglu")
    return out


def cast(src: torch.Tensor, dtype: torch.dtype, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``src`` in another of the two types (fp32 to bf16 rounds to nearest even; bf16 to fp32 is exact)."""
    _dev(src, out)
    _need(src.dtype in DTYPE_CODE and dtype in DTYPE_CODE, "cast: fp32 and bf16 only")
    if out is None:
        out = torch.empty(src.shape, dtype=dtype, device=src.device)
    _need(out.dtype == dtype and out.numel() == src.numel(), "cast: out must have src's size and the asked type")
    _ok(_core().ia_cast(_p(src), DTYPE_CODE[src.dtype], _p(out), DTYPE_CODE[dtype], ctypes.c_size_t(src.numel()),
                        _stream()), "cast")
    return out


def gather_tokens(token_ids: torch.Tensor, source: torch.Tensor, index: torch.Tensor) -> None:
    """token_ids[i] = source[index[i]] where index[i] >= 0; other places stay.  All int32 on the device."""
    _dev(token_ids, source, index)
    n = token_ids.numel()
    _i32(token_ids, n, "gather_tokens token_ids")
    _i32(index, n, "gather_tokens index")
    _i32(source, 0, "gather_tokens source")
    _ok(_core().ia_gather_tokens(_p(token_ids), _p(source), _p(index), n, source.numel(), _stream()), "gather_tokens")


def words_from_host(dst: torch.Tensor, pinned: torch.Tensor, n: int, token_off: int = 0, nd: int = 0,
                    source: Optional[torch.Tensor] = None, index_off: int = 0) -> None:
    """dst[:n] = pinned[:n] (4-byte words; ``pinned`` in pinned host memory) by a kernel of the current stream;
    with ``nd`` > 0 the words dst[token_off + r], r < nd, whose index pinned[index_off + r] is j >= 0 become
    source[j] (int32 on the device)."""
    _need(dst.is_cuda and dst.is_contiguous() and dst.element_size() == 4 and dst.numel() >= n,
          "words_from_host: a contiguous device tensor of 4-byte elements, at least n long")
    _need(pinned.is_pinned() and pinned.element_size() == 4 and pinned.numel() >= max(n, index_off + nd),
          "words_from_host: the source must be pinned host memory of 4-byte elements, long enough")
    if nd:
        _i32(source, 0, "words_from_host tokens")
    _ok(_core().ia_words_from_host(_p(dst), ctypes.c_void_p(pinned.data_ptr()), int(n), int(token_off), int(nd),
                                   _p(source), source.numel() if source is not None else 0, int(index_off), _stream()),
        "words_from_host")


def words_to_host(pinned: torch.Tensor, src: torch.Tensor) -> None:
    """pinned[:n] = src (4-byte words) by a kernel of the current stream; an event recorded after it tells the
    host when the words are there."""
    n = src.numel()
    _need(src.is_cuda and src.is_contiguous() and src.element_size() == 4, "words_to_host: a device tensor of 4-byte elements")
    _need(pinned.is_pinned() and pinned.element_size() == 4 and pinned.numel() >= n,
          "words_to_host: the target must be pinned host memory of 4-byte elements, long enough")
    _ok(_core().ia_words_to_host(ctypes.c_void_p(pinned.data_ptr()), _p(src), n, _stream()), "words_to_host")


def copy_pages(pool: torch.Tensor, src_pages: torch.Tensor, dst_pages: torch.Tensor) -> None:
    """pool[dst_pages[i]] = pool[src_pages[i]] for a pool [num_pages, ...]; pairs with a page outside the pool
    are left out.  The targets must differ from each other and from every source."""
    _dev(pool, src_pages, dst_pages)
    n = src_pages.numel()
    _need(pool.dim() >= 2 and pool.shape[0] > 0, "copy_pages: a pool [num_pages, ...]")
    _i32(src_pages, n, "copy_pages sources")
    _i32(dst_pages, n, "copy_pages targets")
    page_bytes = pool[0].numel() * pool.element_size()
    _need(page_bytes % 4 == 0 and n <= 65535, "copy_pages: pages of a multiple of 4 bytes, at most 65,535 pairs")
    _ok(_core().ia_copy_pages(_p(pool), ctypes.c_size_t(page_bytes), pool.shape[0], _p(src_pages), _p(dst_pages), n,
                              _stream()), "copy_pages")


# ------------------------------------------------------------------ matrix products
def gemm_generic(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[M, N] = a[M, K] @ w[N, K]^T with fp32 multiply-adds in the order of k."""
    _dev(w, out)
    _need(a.is_cuda and a.dim() == 2 and a.stride(1) == 1, "gemm: a must be a GPU matrix with unit inner stride")
    M, K = a.shape
    N = w.shape[0]
    _need(w.dim() == 2 and w.shape[1] == K, f"gemm: weight must be [N, {K}], got {tuple(w.shape)}")
    _need(a.dtype == w.dtype and a.dtype in DTYPE_CODE and out.dtype in DTYPE_CODE, "gemm: dtypes")
    _need(tuple(out.shape) == (M, N), f"gemm: out must be [{M}, {N}]")
    lda = a.stride(0) if M > 1 else K
    _need(lda >= K, "gemm: a's rows overlap")
    _ok(_core().ia_gemm_generic(_p(a), _p(w), _p(out), DTYPE_CODE[a.dtype], DTYPE_CODE[out.dtype], M, N, K, lda, K, N,
                                _stream()), "gemm_generic")
    return out


MFMA_GEMM_TILES = {"auto": 0, "256x256": 1, "128x256": 2, "128x128": 3}


def gemm_mfma_supported(M: int, N: int, K: int) -> bool:
    """Sizes the LDS-tiled MFMA product takes: K in steps of 64, rows addressed with 32-bit byte offsets."""
    return M >= 1 and N >= 1 and K >= 64 and K % 64 == 0 and M * K * 2 < 2 ** 32 and N * K * 2 < 2 ** 32


def gemm_mfma(a: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None, tile: str = "auto") -> torch.Tensor:
    """out[M, N] = a[M, K] @ w[N, K]^T, bf16 with fp32 accumulation, for many rows (prefill): both operands
    tiled through LDS, ``v_mfma_f32_32x32x16_bf16``.  A row of the result depends on its own row of ``a`` only."""
    _dev(a, w, out)
    _need(a.dim() == 2 and w.dim() == 2 and a.shape[1] == w.shape[1], "gemm_mfma: shapes")
    M, K = a.shape
    N = w.shape[0]
    _need(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_mfma: bf16 operands")
    _need(a.is_contiguous() and w.is_contiguous(), "gemm_mfma: contiguous operands")
    _need(gemm_mfma_supported(M, N, K), f"gemm_mfma: M={M} N={N} K={K} not supported (K % 64 == 0, below 4 GiB)")
    _need(tile in MFMA_GEMM_TILES, f"gemm_mfma: unknown tile {tile!r}")
    if out is None:
        out = torch.empty((M, N), dtype=torch.bfloat16, device=a.device)
    _need(out.dtype == torch.bfloat16 and out.is_contiguous() and tuple(out.shape) == (M, N),
          f"gemm_mfma: out must be contiguous bf16 [{M}, {N}]")
    _ok(_core().ia_gemm_mfma(_p(a), _p(w), _p(out), M, N, K, MFMA_GEMM_TILES[tile], _stream()), "gemm_mfma")
    return out


def gemm_mfma_swiglu(a: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None,
                     tiled: Optional[torch.Tensor] = None) -> torch.Tensor:
    """silu(a @ w[:N/2]^T) * (a @ w[N/2:]^T) as bf16 [M, N/2]: the LDS-tiled MFMA product (tiles of 128 x 128) with
    the activation on its fp32 sums in the epilogue, for up to some hundred rows.  ``tiled``: the copy of ``w`` that
    :func:`tile_weight` made with the "swiglu" epilogue, read instead of ``w`` (the same bits)."""
    _dev(a, w, out, tiled)
    _need(a.dim() == 2 and w.dim() == 2 and a.shape[1] == w.shape[1], "gemm_mfma_swiglu: shapes")
    M, K = a.shape
    N = w.shape[0]
    _need(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_mfma_swiglu: bf16 operands")
    _need(a.is_contiguous() and w.is_contiguous(), "gemm_mfma_swiglu: contiguous operands")
    _need(N % 2 == 0 and gemm_mfma_supported(M, N, K),
          f"gemm_mfma_swiglu: M={M} N={N} K={K} not supported (N even, K % 64 == 0, below 4 GiB)")
    if out is None:
        out = torch.empty((M, N // 2), dtype=torch.bfloat16, device=a.device)
    _need(out.dtype == torch.bfloat16 and out.is_contiguous() and tuple(out.shape) == (M, N // 2),
          f"gemm_mfma_swiglu: out must be contiguous bf16 [{M}, {N // 2}]")
    if tiled is not None:
        _core().ia_gemm_skinny_tiled_elements.restype = ctypes.c_size_t
        _need(tiled.dtype == torch.bfloat16 and tiled.is_contiguous() and gemm_skinny_splits(N, K) == 1 and
              tiled.numel() == int(_core().ia_gemm_skinny_tiled_elements(N, K, EPILOGUE["swiglu"])),
              "gemm_mfma_swiglu: tiled is not the copy, made for the swiglu epilogue, of a weight that is not split over K")
    _ok(_core().ia_gemm_mfma_swiglu(_p(a), _p(tiled if tiled is not None else w), int(tiled is not None), _p(out),
                                    M, N, K, _stream()), "gemm_mfma_swiglu")
    return out


def gemm_mfma_split(a: torch.Tensor, w: torch.Tensor, splits: int, parts: Optional[torch.Tensor] = None) -> SplitSum:
    """a[M, K] @ w[N, K]^T for a few hundred rows as fp32 partial sums [splits, M, N]: the LDS-tiled MFMA product
    with tiles of 128 x 128 and K split over ``splits`` workgroups a tile, so that the launch fills the GPU where the
    tiles alone would not and the weight comes at the memory's rate; the next kernel adds the parts."""
    _dev(a, w, parts)
    _need(a.dim() == 2 and w.dim() == 2 and a.shape[1] == w.shape[1], "gemm_mfma_split: shapes")
    M, K = a.shape
    N = w.shape[0]
    _need(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_mfma_split: bf16 operands")
    _need(a.is_contiguous() and w.is_contiguous(), "gemm_mfma_split: contiguous operands")
    _need(gemm_mfma_supported(M, N, K), f"gemm_mfma_split: M={M} N={N} K={K} not supported (K % 64 == 0, below 4 GiB)")
    _need(1 <= splits <= K // 64, f"gemm_mfma_split: {splits} parts of K={K} (1 to K / 64)")
    if parts is None:
        parts = torch.empty((splits, M, N), dtype=torch.float32, device=a.device)
    _need(parts.dtype == torch.float32 and parts.is_contiguous() and tuple(parts.shape) == (splits, M, N),
          f"gemm_mfma_split: parts must be contiguous fp32 [{splits}, {M}, {N}]")
    _ok(_core().ia_gemm_mfma_split(_p(a), _p(w), _p(parts), M, N, K, splits, _stream()), "gemm_mfma_split")
    return SplitSum(parts)


LIBRARY_WORKSPACE_BYTES = 128 << 20
_library_workspace: Dict[torch.device, torch.Tensor] = {}


def library_workspace(device: torch.device) -> torch.Tensor:
    """The one workspace of the library's products on a device."""
    ws = _library_workspace.get(device)
    if ws is None:
        ws = _library_workspace[device] = torch.empty(LIBRARY_WORKSPACE_BYTES, dtype=torch.uint8, device=device)
    return ws


def gemm_library(a: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[M, N] = a[M, K] @ w[N, K]^T by the vendor's library (hipBLASLt), called directly: bf16 with fp32
    accumulation, or fp32 throughout.  The library's choice of an algorithm is asked once per shape and kept,
    so a later product of the same shape costs one call on the host.  All products share one workspace per
    device: they must be on one stream, or ordered otherwise."""
    _dev(a, w, out)
    _need(a.dim() == 2 and w.dim() == 2 and a.shape[1] == w.shape[1], "gemm_library: shapes")
    M, K = a.shape
    N = w.shape[0]
    _need(a.dtype == w.dtype and a.dtype in DTYPE_CODE, "gemm_library: bf16 or fp32 operands of one dtype")
    _need(M >= 1 and N >= 1 and K >= 1, "gemm_library: empty operand")
    if out is None:
        out = torch.empty((M, N), dtype=a.dtype, device=a.device)
    _need(out.dtype == a.dtype and tuple(out.shape) == (M, N), f"gemm_library: out must be {a.dtype} [{M}, {N}]")
    ws = library_workspace(a.device)
    lib = load_library("blaslt")
    code = lib.ia_gemm_lt(_p(a), _p(w), _p(out), M, N, K, DTYPE_CODE[a.dtype], _p(ws), ctypes.c_size_t(ws.numel()),
                          _stream())
    if code == 10003:
        raise KernelError(f"gemm_library: hipBLASLt failed with status {lib.ia_gemm_lt_last_status()} "
                          f"(M={M} N={N} K={K} {a.dtype})")
    _ok(code, f"gemm_library (M={M} N={N} K={K})")
    return out


SKINNY_MAX_M = 128
EPILOGUE = {None: 0, "swiglu": 1}


def gemm_skinny_supported(M: int, N: int, K: int) -> bool:
    return 0 < M <= SKINNY_MAX_M and K % 8 == 0 and K >= 8 and N >= 1


def gemm_skinny_splits(N: int, K: int) -> int:
    """Parts the inner dimension is split into for a weight [N, K] (depends on N and K only)."""
    return int(_core().ia_gemm_skinny_splits(N, K))


def tile_weight(w: torch.Tensor, epilogue: Optional[str] = None) -> torch.Tensor:
    """A copy of the weight [N, K] (bf16) laid out for :func:`gemm_skinny` with this epilogue: the 64 rows x 256
    values that a workgroup multiplies with in one chunk are 32 KB of consecutive memory, chunk after chunk, so
    every workgroup reads one stretch of memory front to back (rows padded to whole workgroups, K to whole chunks,
    with zeros).  Pass it as ``tiled``; the result has the same bits."""
    _dev(w)
    _need(w.dim() == 2 and w.dtype == torch.bfloat16 and epilogue in EPILOGUE, "tile_weight: a bf16 matrix [N, K]")
    N, K = w.shape
    lib = _core()
    lib.ia_gemm_skinny_tiled_elements.restype = ctypes.c_size_t
    n = int(lib.ia_gemm_skinny_tiled_elements(N, K, EPILOGUE[epilogue]))
    out = torch.empty(n, dtype=torch.bfloat16, device=w.device)
    _ok(lib.ia_gemm_skinny_tile(_p(w), _p(out), N, K, EPILOGUE[epilogue], _stream()), "tile_weight")
    return out


def gemm_skinny(a: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None,
                epilogue: Optional[str] = None, keep_split: bool = False,
                out_dtype: torch.dtype = torch.bfloat16, tiled: Optional[torch.Tensor] = None):
    """a[M, K] @ w[N, K]^T for M <= 64 on MFMA, weights streamed once; bf16 operands, fp32 sums.

    Returns ``out`` ([M, N] bf16 or fp32; [M, N/2] with the "swiglu" epilogue, silu(left half) * right half),
    or, with ``keep_split`` and a product that is split, a :class:`SplitSum` for the next kernel to join.
    """
    _dev(a, w, out)
    M, K = a.shape
    N = w.shape[0]
    _need(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_skinny: bf16 operands")
    _need(w.dim() == 2 and w.shape[1] == K, "gemm_skinny: shapes")
    _need(gemm_skinny_supported(M, N, K), f"gemm_skinny: M={M} N={N} K={K} not supported (M <= 128, K % 8 == 0)")
    _need(epilogue in EPILOGUE, f"gemm_skinny: unknown epilogue {epilogue!r}")
    _need(epilogue is None or N % 2 == 0, "gemm_skinny: the swiglu epilogue needs an even N")
    splits = gemm_skinny_splits(N, K)
    ws = None
    if splits > 1:
        ws = torch.empty((splits, M, N), dtype=torch.float32, device=a.device)
    launch, wp = _core().ia_gemm_skinny, _p(w)
    if tiled is not None:
        _need(tiled.is_cuda and tiled.dtype == torch.bfloat16 and tiled.is_contiguous(), "gemm_skinny: the tiled copy")
        launch, wp = _core().ia_gemm_skinny_tiled, _p(tiled)
    if keep_split and epilogue is None and splits > 1:
        _ok(launch(_p(a), wp, None, 0, M, N, K, 0, _p(ws), ctypes.c_size_t(ws.numel()), _stream()), "gemm_skinny")
        return SplitSum(ws)
    n_out = N // 2 if epilogue == "swiglu" else N
    if out is None:
        out = torch.empty((M, n_out), dtype=out_dtype, device=a.device)
    _need(out.dtype in DTYPE_CODE and tuple(out.shape) == (M, n_out) and out.is_contiguous(),
          f"gemm_skinny: out must be contiguous [{M}, {n_out}]")
    _ok(launch(_p(a), wp, _p(out), DTYPE_CODE[out.dtype], M, N, K, EPILOGUE[epilogue], _p(ws),
               ctypes.c_size_t(ws.numel() if ws is not None else 0), _stream()), "gemm_skinny")
    return out


def gemm_skinny_rows(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, tiled: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[M, N] = a[M, K] @ w[N, K]^T for any M through :func:`gemm_skinny`'s kernel, 128 rows at a time (an fp32
    result from bf16 operands has no other kernel: the head of a step that wants the logits of many places)."""
    _dev(a, w, out)
    M, K = a.shape
    N = w.shape[0]
    _need(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and w.dim() == 2 and w.shape[1] == K,
          "gemm_skinny_rows: bf16 operands [M, K] and [N, K]")
    _need(M >= 1 and gemm_skinny_supported(1, N, K), f"gemm_skinny_rows: M={M} N={N} K={K} not supported (K % 8 == 0)")
    _need(out.dtype in DTYPE_CODE and tuple(out.shape) == (M, N), f"gemm_skinny_rows: out must be contiguous [{M}, {N}]")
    splits = gemm_skinny_splits(N, K)
    ws = torch.empty((splits, min(M, SKINNY_MAX_M), N), dtype=torch.float32, device=a.device) if splits > 1 else None
    _ok(_core().ia_gemm_skinny_rows(_p(a), _p(tiled if tiled is not None else w), int(tiled is not None), _p(out),
                                    DTYPE_CODE[out.dtype], M, N, K, _p(ws),
                                    ctypes.c_size_t(ws.numel() if ws is not None else 0), _stream()), "gemm_skinny_rows")
    return out


# ------------------------------------------------------------------------ attention
def _check_paged(qkv, k_pages, v_pages, out, block_tables, nh, nkv, d, what):
    _dev(qkv, k_pages, v_pages, out, block_tables)
    _need(qkv.dtype == out.dtype == k_pages.dtype == v_pages.dtype and qkv.dtype in DTYPE_CODE,
          f"{what}: q, pages and out must share one dtype")
    _need(qkv.dim() == 2 and qkv.shape[1] >= nh * d, f"{what}: q rows must hold nh*d values")
    _need(out.dim() == 2 and out.shape[1] == nh * d and out.shape[0] == qkv.shape[0],
          f"{what}: out must be [N, nh*d]")
    _need(k_pages.dim() == 4 and k_pages.shape[1] == nkv and k_pages.shape[3] == d
          and tuple(v_pages.shape) == (k_pages.shape[0], nkv, d, k_pages.shape[2]),
          f"{what}: key pages must be [num_pages, nkv, page_size, d], value pages [num_pages, nkv, d, page_size]")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2, f"{what}: block_tables int32 [B, MB]")
    _need(nh % nkv == 0, f"{what}: nh must be a multiple of nkv")


def attention_generic(qkv: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, out: torch.Tensor,
                      token_seq: torch.Tensor, positions: torch.Tensor, block_tables: torch.Tensor, nh: int,
                      nkv: int, d: int, scale: float, window: int = 0) -> None:
    """Causal paged attention, one wave per (token, head), fp32 arithmetic.

    qkv [N, >= nh*d]: the q heads of token n are the first nh*d values of row n.
    token_seq[n] is the row of block_tables of token n; positions[n] its position.
    """
    _check_paged(qkv, k_pages, v_pages, out, block_tables, nh, nkv, d, "attention")
    N = out.shape[0]
    _i32(token_seq, N, "attention token_seq")
    _i32(positions, N, "attention positions")
    _need(0 < d <= 256, "attention: head size must be at most 256")
    _ok(_core().ia_attention_generic(_p(qkv), qkv.shape[1], _p(k_pages), _p(v_pages), _p(out), nh * d,
                                     DTYPE_CODE[out.dtype], _p(token_seq), _p(positions), _p(block_tables),
                                     block_tables.shape[1], N, nh, nkv, d, k_pages.shape[2], k_pages.shape[0],
                                     ctypes.c_float(scale), int(window), _stream()), "attention_generic")


def _attn(d: int) -> ctypes.CDLL:
    lib = load_library(f"attn_d{d}")
    return lib


_compute_units: Dict[int, int] = {}


def compute_units(device: Optional[torch.device] = None) -> int:
    """Compute units of the device (asked once): what the launch shapes below are sized against."""
    idx = device.index if (device is not None and device.index is not None) else torch.cuda.current_device()
    cus = _compute_units.get(idx)
    if cus is None:
        cus = _compute_units[idx] = int(torch.cuda.get_device_properties(idx).multi_processor_count)
    return cus


def decode_splits(batch: int, nh: int, nkv: int, max_len: int, device: Optional[torch.device] = None,
                  head_dim: int = 128) -> int:
    """Parts the keys of a request are cut into, so that a small batch still fills the GPU (workgroups of
    four waves, each wave one tile of 16 keys at a time).  Measured on 256 compute units, with the join's launch:

    * head sizes up to 128: about one workgroup a compute unit while the batch alone gives at most a quarter of
      that, about two up to five eighths, and no parts above that (8B shape, 527 keys: 24 requests 13.9 us whole
      against 15.3 in three parts, 32 requests 15.4 against 17.1 in two); at head sizes up to 64 a tile is half the
      bytes and twice as many workgroups are wanted (8 requests with 32,768 keys each: 97 us in eight parts, 138
      in four; 32 requests: 364 in two, 520 whole);
    * above 128 a compute unit holds one workgroup, and more parts than compute units only cost (head size 256, 32
      requests on 4 key/value heads: 19 us in two parts, 23 in four);
    * the join grows with the parts as the work of a part shrinks with them: the best number of parts for one
      request went with the square root of its tiles (4 parts at 512 keys, 8 at 2,048, 16 at 8,192, 32 at 32,768, for
      head sizes 64, 128 and 256 alike), so that bounds the parts; never more than 64."""
    cus = compute_units(device)
    fill = cus * (2 if head_dim <= 64 else 1)
    groups = batch * nkv * ((nh // nkv + 15) // 16)
    tiles = max(1, (max_len + 15) // 16)
    if 8 * groups >= 5 * fill:
        return 1
    if head_dim > 128:
        wanted = fill // groups
    else:
        wanted = fill // groups if 4 * groups <= fill else 2 * fill // groups
    return max(1, min(wanted, math.isqrt(tiles // 2), 64))


def attention_decode(qkv: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, out: torch.Tensor,
                     positions: torch.Tensor, block_tables: torch.Tensor, nh: int, nkv: int, d: int, scale: float,
                     window: int, max_len: int, num_splits: Optional[int] = None) -> None:
    """bf16 attention of B single tokens (row b of qkv: token b at positions[b]) over their pages, on MFMA.

    ``max_len`` bounds the positions (host side), and sets how many parts the keys are split into.
    """
    _check_paged(qkv, k_pages, v_pages, out, block_tables, nh, nkv, d, "attention_decode")
    B = out.shape[0]
    _need(qkv.dtype == torch.bfloat16, "attention_decode: bf16 only")
    _i32(positions, B, "attention_decode positions")
    _need(block_tables.shape[0] >= B, "attention_decode: one row of block_tables per token")
    ps = k_pages.shape[2]
    _need(ps % 4 == 0, f"attention_decode: page size {ps} is not a multiple of 4")
    _need(block_tables.shape[1] * ps >= max_len, "attention_decode: block_tables are narrower than max_len")
    splits = num_splits or decode_splits(B, nh, nkv, max_len, out.device, d)
    part_o = part_ml = None
    if splits > 1:
        part_o = torch.empty(B * nh * splits * d, dtype=torch.float32, device=out.device)
        part_ml = torch.empty(B * nh * splits * 2, dtype=torch.float32, device=out.device)
    _ok(_attn(d).ia_attn_decode(_p(qkv), qkv.shape[1], _p(k_pages), _p(v_pages), _p(out), nh * d, _p(part_o),
                                _p(part_ml), _p(positions), _p(block_tables), block_tables.shape[1], B, nh, nkv, ps,
                                k_pages.shape[0], ctypes.c_float(scale), int(window), splits, _stream()),
        "attention_decode")


def attention_decode_rotating(qkv, positions: torch.Tensor, inv_freq: Optional[torch.Tensor], rot: int,
                              slots: Optional[torch.Tensor], k_pages: torch.Tensor, v_pages: torch.Tensor,
                              out: torch.Tensor, block_tables: torch.Tensor, nh: int, nkv: int, d: int, scale: float,
                              window: int, max_len: int, num_splits: Optional[int] = None) -> None:
    """:func:`rope_kv_append` and :func:`attention_decode` of B single tokens in one launch (the same bits).

    ``qkv`` is the QKV product of the tokens, [B, (nh + 2 nkv) d] in bf16 or a :class:`SplitSum` of it (with
    ``slots`` None only the nh query heads are read and no key or value is made: the pages belong to another
    run of a layer).  Rotated queries stay inside the kernel; the token's key and value go to their slot of the
    pages and take part in the attention.
    """
    split = isinstance(qkv, SplitSum)
    src = qkv.parts if split else qkv
    B = out.shape[0]
    rows, row = (src.shape[1], src.shape[2]) if split else tuple(src.shape)
    _need(src.is_cuda and src.is_contiguous(), "attention_decode_rotating: qkv must be contiguous on the GPU")
    _need(src.dtype == (torch.float32 if split else torch.bfloat16),
          "attention_decode_rotating: bf16 rows or fp32 partial sums")
    _need(rows >= B and row >= (nh + (2 * nkv if slots is not None else 0)) * d,
          "attention_decode_rotating: rows of qkv are too few or too short for their heads")
    _need(k_pages.dtype == torch.bfloat16 and v_pages.dtype == torch.bfloat16 and out.dtype == torch.bfloat16
          and k_pages.dim() == 4 and k_pages.shape[1] == nkv and k_pages.shape[3] == d and out.is_cuda
          and tuple(v_pages.shape) == (k_pages.shape[0], nkv, d, k_pages.shape[2]) and tuple(out.shape) == (B, nh * d)
          and out.is_contiguous() and k_pages.is_contiguous() and v_pages.is_contiguous(),
          "attention_decode_rotating: bf16 key pages [num_pages, nkv, page_size, d], value pages "
          "[num_pages, nkv, d, page_size], out [B, nh d]")
    _dev(src, positions, inv_freq, slots, k_pages, v_pages, out, block_tables)
    _i32(positions, B, "attention_decode_rotating positions")
    if slots is not None:
        _i32(slots, B, "attention_decode_rotating slots")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous()
          and block_tables.shape[0] >= B, "attention_decode_rotating: one int32 row of block_tables per token")
    if inv_freq is not None:
        _need(inv_freq.dtype in (torch.float32, torch.float64) and inv_freq.numel() == rot // 2 and rot % 2 == 0
              and 0 < rot <= d and inv_freq.is_contiguous(),
              "attention_decode_rotating: inv_freq must hold rot/2 fp32 or float64 values, rot even and at most d")
    ps = k_pages.shape[2]
    _need(ps % 4 == 0, f"attention_decode_rotating: page size {ps} is not a multiple of 4")
    _need(block_tables.shape[1] * ps >= max_len, "attention_decode_rotating: block_tables are narrower than max_len")
    splits = num_splits or decode_splits(B, nh, nkv, max_len, out.device, d)
    part_o = part_ml = None
    if splits > 1:
        part_o = torch.empty(B * nh * splits * d, dtype=torch.float32, device=out.device)
        part_ml = torch.empty(B * nh * splits * 2, dtype=torch.float32, device=out.device)
    _ok(_attn(d).ia_attn_decode_fused(
        _p(src), DTYPE_CODE[src.dtype], src.shape[0] if split else 1, rows, row, _p(slots), _p(inv_freq),
        1 if (inv_freq is not None and inv_freq.dtype == torch.float64) else 0, rot if inv_freq is not None else 0,
        _p(k_pages), _p(v_pages), _p(out), nh * d, _p(part_o), _p(part_ml), _p(positions), _p(block_tables),
        block_tables.shape[1], B, nh, nkv, ps, k_pages.shape[0], ctypes.c_float(scale), int(window), splits, _stream()),
        "attention_decode_rotating")


PREFILL_TILE_ROWS = 64      # query rows of a workgroup's tile in attention_prefill
PREFILL_PAIRED = 0x100      # in a launch shape: 32 rows from each end of a request in place of 64 consecutive ones


def attention_prefill(qkv: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, out: torch.Tensor,
                      seq_starts: torch.Tensor, seq_ctx: torch.Tensor, block_tables: torch.Tensor,
                      tiles: torch.Tensor, num_tiles: int, nh: int, nkv: int, d: int, scale: float,
                      window: int, heads_per_workgroup: int = 0, paired: bool = False) -> None:
    """bf16 causal attention of portions of prompts over their pages, on MFMA.

    Request s brings rows seq_starts[s] .. seq_starts[s+1]-1 of qkv and had seq_ctx[s] tokens cached
    before; tiles[i] = (s, first row of a block of PREFILL_TILE_ROWS among the request's rows).  ``heads_per_workgroup``:
    0 for the kernel's own choice, or 1, 2, 4; ``paired``: a workgroup takes half a block of rows from each end of
    its request's new tokens, so that all workgroups of a request have the same work under the causal mask (every
    block of every request must be listed then; without effect under a window).  A value of :func:`prefill_launch_shape` may stand in
    ``heads_per_workgroup`` for both.  The result has the same bits whatever the shape.
    """
    _check_paged(qkv, k_pages, v_pages, out, block_tables, nh, nkv, d, "attention_prefill")
    _need(qkv.dtype == torch.bfloat16, "attention_prefill: bf16 only")
    B = block_tables.shape[0]
    _i32(seq_starts, B + 1, "attention_prefill seq_starts")
    _i32(seq_ctx, B, "attention_prefill seq_ctx")
    _need(tiles.dtype == torch.int32 and tiles.is_cuda and tiles.is_contiguous() and tiles.numel() >= 2 * num_tiles,
          "attention_prefill: tiles int32 [num_tiles, 2]")
    ps = k_pages.shape[2]
    _need(ps % 4 == 0, f"attention_prefill: page size {ps} is not a multiple of 4")
    _ok(_attn(d).ia_attn_prefill(_p(qkv), qkv.shape[1], _p(k_pages), _p(v_pages), _p(out), nh * d, _p(seq_starts),
                                 _p(seq_ctx), _p(block_tables), block_tables.shape[1], _p(tiles), num_tiles, nh, nkv,
                                 ps, k_pages.shape[0], ctypes.c_float(scale), int(window),
                                 int(heads_per_workgroup) | (PREFILL_PAIRED if paired else 0), _stream()),
        "attention_prefill")


def prefill_launch_shape(nh: int, nkv: int, d: int, q_lens: Sequence[int], ctx_lens: Sequence[int],
                         window: int, device: torch.device) -> int:
    """The shape of the :func:`attention_prefill` launch for these portions of prompts (``q_lens`` new tokens
    after ``ctx_lens`` cached ones each): how many query heads share a workgroup's tiles of keys (0: the kernel's
    default), with :data:`PREFILL_PAIRED` added when a workgroup should take half its rows from each end of its
    request.  The bits of the result do not depend on it; all figures are of the 8B shape (32 heads over 8, 128).

    Four heads a workgroup (the default at head sizes 80 to 160 with three or more query heads to a key/value
    head) read the keys least often but make few workgroups: when they would fill fewer than three quarters of
    the compute units, two heads are taken (1,024 tokens: 34 against 49 us).  When the launch has no more
    workgroups than compute units, every workgroup runs from start to end and the longest sets the time: under
    the causal mask that is the last block of a prompt, with twice the rounds of the average one.  Paired rows
    give all workgroups of a request the same work then (2,048 tokens: 66 against 89 us with four heads, 71 with
    two unpaired; 2,048 after 2,048: 147 against 171).  With more workgroups than compute units the rounds of a
    paired workgroup in which half its waves have run out of keys cost more than the balance gains (4,096
    tokens: 220 against 192 us), and under a window the rows of the two ends share no keys: not paired then.
    """
    G = nh // nkv
    widest = 4 if 80 <= d <= 160 else 2
    hpw = widest if G >= 3 else (2 if G == 2 else 1)
    tiles = total = longest = 0
    for q, c in zip(q_lens, ctx_lens):
        for first in range(0, q, 64):           # a block of 64 rows sees the keys up to its last row, or a window's worth
            keys = c + min(q, first + 64)
            if window > 0:
                keys = min(keys, window + 64)
            tiles += 1
            total += keys
            longest = max(longest, keys)
    if tiles == 0:
        return 0
    cus = compute_units(device)
    workgroups = tiles * nkv * ((G + hpw - 1) // hpw)
    if hpw == 4 and 4 * workgroups < 3 * cus:
        hpw, workgroups = 2, tiles * nkv * ((G + 1) // 2)
    if window == 0:
        return hpw | (PREFILL_PAIRED if workgroups <= cus else 0)
    # under a window: two heads where four would give at most one workgroup a compute unit with the longest
    # block at 1.5 times the average (more, smaller workgroups fill what the long ones leave idle)
    if hpw == 4 and workgroups <= cus and longest * tiles >= 1.5 * total:
        hpw = 2
    return hpw


# ------------------------------------------------------------------------- sampling
def argmax(logits: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    _dev(logits, out)
    R, V = logits.shape
    _need(logits.dtype == torch.float32, "argmax: logits must be fp32")
    _i32(out, R, "argmax out")
    _ok(_core().ia_argmax(_p(logits), V, _p(out), R, V, _stream()), "argmax")
    return out


def repetition_penalty(logits: torch.Tensor, recent: torch.Tensor, counts: torch.Tensor,
                       penalty: torch.Tensor, previous: Optional[torch.Tensor] = None,
                       previous_index: Optional[torch.Tensor] = None) -> None:
    """Every token of recent[r, :counts[r]] is penalised in row r (a positive logit divided by penalty[r], another
    multiplied by it; a token that stands twice, twice).  ``previous`` (int32 tokens that an earlier launch left
    on the device) and ``previous_index`` (int32 [R]: which of them is row r's newest token, -1: none) add a token
    that the host has not seen yet."""
    _dev(logits, recent, counts, penalty, previous, previous_index)
    R, V = logits.shape
    _need(logits.dtype == torch.float32, "penalty: logits must be fp32")
    _need(recent.dtype == torch.int32 and recent.dim() == 2 and recent.shape[0] == R, "penalty: recent int32 [R, W]")
    _i32(counts, R, "penalty counts")
    _need(penalty.dtype == torch.float32 and penalty.numel() == R, "penalty: one fp32 factor per row")
    if previous is not None or previous_index is not None:
        _need(previous is not None and previous_index is not None and previous.dtype == torch.int32
              and previous.is_contiguous(), "penalty: previous tokens int32 with their index")
        _i32(previous_index, R, "penalty previous_index")
    _ok(_core().ia_repetition_penalty(_p(logits), V, _p(recent), recent.shape[1], _p(counts), _p(penalty),
                                      _p(previous), _p(previous_index), R, V, _stream()), "repetition_penalty")


def sample(logits: torch.Tensor, work: torch.Tensor, temperature: torch.Tensor, top_p: torch.Tensor,
           u: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    _dev(logits, work, temperature, top_p, u, out)
    R, V = logits.shape
    _need(logits.dtype == torch.float32 and work.dtype == torch.float32 and work.numel() >= R * V,
          "sample: logits fp32 [R, V] and fp32 work space of the same size")
    for name, t in (("temperature", temperature), ("top_p", top_p), ("u", u)):
        _need(t.dtype == torch.float32 and t.numel() == R, f"sample: {name} must hold one fp32 value per row")
    _i32(out, R, "sample out")
    _ok(_core().ia_sample(_p(logits), V, _p(work), _p(temperature), _p(top_p), _p(u), _p(out), R, V, _stream()),
        "sample")
    return out


# ---------------------------------------------------- which head sizes the MFMA kernels take
def attention_mfma_available(d: int) -> bool:
    """Whether the MFMA attention kernels take head size d (their library is built at its first use)."""
    return d in _build.SUPPORTED_HEAD_DIMS


# ------------------------------------------------- time per kernel, by the device's clock
# INFERNUM_PROFILE=1 in the environment (or ``set_profile(True)``): every call of a kernel function of this
# module is bracketed by two events on its stream, and a table of calls and device time per function goes to
# standard error when the process ends (``profile_report`` gives it at any time).  The reference's switch of the
# same name prints the time per operation of its graph executor (infernum-cpu/src/executor.rs:24-71).  Steps
# are not recorded into HIP graphs meanwhile (a replayed launch has no call to bracket).
_PROFILED = ("cast", "copy_pages", "gather_tokens", "words_from_host", "words_to_host", "embed", "add_rmsnorm", "residual_add", "rope_kv_append", "swiglu", "gemm_generic", "gemm_mfma",
             "gemm_library", "gemm_skinny", "gemm_skinny_rows", "attention_generic", "attention_decode", "attention_decode_rotating",
             "attention_prefill", "argmax", "repetition_penalty", "sample")
_profile_on = False
_profile_open: List[Tuple[str, "torch.cuda.Event", "torch.cuda.Event"]] = []
_profile_sum: Dict[str, List[float]] = {}          # function -> [calls, milliseconds]
_plain = {name: globals()[name] for name in _PROFILED}


def _fold_profile() -> None:
    if _profile_open:
        torch.cuda.synchronize()
        for name, a, b in _profile_open:
            acc = _profile_sum.setdefault(name, [0, 0.0])
            acc[0] += 1
            acc[1] += a.elapsed_time(b)
        _profile_open.clear()


def _timed(name: str, fn):
    @functools.wraps(fn)
    def call(*args, **kw):
        if not _profile_on or torch.cuda.is_current_stream_capturing():
            return fn(*args, **kw)
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        try:
            return fn(*args, **kw)
        finally:
            b.record()
            _profile_open.append((name, a, b))
            if len(_profile_open) >= 4096:
                _fold_profile()
    return call


for _name in _PROFILED:
    globals()[_name] = _timed(_name, _plain[_name])


def profiling() -> bool:
    return _profile_on


def set_profile(on: bool) -> bool:
    """Switch the timing of every kernel call on or off; returns what it was.  Engines made while it is on
    do not record their decode steps into graphs."""
    global _profile_on
    before, _profile_on = _profile_on, bool(on)
    return before


def profile_report(reset: bool = False) -> Dict[str, Tuple[int, float]]:
    """function -> (calls, milliseconds on the device) since the start or the last reset."""
    _fold_profile()
    out = {k: (int(v[0]), float(v[1])) for k, v in _profile_sum.items()}
    if reset:
        _profile_sum.clear()
    return out


def _print_profile() -> None:
    try:
        rep = profile_report()
    except Exception:                                   # the device is gone at exit: nothing to print
        return
    if not rep:
        return
    total = sum(ms for _, ms in rep.values())
    print(f"[infernum_amd profile] {total:.3f} ms in {sum(c for c, _ in rep.values())} kernel calls", file=sys.stderr)
    for name, (calls, ms) in sorted(rep.items(), key=lambda kv: -kv[1][1]):
        print(f"[infernum_amd profile] {name:28s} {calls:8d} calls {ms:12.3f} ms {ms / calls * 1e3:10.1f} us/call "
              f"{100 * ms / total:5.1f} %", file=sys.stderr)


if os.environ.get("INFERNUM_PROFILE") == "1":
    _profile_on = True
atexit.register(_print_profile)
