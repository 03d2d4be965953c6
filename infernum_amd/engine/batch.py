"""Packing of one step's batch: from (request, tokens, wanted places) entries and
the cache manager's block tables to the int32 arrays the kernels read.

All arrays of a step lie in one host buffer, in segments aligned to 16 bytes, and
go to the device in one copy.  Requests that bring a single token are put first,
portions of prompts after them, so that the decode kernels work on rows
0 .. num_decode-1 and the prefill kernels on the rest.
(The reference uploads four tensors per decode step and reads two of them back,
infernum/src/backend.rs:209-241, infernum-cuda/src/inner/cuda_graph_engine.rs:
1500-1503; its prefill uploads the block table once per layer,
infernum-cuda/src/inner/cuda/paged_kv_cache.rs:158-159.)
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass, field
from typing import Hashable, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache import CacheManager, native
from ..parts.base import StepContext

POW2_WIDTH = -1             # for pack_step's bt_width


class StepError(ValueError):
    """A step's entries are malformed (unknown place wanted, token outside the vocabulary, ...)."""


@dataclass
class StepEntry:
    request: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = field(default_factory=list)     # places among ``tokens`` whose logits are wanted


@dataclass
class PackedStep:
    """Host side of a step: the int32 buffer, where each array lies in it, and the sizes."""

    host: np.ndarray
    offsets: List[int]
    sizes: List[int]
    bt_shapes: List[Tuple[int, int]]
    batch: List[StepEntry]               # entries in the order of the rows
    q_lens: List[int]
    ctx_lens: List[int]
    num_decode: int
    num_tiles: int
    num_logit_rows: int
    tile_rows: int = 0                   # height of the row tiles that were packed (0: none)
    order: Sequence[int] = ()            # row r of the batch is entry order[r] of the step

    def context(self, dev: torch.Tensor) -> StepContext:
        """The step as the parts see it, over ``dev``, the device copy of ``host``."""
        def seg(i: int) -> torch.Tensor:
            return dev[self.offsets[i]:self.offsets[i] + self.sizes[i]]
        n_groups = len(self.bt_shapes)
        return StepContext(
            num_tokens=sum(self.q_lens), num_seqs=len(self.batch), num_decode=self.num_decode,
            token_ids=seg(0), positions=seg(1), token_seq=seg(2), seq_starts=seg(3), seq_ctx=seg(4),
            state_slots=seg(5), logit_rows=seg(6),
            block_tables=[seg(9 + 2 * g).view(self.bt_shapes[g]) for g in range(n_groups)],
            slots=[seg(8 + 2 * g) for g in range(n_groups)],
            q_lens=self.q_lens, ctx_lens=self.ctx_lens, max_q_len=max(self.q_lens),
            max_total_len=max(c + q for c, q in zip(self.ctx_lens, self.q_lens)),
            packed_row_tiles={self.tile_rows: (seg(7).view(-1, 2), self.num_tiles)} if self.tile_rows else {},
        )


def check_entries(entries: Sequence[StepEntry], vocab_size: int, max_tokens: int) -> None:
    total = 0
    for e in entries:
        toks = e.tokens
        n = len(toks)
        total += n
        if n == 1:                              # the common case of a decoding request, without min() and max()
            if not 0 <= toks[0] < vocab_size:
                raise StepError(f"request {e.request!r}: token id outside the vocabulary [0, {vocab_size})")
        elif n == 0:
            raise StepError(f"request {e.request!r} brings no tokens")
        elif min(toks) < 0 or max(toks) >= vocab_size:
            raise StepError(f"request {e.request!r}: token id outside the vocabulary [0, {vocab_size})")
        for w in e.want:
            if not 0 <= w < n:
                raise StepError(f"request {e.request!r}: wanted place {w} is outside its {n} tokens")
    if len({e.request for e in entries}) != len(entries):
        seen = set()
        for e in entries:
            if e.request in seen:
                raise StepError(f"request {e.request!r} stands twice in one step")
            seen.add(e.request)
    if total > max_tokens:
        raise StepError(f"a step of {total} tokens is above max_tokens_per_step {max_tokens}")


def pack_step(cache: CacheManager, entries: Sequence[StepEntry], bt_width: Optional[int] = None,
              tile_rows: int = 0) -> PackedStep:
    """Pages for the entries' tokens must be reserved already.  ``bt_width`` widens the block
    tables to a fixed number of columns (filled with NO_PAGE); ``POW2_WIDTH`` to the power of two
    (at least 8) that holds the longest table of any group.  ``tile_rows``: the height of the row tiles
    that a part of the model asked for (``Part.step_needs``), 0 for none.  The arrays are laid out natively
    (``ia_cache_pack_step``); the buffer returned is a copy of the native one."""
    n = len(entries)
    G = len(cache.groups)
    q_lens_in = [len(e.tokens) for e in entries]
    want_counts = [len(e.want) for e in entries]
    if max(q_lens_in, default=0) == 1:       # a step of single tokens: no nested walk
        flat_tokens = [e.tokens[0] for e in entries]
    else:
        flat_tokens = [t for e in entries for t in e.tokens]
    flat_wants = [w for e in entries for w in e.want]
    S = 8 + 2 * G
    meta_len = 7 + 2 * S + G + 2 * n
    meta = (ctypes.c_int32 * meta_len)()
    lib, h = native.lib(), cache.native_handle()
    # short lists go over as ctypes arrays (a microsecond each); a prompt's many tokens through numpy
    if len(flat_tokens) <= 256:
        tokens = (ctypes.c_int32 * max(len(flat_tokens), 1))(*flat_tokens)
    else:
        keep = np.array(flat_tokens, dtype=np.int32)
        tokens = keep.ctypes.data_as(ctypes.POINTER(ctypes.c_int32))
    rc = lib.ia_cache_pack_step(
        h, n, (ctypes.c_int64 * max(n, 1))(*cache.request_ids([e.request for e in entries])),
        (ctypes.c_int * max(n, 1))(*q_lens_in), tokens, (ctypes.c_int * max(n, 1))(*want_counts),
        (ctypes.c_int32 * max(len(flat_wants), 1))(*flat_wants), int(bt_width or 0), int(tile_rows) if tile_rows > 0 else (1 << 30), meta, meta_len)
    if rc != 0:
        cache._fail()
    m = meta[:]
    total, num_decode, num_tiles, num_rows = m[:4]
    offsets = m[7:7 + S]
    sizes = m[7 + S:7 + 2 * S]
    cols = m[7 + 2 * S:7 + 2 * S + G]
    order = m[7 + 2 * S + G:7 + 2 * S + G + n]
    ctx_lens = m[7 + 2 * S + G + n:7 + 2 * S + G + 2 * n]
    buf = (ctypes.c_int32 * total)()         # a copy of the native buffer, which the next step overwrites
    ctypes.memmove(buf, lib.ia_cache_packed(h), total * 4)
    host = np.frombuffer(buf, dtype=np.int32)
    batch = [entries[i] for i in order]
    return PackedStep(host, offsets, sizes, [(n, c) for c in cols], batch, [q_lens_in[i] for i in order], ctx_lens,
                      num_decode, num_tiles, num_rows, int(tile_rows), order)
