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

from dataclasses import dataclass, field
from typing import Hashable, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache import CacheManager
from ..parts.base import StepContext

PREFILL_TILE_ROWS = 64      # query rows per workgroup tile of the MFMA prefill attention


class StepError(ValueError):
    """A step's entries are malformed (unknown place wanted, token outside the vocabulary, ...)."""


@dataclass
class StepEntry:
    request: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = field(default_factory=list)     # places among ``tokens`` whose logits are wanted


def _align4(n: int) -> int:
    return (n + 3) & ~3


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
            prefill_tiles=seg(7).view(-1, 2), num_prefill_tiles=self.num_tiles,
        )


def check_entries(entries: Sequence[StepEntry], vocab_size: int, max_tokens: int) -> None:
    seen = set()
    for e in entries:
        if e.request in seen:
            raise StepError(f"request {e.request!r} stands twice in one step")
        seen.add(e.request)
        if len(e.tokens) == 0:
            raise StepError(f"request {e.request!r} brings no tokens")
        for w in e.want:
            if not 0 <= w < len(e.tokens):
                raise StepError(f"request {e.request!r}: wanted place {w} is outside its {len(e.tokens)} tokens")
        if min(e.tokens) < 0 or max(e.tokens) >= vocab_size:
            raise StepError(f"request {e.request!r}: token id outside the vocabulary [0, {vocab_size})")
    total = sum(len(e.tokens) for e in entries)
    if total > max_tokens:
        raise StepError(f"a step of {total} tokens is above max_tokens_per_step {max_tokens}")


def pack_step(cache: CacheManager, entries: Sequence[StepEntry], bt_width: Optional[int] = None) -> PackedStep:
    """Pages for the entries' tokens must be reserved already.  ``bt_width`` widens the block
    tables to a fixed number of columns (filled with NO_PAGE)."""
    order = sorted(range(len(entries)), key=lambda i: (len(entries[i].tokens) != 1, i))
    batch = [entries[i] for i in order]
    B = len(batch)
    num_decode = sum(1 for e in batch if len(e.tokens) == 1)
    q_lens = [len(e.tokens) for e in batch]
    ctx_lens = [cache.num_tokens(e.request) for e in batch]
    starts = np.zeros(B + 1, dtype=np.int32)
    starts[1:] = np.cumsum(q_lens)
    start_of = {e.request: int(starts[i]) for i, e in enumerate(batch)}
    reqs = [e.request for e in batch]
    if num_decode == B:
        token_ids = np.fromiter((e.tokens[0] for e in batch), dtype=np.int32, count=B)
        positions = np.asarray(ctx_lens, dtype=np.int32)
        token_seq = np.arange(B, dtype=np.int32)
    else:
        token_ids = np.concatenate([np.asarray(e.tokens, dtype=np.int32) for e in batch])
        positions = np.concatenate([np.arange(c, c + q, dtype=np.int32) for c, q in zip(ctx_lens, q_lens)])
        token_seq = np.repeat(np.arange(B, dtype=np.int32), q_lens)
    logit_rows = np.asarray([start_of[e.request] + w for e in entries for w in e.want], dtype=np.int32)
    state_slots = np.asarray([cache.state_slot(r) for r in reqs], dtype=np.int32)
    tiles = [(s, r) for s in range(num_decode, B) for r in range(0, q_lens[s], PREFILL_TILE_ROWS)]
    tiles_np = np.asarray(tiles, dtype=np.int32).reshape(-1)
    segs: List[np.ndarray] = [token_ids, positions, token_seq, starts, np.asarray(ctx_lens, dtype=np.int32),
                              state_slots, logit_rows, tiles_np]
    bt_shapes = []
    for g in cache.groups:
        bt = cache.block_table_rows(g.index, reqs, bt_width)
        bt_shapes.append(bt.shape)
        segs.append(np.concatenate([cache.token_slots(g.index, r, c, q) for r, c, q in zip(reqs, ctx_lens, q_lens)]))
        segs.append(bt.reshape(-1))
    offsets, total = [], 0
    for s in segs:
        offsets.append(total)
        total += _align4(max(s.size, 1))
    host = np.zeros(total, dtype=np.int32)
    for o, s in zip(offsets, segs):
        host[o:o + s.size] = s
    return PackedStep(host, offsets, [s.size for s in segs], bt_shapes, batch, q_lens, ctx_lens, num_decode,
                      len(tiles), int(logit_rows.size))
