"""The cache manager: paged keys and values per group of layers, block tables
per request, and slots for per-request state of fixed size.

Layer runs whose mixers need the same thing of the cache (all keys; a window
of them) form a group.  A group has its own pool of pages and its own block
tables; all runs of a group share the block table of a request, each with pages
of its own ([num_pages, nkv, page_size, d] for keys, the same for values;
the reference keeps [num_pages, page_size, nkv, d] per layer,
infernum-cuda/src/inner/cuda/paged_kv_cache.rs:88-102, and has one group only).
Pages go back to the pool when a request ends (infernum-runtime/src/scheduler.rs:
289-305) or, in a window group, when every later query's window has passed them
(the reference keeps them, TABNINE.md:53).

State slots: a mixer that declares a StateSpec gets a [num_slots, *shape] tensor
per run; a request owns one slot index from admission to release, zeroed when
it is taken.  Attention needs none; the slots are there for mixers with
recurrent state.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..parts.base import CacheSpec, CacheView, StateSpec
from .pages import NO_PAGE, BlockTable, PageAllocator, PageError, pages_for


class CacheGroup:
    """Host bookkeeping of one group: its allocator and its requests' block tables."""

    def __init__(self, index: int, kind: str, window: int, page_size: int, num_pages: int):
        self.index, self.kind, self.window = index, kind, int(window)
        self.page_size = int(page_size)
        self.allocator = PageAllocator(num_pages)
        self.tables: Dict[Hashable, BlockTable] = {}
        self.entries: List[int] = []         # schedule entries that own pages in this group

    def pages_missing(self, req: Hashable, n_new: int) -> int:
        t = self.tables[req]
        return max(0, pages_for(t.num_tokens + n_new, self.page_size) - len(t.pages))

    def grow(self, req: Hashable, n_new: int) -> bool:
        t = self.tables[req]
        got = self.allocator.allocate_many(self.pages_missing(req, n_new))
        if got is None:
            return False
        t.pages.extend(got)
        return True

    def advance(self, req: Hashable, n_new: int) -> List[int]:
        """Count n_new more tokens as stored; returns the pages a window has passed (now free)."""
        t = self.tables[req]
        t.num_tokens += n_new
        if t.num_tokens > len(t.pages) * self.page_size:
            raise PageError(f"request {req!r} stored {t.num_tokens} tokens in {len(t.pages)} pages")
        freed: List[int] = []
        if self.kind == "window" and self.window > 0:
            # the next query stands at position num_tokens and sees keys >= num_tokens - window + 1
            first_needed = max(0, t.num_tokens - self.window + 1) // self.page_size
            while t.first_live < min(first_needed, len(t.pages)):
                p = t.pages[t.first_live]
                if p != NO_PAGE:
                    self.allocator.free(p)
                    freed.append(p)
                    t.pages[t.first_live] = NO_PAGE
                t.first_live += 1
        return freed

    def release(self, req: Hashable) -> List[int]:
        t = self.tables.pop(req)
        freed = t.live_pages()
        for p in freed:
            self.allocator.free(p)
        return freed


class StateSlotPool:
    """Indices of per-request state records of fixed size."""

    def __init__(self, num_slots: int):
        self.num_slots = int(num_slots)
        self._free = list(range(self.num_slots - 1, -1, -1))
        self._used = bytearray(self.num_slots)

    @property
    def num_free(self) -> int:
        return len(self._free)

    def acquire(self) -> Optional[int]:
        if not self._free:
            return None
        s = self._free.pop()
        self._used[s] = 1
        return s

    def release(self, slot: int) -> None:
        if not 0 <= slot < self.num_slots or not self._used[slot]:
            raise PageError(f"state slot {slot} is released twice or was never taken")
        self._used[slot] = 0
        self._free.append(slot)


@dataclass
class CacheConfig:
    page_size: int = 16
    num_pages: int = 1024                  # per group
    num_state_slots: int = 64
    poison_freed_pages: bool = False       # fill freed pages with NaN: a read after free shows in the logits


class CacheManager:
    """``needs[i]`` = (CacheSpec or None, StateSpec or None) of schedule entry i;
    ``cache_of[i]`` = the entry whose cache entry i reads, or None."""

    def __init__(self, needs: Sequence[Tuple[Optional[CacheSpec], Optional[StateSpec]]],
                 cache_of: Sequence[Optional[int]], config: CacheConfig, dtype: torch.dtype = torch.float32,
                 device: Optional[torch.device] = None):
        self.config = config
        self.page_size = int(config.page_size)
        if self.page_size <= 0:
            raise ValueError("page_size must be positive")
        self.device = device
        self.dtype = dtype
        self.groups: List[CacheGroup] = []
        self._entry_group: List[int] = []
        self._entry_spec: List[Optional[CacheSpec]] = []
        self._cache_of = list(cache_of)
        key_to_group: Dict[Tuple, int] = {}
        for i, (cs, _) in enumerate(needs):
            self._entry_spec.append(cs)
            if cs is None:
                self._entry_group.append(-1)
                continue
            key = cs.group_key()
            if key not in key_to_group:
                key_to_group[key] = len(self.groups)
                self.groups.append(CacheGroup(len(self.groups), cs.kind, cs.window, self.page_size, config.num_pages))
            g = key_to_group[key]
            self.groups[g].entries.append(i)
            self._entry_group.append(g)
        self.slots = StateSlotPool(config.num_state_slots)
        self._slot_of: Dict[Hashable, int] = {}
        self._tokens: Dict[Hashable, int] = {}
        # device memory
        self.k_pages: List[Optional[torch.Tensor]] = [None] * len(needs)
        self.v_pages: List[Optional[torch.Tensor]] = [None] * len(needs)
        self.state: List[Optional[torch.Tensor]] = [None] * len(needs)
        if device is not None:
            for i, (cs, ss) in enumerate(needs):
                if cs is not None:
                    # values are kept transposed within a page: what the PV product of the matrix cores reads
                    self.k_pages[i] = torch.zeros((config.num_pages, cs.num_kv_heads, self.page_size, cs.head_dim),
                                                  dtype=dtype, device=device)
                    self.v_pages[i] = torch.zeros((config.num_pages, cs.num_kv_heads, cs.head_dim, self.page_size),
                                                  dtype=dtype, device=device)
                if ss is not None:
                    self.state[i] = torch.zeros((config.num_state_slots,) + tuple(ss.shape), dtype=ss.dtype,
                                                device=device)

    # ---- requests -------------------------------------------------------------
    def has(self, req: Hashable) -> bool:
        return req in self._slot_of

    def requests(self) -> List[Hashable]:
        return list(self._slot_of)

    def admit(self, req: Hashable) -> bool:
        """Give the request empty block tables and a state slot; False when no slot is free."""
        if req in self._slot_of:
            raise PageError(f"request {req!r} is admitted twice")
        slot = self.slots.acquire()
        if slot is None:
            return False
        self._slot_of[req] = slot
        self._tokens[req] = 0
        for g in self.groups:
            g.tables[req] = BlockTable()
        for st in self.state:
            if st is not None:
                st[slot].zero_()
        return True

    def state_slot(self, req: Hashable) -> int:
        return self._slot_of[req]

    def num_tokens(self, req: Hashable) -> int:
        return self._tokens[req]

    def pages_needed(self, req: Optional[Hashable], n_new: int) -> List[int]:
        """Per group, the pages that n_new more tokens of the request would take from the pool
        (a request that is not admitted yet holds nothing)."""
        if req is not None and req in self._slot_of:
            return [g.pages_missing(req, n_new) for g in self.groups]
        return [pages_for(n_new, g.page_size) for g in self.groups]

    def tokens_that_fit(self, req: Optional[Hashable], promised: Optional[Sequence[int]] = None) -> int:
        """How many more tokens of the request the pool can hold, with ``promised[g]`` pages of
        every group already spoken for."""
        best = 1 << 60
        for i, g in enumerate(self.groups):
            avail = g.allocator.num_free - (promised[i] if promised is not None else 0)
            if req is not None and req in self._slot_of:
                t = g.tables[req]
                room = (len(t.pages) + max(avail, 0)) * g.page_size - t.num_tokens
            else:
                room = max(avail, 0) * g.page_size
            best = min(best, room)
        return max(best, 0)

    def can_reserve(self, req: Hashable, n_new: int) -> bool:
        return all(g.allocator.can_allocate(g.pages_missing(req, n_new)) for g in self.groups)

    def reserve(self, req: Hashable, n_new: int) -> bool:
        """Pages for the next n_new tokens in every group, or nothing at all."""
        if not self.can_reserve(req, n_new):
            return False
        for g in self.groups:
            ok = g.grow(req, n_new)
            assert ok
        return True

    def commit(self, req: Hashable, n_new: int) -> None:
        """The n_new tokens are stored; pages that a window has passed go back to the pool."""
        self._tokens[req] += n_new
        for g in self.groups:
            self._poison(g, g.advance(req, n_new))

    def release(self, req: Hashable) -> None:
        """The request is over (finished, cancelled or preempted): everything it holds goes back."""
        slot = self._slot_of.pop(req, None)
        if slot is None:
            raise PageError(f"request {req!r} is released but not admitted")
        del self._tokens[req]
        for g in self.groups:
            self._poison(g, g.release(req))
        self.slots.release(slot)

    def _poison(self, g: CacheGroup, pages: List[int]) -> None:
        if not self.config.poison_freed_pages or not pages or self.device is None:
            return
        idx = torch.tensor(pages, dtype=torch.long, device=self.device)
        for e in g.entries:
            self.k_pages[e].index_fill_(0, idx, float("nan"))
            self.v_pages[e].index_fill_(0, idx, float("nan"))

    # ---- what a step needs --------------------------------------------------------
    def free_pages(self, group: int = 0) -> int:
        return self.groups[group].allocator.num_free

    def min_free_pages(self) -> int:
        return min((g.allocator.num_free for g in self.groups), default=1 << 30)

    def block_table(self, group: int, req: Hashable) -> BlockTable:
        return self.groups[group].tables[req]

    def block_table_rows(self, group: int, reqs: Sequence[Hashable], width: Optional[int] = None) -> np.ndarray:
        """int32 [len(reqs), width], NO_PAGE where a request holds no page."""
        g = self.groups[group]
        if width is None:
            width = max((len(g.tables[r].pages) for r in reqs), default=1)
        width = max(width, 1)
        out = np.full((len(reqs), width), NO_PAGE, dtype=np.int32)
        for i, r in enumerate(reqs):
            p = g.tables[r].pages
            out[i, :len(p)] = p
        return out

    def token_slots(self, group: int, req: Hashable, start: int, n: int) -> np.ndarray:
        """page * page_size + offset of positions start .. start+n-1 (pages must be reserved)."""
        g = self.groups[group]
        if n == 1:                                   # a decoded token: no arrays needed
            t = g.tables[req].pages
            i = start // g.page_size
            if i >= len(t) or t[i] < 0:
                raise PageError(f"request {req!r} has no page for position {start}")
            return np.asarray([t[i] * g.page_size + start % g.page_size], dtype=np.int32)
        pos = np.arange(start, start + n, dtype=np.int64)
        pages = np.asarray(g.tables[req].pages, dtype=np.int64)
        idx = pos // g.page_size
        if n and (idx[-1] >= len(pages) or (pages[idx] < 0).any()):
            raise PageError(f"request {req!r} has no page for positions {start}..{start + n - 1}")
        return (pages[idx] * g.page_size + pos % g.page_size).astype(np.int32)

    def views(self) -> List[CacheView]:
        """One CacheView per schedule entry."""
        out = []
        for i, src in enumerate(self._cache_of):
            j = i if src is None else src
            out.append(CacheView(group=self._entry_group[j], k_pages=self.k_pages[j], v_pages=self.v_pages[j],
                                 writable=src is None, state=self.state[j]))
        return out

    # ---- invariants (tests) ---------------------------------------------------------
    def check(self) -> None:
        """Every page is free or held by exactly one request; counts agree."""
        for g in self.groups:
            held: Dict[int, Hashable] = {}
            for r, t in g.tables.items():
                for p in t.live_pages():
                    if p in held:
                        raise PageError(f"group {g.index}: page {p} is held by {held[p]!r} and {r!r}")
                    if not g.allocator.is_used(p):
                        raise PageError(f"group {g.index}: page {p} of {r!r} is marked free")
                    held[p] = r
                if t.num_tokens > len(t.pages) * g.page_size:
                    raise PageError(f"group {g.index}: {r!r} holds too few pages")
            if len(held) != g.allocator.num_used:
                raise PageError(f"group {g.index}: {g.allocator.num_used} pages in use, {len(held)} held: a page is lost")
        if len(self._slot_of) != self.slots.num_slots - self.slots.num_free:
            raise PageError("state slots in use do not match the admitted requests")
        if len(set(self._slot_of.values())) != len(self._slot_of):
            raise PageError("two requests share a state slot")
