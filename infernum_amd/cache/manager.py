"""The cache manager: paged keys and values per group of layers, block tables
per request, and slots for per-request state of fixed size.

Layer runs whose mixers need the same thing of the cache (all keys; a window
of them) form a group.  A group has its own pool of pages and its own block
tables; all runs of a group share the block table of a request, each with pages
of its own (what a page holds is declared by the mixer's CacheSpec as named tensors with a per-token
shape; for attention [num_pages, nkv, page_size, d] for keys and the transposed [num_pages, nkv, d,
page_size] for values; the reference keeps [num_pages, page_size, nkv, d] per layer,
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

import ctypes
import re
from dataclasses import dataclass
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..parts.base import CacheSpec, CacheView, StateSpec
from . import native
from .pages import NO_PAGE, BlockTable, PageAllocator, PageError, pages_for  # noqa: F401  (NO_PAGE: part of this module's face)

_KINDS = {"full": 0, "window": 1}


class CacheGroup:
    """One group as the host sees it: what kind it is, which schedule entries own pages in it, and its pool
    (the tables themselves are kept natively by the manager)."""

    def __init__(self, index: int, kind: str, window: int, page_size: int):
        self.index, self.kind, self.window = index, kind, int(window)
        self.page_size = int(page_size)
        self.entries: List[int] = []         # schedule entries that own pages in this group
        self.allocator: Optional[PageAllocator] = None


class StateSlotPool:
    """Indices of per-request state records of fixed size (alone, or the slots of a cache manager)."""

    def __init__(self, num_slots: int, _view: Optional[ctypes.c_void_p] = None, _owner: object = None):
        self._lib = native.lib()
        self._owner = _owner                 # the cache manager whose slots these are, kept alive
        self.num_slots = int(num_slots)
        if _view is not None:
            self._h, self._owned = _view, False
        else:
            self._h = ctypes.c_void_p(self._lib.ia_cache_create(0, None, None, 1, 1, self.num_slots))
            self._owned = True

    def __del__(self):
        if getattr(self, "_owned", False) and self._h:
            self._lib.ia_cache_destroy(self._h)
            self._h = None

    @property
    def num_free(self) -> int:
        return int(self._lib.ia_cache_num_free_slots(self._h))

    def acquire(self) -> Optional[int]:
        s = int(self._lib.ia_cache_acquire_slot(self._h))
        return None if s < 0 else s

    def release(self, slot: int) -> None:
        if self._lib.ia_cache_release_slot(self._h, int(slot)) != 0:
            raise PageError(self._lib.ia_cache_error(self._h).decode())


@dataclass
class CacheConfig:
    page_size: int = 16
    num_pages: int = 1024                  # per group
    num_state_slots: int = 64
    poison_freed_pages: bool = False       # fill freed pages with NaN: a read after free shows in the logits


class CacheManager:
    """``needs[i]`` = (CacheSpec or None, StateSpec or None) of schedule entry i;
    ``cache_of[i]`` = the entry whose cache entry i reads, or None.

    Requests are named by any hashable value here and by a number in the native bookkeeping."""

    def __init__(self, needs: Sequence[Tuple[Optional[CacheSpec], Optional[StateSpec]]],
                 cache_of: Sequence[Optional[int]], config: CacheConfig, dtype: torch.dtype = torch.float32,
                 device: Optional[torch.device] = None):
        self.config = config
        self.page_size = int(config.page_size)
        if self.page_size <= 0:
            raise ValueError("page_size must be positive")
        if config.num_pages <= 0:
            raise ValueError("a page pool needs at least one page")
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
            if cs.kind not in _KINDS:
                raise ValueError(f"cache kind {cs.kind!r}: one of {sorted(_KINDS)}")
            key = cs.group_key()
            if key not in key_to_group:
                key_to_group[key] = len(self.groups)
                self.groups.append(CacheGroup(len(self.groups), cs.kind, cs.window, self.page_size))
            g = key_to_group[key]
            self.groups[g].entries.append(i)
            self._entry_group.append(g)
        # the bookkeeping itself, natively
        self._lib = native.lib()
        G = len(self.groups)
        kinds = (ctypes.c_int * max(G, 1))(*[_KINDS[g.kind] for g in self.groups])
        windows = (ctypes.c_int * max(G, 1))(*[g.window for g in self.groups])
        self._h = ctypes.c_void_p(self._lib.ia_cache_create(G, kinds, windows, self.page_size, int(config.num_pages),
                                                            int(config.num_state_slots)))
        if not self._h:
            raise ValueError("the cache could not be created: page_size, num_pages must be positive, slots not negative")
        for g in self.groups:
            g.allocator = PageAllocator(0, _view=self._lib.ia_cache_group_pool(self._h, g.index), _owner=self)
        self.slots = StateSlotPool(config.num_state_slots, _view=self._h, _owner=self)
        self._ids: Dict[Hashable, int] = {}          # request -> its number in the native bookkeeping
        self._names: Dict[int, Hashable] = {}
        self._next_id = 0
        self._per_group = (ctypes.c_int * max(G, 1))()
        # device memory: per schedule entry the pools that its mixer's CacheSpec declares, by name
        self.pages: List[Dict[str, torch.Tensor]] = [{} for _ in needs]
        self.state: List[Optional[torch.Tensor]] = [None] * len(needs)
        if device is not None:
            for i, (cs, ss) in enumerate(needs):
                if cs is not None:
                    for pt in cs.payload:
                        self.pages[i][pt.name] = torch.zeros(pt.pool_shape(int(config.num_pages), self.page_size),
                                                             dtype=pt.dtype or dtype, device=device)
                if ss is not None:
                    self.state[i] = torch.zeros((config.num_state_slots,) + tuple(ss.shape), dtype=ss.dtype,
                                                device=device)

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.ia_cache_destroy(self._h)
            self._h = None

    def _fail(self) -> None:
        """Raise the native call's error, with the request's own name in place of its number."""
        msg = self._lib.ia_cache_error(self._h).decode()
        msg = re.sub(r"request #(\d+)", lambda m: f"request {self._names.get(int(m.group(1)), m.group(0))!r}", msg)
        raise PageError(msg)

    def _id(self, req: Hashable) -> int:
        i = self._ids.get(req)
        if i is None:
            raise PageError(f"request {req!r} is not admitted")
        return i

    @property
    def k_pages(self) -> List[Optional[torch.Tensor]]:
        """Per schedule entry the pool named "k" (None where the entry has none)."""
        return [p.get("k") for p in self.pages]

    @property
    def v_pages(self) -> List[Optional[torch.Tensor]]:
        return [p.get("v") for p in self.pages]

    def native_handle(self) -> ctypes.c_void_p:
        return self._h

    def request_id(self, req: Hashable) -> int:
        """The request's number in the native bookkeeping."""
        return self._id(req)

    def request_ids(self, reqs: Sequence[Hashable]) -> List[int]:
        """The numbers of several requests, all admitted."""
        ids = self._ids
        try:
            return [ids[r] for r in reqs]
        except KeyError as e:
            raise PageError(f"request {e.args[0]!r} is not admitted") from None

    # ---- requests -------------------------------------------------------------
    def has(self, req: Hashable) -> bool:
        return req in self._ids

    def requests(self) -> List[Hashable]:
        return list(self._ids)

    def admit(self, req: Hashable) -> bool:
        """Give the request empty block tables and a state slot; False when no slot is free."""
        if req in self._ids:
            raise PageError(f"request {req!r} is admitted twice")
        rid = self._next_id
        slot = int(self._lib.ia_cache_admit(self._h, rid))
        if slot == native.HOST_ERROR:
            self._fail()
        if slot < 0:
            return False
        self._next_id += 1
        self._ids[req] = rid
        self._names[rid] = req
        for st in self.state:
            if st is not None:
                st[slot].zero_()
        return True

    def state_slot(self, req: Hashable) -> int:
        return int(self._lib.ia_cache_state_slot(self._h, self._id(req)))

    def num_tokens(self, req: Hashable) -> int:
        return int(self._lib.ia_cache_num_tokens(self._h, self._id(req)))

    def pages_needed(self, req: Optional[Hashable], n_new: int) -> List[int]:
        """Per group, the pages that n_new more tokens of the request would take from the pool
        (a request that is not admitted yet holds nothing)."""
        rid = self._ids.get(req) if req is not None else None
        self._lib.ia_cache_pages_needed(self._h, int(rid is not None), rid or 0, int(n_new), self._per_group)
        return list(self._per_group[:len(self.groups)])

    def tokens_that_fit(self, req: Optional[Hashable], promised: Optional[Sequence[int]] = None) -> int:
        """How many more tokens of the request the pool can hold, with ``promised[g]`` pages of
        every group already spoken for."""
        rid = self._ids.get(req) if req is not None else None
        prom = (ctypes.c_int * max(len(self.groups), 1))(*promised) if promised is not None else None
        return int(self._lib.ia_cache_tokens_that_fit(self._h, int(rid is not None), rid or 0, prom))

    def can_reserve(self, req: Hashable, n_new: int) -> bool:
        return self._lib.ia_cache_can_reserve(self._h, self._id(req), int(n_new)) == 1

    def reserve(self, req: Hashable, n_new: int) -> bool:
        """Pages for the next n_new tokens in every group, or nothing at all."""
        return self._lib.ia_cache_reserve(self._h, self._id(req), int(n_new)) == 1

    def step_fits(self, reqs: Sequence[Hashable], q_lens: Sequence[int]) -> bool:
        """Whether the pools and the state slots can take a whole step: ``q_lens[i]`` more tokens of
        ``reqs[i]``, admitted or not."""
        n = len(reqs)
        ids = [self._ids.get(r) for r in reqs]
        return self._lib.ia_cache_step_fits(
            self._h, n, (ctypes.c_int64 * max(n, 1))(*[i or 0 for i in ids]),
            (ctypes.c_int * max(n, 1))(*[int(i is not None) for i in ids]), (ctypes.c_int * max(n, 1))(*q_lens)) == 1

    def step_arrays(self, reqs: Sequence[Hashable], q_lens: Sequence[int]):
        """A step's requests (all admitted) and token counts as the native calls take them; ``reserve_step`` and
        ``commit_step`` of one step can share them."""
        n = len(reqs)
        return n, (ctypes.c_int64 * max(n, 1))(*self.request_ids(reqs)), (ctypes.c_int * max(n, 1))(*q_lens)

    def reserve_step(self, reqs: Sequence[Hashable], q_lens: Sequence[int], arrays=None) -> bool:
        """Pages for ``q_lens[i]`` more tokens of every ``reqs[i]`` (all admitted), or nothing at all."""
        rc = self._lib.ia_cache_reserve_step(self._h, *(arrays or self.step_arrays(reqs, q_lens)))
        if rc == native.HOST_ERROR:
            self._fail()
        return rc == 1

    def unreserve_step(self, reqs: Sequence[Hashable]) -> None:
        """A step whose pages were reserved did not run: the pages beyond what each request's stored tokens
        need go back to the pools."""
        n = len(reqs)
        if self._lib.ia_cache_unreserve_step(self._h, n, (ctypes.c_int64 * max(n, 1))(*self.request_ids(reqs))) != 0:
            self._fail()
        self._poison()

    def commit_step(self, reqs: Sequence[Hashable], q_lens: Sequence[int], arrays=None) -> None:
        """``commit`` for every request of a step."""
        if self._lib.ia_cache_commit_step(self._h, *(arrays or self.step_arrays(reqs, q_lens))) != 0:
            self._fail()
        self._poison()

    def commit(self, req: Hashable, n_new: int) -> None:
        """The n_new tokens are stored; pages that a window has passed go back to the pool."""
        if self._lib.ia_cache_commit(self._h, self._id(req), int(n_new)) != 0:
            self._fail()
        self._poison()

    def release(self, req: Hashable) -> None:
        """The request is over (finished, cancelled or preempted): everything it holds goes back."""
        rid = self._ids.get(req)
        if rid is None:
            raise PageError(f"request {req!r} is released but not admitted")
        if self._lib.ia_cache_release(self._h, rid) != 0:
            self._fail()
        del self._ids[req]
        del self._names[rid]
        self._poison()

    def forget(self, req: Hashable) -> None:
        """The native side has released the request already (while scheduling): drop its name here."""
        rid = self._ids.pop(req, None)
        if rid is not None:
            del self._names[rid]
            if self._lib.ia_cache_has(self._h, rid):
                raise PageError(f"request {req!r} is forgotten but still holds pages")

    def poison_freed(self) -> None:
        """After native calls that released requests themselves: what they gave back is filled with NaN
        (when ``poison_freed_pages`` is set)."""
        self._poison()

    def _poison(self) -> None:
        """Fill the pages that the last commit or release gave back with NaN (when asked to)."""
        if not self.config.poison_freed_pages or self.device is None:
            return
        n = int(self._lib.ia_cache_last_freed(self._h, None, 0))
        if n == 0:
            return
        pairs = (ctypes.c_int * (2 * n))()
        self._lib.ia_cache_last_freed(self._h, pairs, n)
        for g in self.groups:
            pages = [pairs[2 * i + 1] for i in range(n) if pairs[2 * i] == g.index]
            if not pages:
                continue
            idx = torch.tensor(pages, dtype=torch.long, device=self.device)
            for e in g.entries:
                for pool in self.pages[e].values():
                    if pool.dtype.is_floating_point:
                        pool.index_fill_(0, idx, float("nan"))

    # ---- what a step needs --------------------------------------------------------
    def free_pages(self, group: int = 0) -> int:
        return self.groups[group].allocator.num_free

    def block_table(self, group: int, req: Hashable) -> BlockTable:
        """A copy of the request's block table in the group."""
        rid = self._id(req)
        tokens, first = ctypes.c_int64(0), ctypes.c_int(0)
        n = int(self._lib.ia_cache_table(self._h, int(group), rid, None, 0, ctypes.byref(tokens), ctypes.byref(first)))
        if n == native.HOST_ERROR:
            self._fail()
        pages = (ctypes.c_int * max(n, 1))()
        self._lib.ia_cache_table(self._h, int(group), rid, pages, n, None, None)
        return BlockTable(list(pages[:n]), tokens.value, first.value)

    def token_slots(self, group: int, req: Hashable, start: int, n: int) -> np.ndarray:
        """page * page_size + offset of positions start .. start+n-1 (pages must be reserved)."""
        out = np.empty(max(n, 0), dtype=np.int32)
        if self._lib.ia_cache_token_slots(self._h, int(group), self._id(req), int(start), int(n),
                                          out.ctypes.data_as(ctypes.POINTER(ctypes.c_int32))) != 0:
            self._fail()
        return out

    def views(self) -> List[CacheView]:
        """One CacheView per schedule entry."""
        out = []
        for i, src in enumerate(self._cache_of):
            j = i if src is None else src
            out.append(CacheView(group=self._entry_group[j], pages=self.pages[j], writable=src is None,
                                 state=self.state[j]))
        return out

    # ---- invariants (tests) ---------------------------------------------------------
    def check(self) -> None:
        """Every page is free or held by exactly one request; counts agree."""
        if self._lib.ia_cache_check(self._h) != 0:
            self._fail()
        if int(self._lib.ia_cache_num_requests(self._h)) != len(self._ids):
            raise PageError("the native bookkeeping and the names of the requests disagree")
