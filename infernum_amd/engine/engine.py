"""The step function: one batch of (request, its next tokens) through the model.

A step takes any mix of portions of prompts and single decoded tokens, cut
anywhere, runs only those tokens against what earlier steps left in the cache,
and returns fp32 logits at the wanted places.  The reference has two calls for
this, one whole prompt of one request (``forward_prefill``, infernum/src/model.rs:
96-103, whose start position the CUDA engine ignores,
infernum-cuda/src/inner/cuda_graph_engine.rs:1318,1363) and one token of each of B
requests (``forward_batch_decode``, model.rs:121-132); here they are one.

The engine owns the model and the cache manager.  It packs the batch into one
int32 buffer, copies it to the device once, and runs the model's forward pass.
"""
from __future__ import annotations

from typing import Any, Dict, Hashable, List, Optional, Sequence

import numpy as np
import torch

from ..cache import CacheConfig, CacheManager
from ..kernels.staging import PinnedUpload
from ..models.model import DecoderModel
from ..parts.base import Runtime

from .batch import POW2_WIDTH, StepEntry, StepError, check_entries, pack_step  # noqa: F401  (StepError is part of this module's face)


class OutOfPages(RuntimeError):
    """The pool has too few free pages (or state slots) for this step; nothing was changed."""


# Recorded decode steps kept at a time.  Each holds its own logits ([requests, vocabulary] fp32) and its
# inputs; in continuous batching the number of live requests takes every value up to the largest batch, times
# a handful of table widths, so the table is bounded and the shape used longest ago makes room.
MAX_RECORDED_STEPS = 64


class _DecodeGraph:
    """A recorded decode step of one shape: its int32 inputs, the recorded launches, its logits."""

    __slots__ = ("inputs", "graph", "logits")

    def __init__(self, inputs: torch.Tensor, graph: "torch.cuda.CUDAGraph", logits: torch.Tensor):
        self.inputs, self.graph, self.logits = inputs, graph, logits


class Engine:
    """``use_graphs``: steps in which every request brings one token are recorded into a HIP graph per shape
    (number of requests, width of the block tables, number of wanted rows) the second time the shape comes,
    and replayed from then on: one launch instead of some hundred.  The step's int32 arrays are copied into
    the graph's own input buffer first; pages, state and weights are where they always are.  Models with a
    part that is not marked ``graph_safe`` (one that reads device memory on the host, say) run without."""

    def __init__(self, model: DecoderModel, cache_config: CacheConfig, use_graphs: bool = True,
                 executor: Optional[str] = None):
        self.model = model
        self.rt: Runtime = model.rt
        self.spec = model.spec
        self.cache = CacheManager(model.cache_needs(), model.cache_sources(), cache_config,
                                  dtype=self.rt.dtype, device=self.rt.device)
        self.views = model.entry_views(self.cache.views())          # one per schedule entry
        # row tiles that parts asked for: one height is laid out with the step's arrays, further ones are
        # made when a part asks (StepContext.row_tiles)
        heights = sorted(model.step_needs().get("row_tiles", ()))
        self._tile_rows = int(heights[0]) if heights else 0
        self.steps_run = 0
        from ..kernels.api import profiling
        self.use_graphs = (bool(use_graphs) and self.rt.device.type == "cuda" and model.graph_safe()
                           and not profiling())         # a replayed launch has no call to time
        self._graphs: Dict[tuple, _DecodeGraph] = {}
        self._shape_seen: Dict[tuple, int] = {}
        self._graph_pool = None
        self.graph_replays = 0
        self.max_recorded_steps = MAX_RECORDED_STEPS
        self._staging = PinnedUpload(self.rt.device) if self.rt.device.type == "cuda" else None
        # "native": the step's launches are made by the host library from one call, from the program that the
        # model's parts wrote (engine/program.py; a part without launchers of its own is called back); "parts":
        # by the parts' own forward, one Python call per launch (the twin that tests hold the program to, and
        # the way of INFERNUM_PROFILE=1).  The same launches either way.
        executor = executor or "native"
        if executor not in ("native", "parts"):
            raise ValueError(f"executor must be 'native' or 'parts', got {executor!r}")
        self.program = None
        if executor == "native" and self.rt.device.type == "cuda":
            from .program import build
            self.program = build(model, self.views, len(self.cache.groups), self.rt.max_tokens_per_step)

    # ---- building ------------------------------------------------------------------
    @staticmethod
    def runtime(dtype: Any = "bfloat16", device: Any = "cuda:0", max_tokens_per_step: int = 8192,
                kernels: str = "auto") -> Runtime:
        from ..kernels.api import KernelError
        dt = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32,
              "f32": torch.float32, torch.bfloat16: torch.bfloat16, torch.float32: torch.float32}.get(dtype)
        if dt is None:
            raise ValueError(f"dtype must be bfloat16 or float32, got {dtype!r}")
        dev = torch.device(device)
        if dev.type != "cuda" or not torch.cuda.is_available():
            raise KernelError("infernum_amd runs on a gfx950 GPU only: no GPU is visible (there is no CPU fallback)")
        return Runtime(dev, dt, max_tokens_per_step, kernels)

    @classmethod
    def from_pretrained(cls, model_dir: str, dtype: Any = "bfloat16", cache_config: Optional[CacheConfig] = None,
                        device: Any = "cuda:0", use_graphs: bool = True, executor: Optional[str] = None,
                        **runtime_kw: Any) -> "Engine":
        """Model class by config.json's model_type, weights from the folder's safetensors.
        ``kernels="generic"`` (a runtime keyword) runs every matrix product and the attention on the plain
        twins of the fast kernels, in either type."""
        from .. import models  # noqa: F401  (registers the architectures)
        from ..config.registry import load_config, model_spec_for
        from ..weights.loader import load_weights
        from ..kernels.api import load_library
        rt = cls.runtime(dtype, device, **runtime_kw)
        load_library("core")
        config = load_config(model_dir)
        model = DecoderModel(model_spec_for(config), rt)
        load_weights(model, model_dir)
        eng = cls(model, cache_config or CacheConfig(), use_graphs=use_graphs, executor=executor)
        eng.config = config
        return eng

    @classmethod
    def from_config(cls, config: Any, seed: int = 0, dtype: Any = "bfloat16",
                    cache_config: Optional[CacheConfig] = None, device: Any = "cuda:0",
                    spec_kw: Optional[Dict[str, Any]] = None, use_graphs: bool = True,
                    stored_as: Any = None, executor: Optional[str] = None, **runtime_kw: Any) -> "Engine":
        """Random weights made on the device from (config, seed); nothing is read or written.  They are the
        numbers of the folder that ``write_random_model`` writes from the same seed in ``stored_as`` (default:
        the compute type)."""
        from .. import models  # noqa: F401
        from ..config.registry import model_spec_for
        from ..weights.random_init import random_weights_on_device
        from ..kernels.api import load_library
        rt = cls.runtime(dtype, device, **runtime_kw)
        load_library("core")
        model = DecoderModel(model_spec_for(config, **(spec_kw or {})), rt)
        stored = {None: None, "bfloat16": torch.bfloat16, "float32": torch.float32}.get(stored_as, stored_as)
        random_weights_on_device(model, seed, stored)
        eng = cls(model, cache_config or CacheConfig(), use_graphs=use_graphs, executor=executor)
        eng.config = config
        return eng

    # ---- the step ------------------------------------------------------------------
    def pages_short(self, entries: Sequence[StepEntry]) -> bool:
        """True when the pools or the state slots cannot hold this step's new tokens."""
        return not self.cache.step_fits([e.request for e in entries], [len(e.tokens) for e in entries])

    supports_device_tokens = True

    def step(self, entries: Sequence[StepEntry], device_tokens: Optional[tuple] = None,
             borrow_logits: bool = False) -> torch.Tensor:
        """Run one batch; returns logits [sum(len(want)), vocab] fp32 in the order of entries and of ``want``.

        ``device_tokens`` = (tokens, index): int32 tokens on the device (what the last step's sampling left
        there) and, per entry, the place among them of the entry's single token, or -1 for an entry whose
        tokens are given; the batch takes those tokens on the device, and the host never sees them before.
        ``borrow_logits``: the caller uses the logits before the next step and does not keep them (a recorded
        step's logits are the recording's own and are written again by the next replay)."""
        entries = [e if isinstance(e, StepEntry) else StepEntry(*e) for e in entries]
        V = self.spec.vocab_size
        if not entries:
            return torch.empty((0, V), dtype=torch.float32, device=self.rt.device)
        check_entries(entries, V, self.rt.max_tokens_per_step)
        if self.pages_short(entries):
            total = sum(len(e.tokens) for e in entries)
            raise OutOfPages(f"not enough free pages or state slots for a step of {total} tokens")
        cache = self.cache
        reqs, q_lens = [e.request for e in entries], [len(e.tokens) for e in entries]
        fresh = [r for r in reqs if not cache.has(r)]
        for r in fresh:
            cache.admit(r)
        reserved = False
        try:
            arrays = cache.step_arrays(reqs, q_lens)        # once for the reservation and the commit
            if not cache.reserve_step(reqs, q_lens, arrays):
                raise OutOfPages("the pages this step was checked for are gone")   # step_fits said they were there
            reserved = True
            if device_tokens is not None:
                for e, j in zip(entries, device_tokens[1]):
                    if j >= 0 and len(e.tokens) != 1:
                        raise StepError(f"request {e.request!r}: a token from the device stands for exactly one token")
            if all(n == 1 for n in q_lens):
                logits = self._decode_step(entries, device_tokens, borrow_logits)
            else:
                packed = pack_step(cache, entries, tile_rows=self._tile_rows)
                ctx = packed.context(self._stage(packed, device_tokens))
                logits = self._forward(ctx)
        except BaseException:
            # the step did not run to its end: requests that came with it leave again, the others give back
            # the pages that were reserved for it; what earlier steps stored stays as it was
            for r in fresh:
                cache.release(r)
            if reserved:
                cache.unreserve_step([r for r in reqs if r not in fresh])
            raise
        cache.commit_step(reqs, q_lens, arrays)
        self.steps_run += 1
        return logits

    def _forward(self, ctx) -> torch.Tensor:
        if self.program is not None:
            from ..kernels.api import on_current_stream
            with on_current_stream():
                return self.program.run(ctx)
        return self.model.forward(ctx, self.views)

    def _stage(self, packed, device_tokens: Optional[tuple], out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """The step's int32 arrays on the device (in ``out`` when given), by way of pinned memory and a kernel of
        the stream; single tokens that the last step chose on the device go into the token ids there."""
        if self._staging is None:
            from ..kernels.api import KernelError
            raise KernelError("no GPU is visible: infernum_amd runs on a gfx950 GPU only (there is no CPU fallback)")
        rows = source = None
        if device_tokens is not None:
            source, index = device_tokens
            nd = packed.num_decode                          # requests that bring one token are the first rows
            rows = np.fromiter((index[i] for i in packed.order[:nd]), dtype=np.int32, count=nd)
            if nd == 0 or int(rows.max()) < 0:
                rows = source = None
            elif int(rows.max()) >= source.numel():
                raise StepError(f"a token is to come from place {int(rows.max())} of the last step's {source.numel()} choices")
        return self._staging.upload(packed.host, out=out, token_off=packed.offsets[0], token_rows=rows, source=source)

    def _decode_step(self, entries: Sequence[StepEntry], device_tokens: Optional[tuple] = None,
                     borrow_logits: bool = False) -> torch.Tensor:
        """Every request brings one token.  Block tables are widened to a power of two of pages, and the
        kernels are told that width as the longest length, so that a shape's launches are the same from
        step to step, recorded or not."""
        cache = self.cache
        packed = pack_step(cache, entries, bt_width=POW2_WIDTH, tile_rows=self._tile_rows)
        widths = tuple(shape[1] for shape in packed.bt_shapes)           # one width per group of the cache
        limit = max(widths, default=0) * cache.page_size
        key = (len(entries), widths, packed.num_logit_rows)
        g = self._graphs.get(key)
        if g is not None:
            self._graphs[key] = self._graphs.pop(key)       # most recently used last
            self._stage(packed, device_tokens, out=g.inputs)
            g.graph.replay()
            self.graph_replays += 1
            return g.logits if borrow_logits else g.logits.clone()
        seen = self._shape_seen.get(key, 0)
        self._shape_seen[key] = seen + 1
        inputs = self._stage(packed, device_tokens)
        ctx = packed.context(inputs)
        ctx.max_total_len = max(limit, ctx.max_total_len)
        if not self.use_graphs or seen < 1:
            return self._forward(ctx)
        # second time this shape comes: record it (kernels were loaded by the first, eager run).  The device
        # is idle before a recording is dropped: a replay of it may still be queued (the host runs a step ahead)
        torch.cuda.synchronize(self.rt.device)
        while len(self._graphs) >= self.max_recorded_steps:
            oldest = next(iter(self._graphs))
            del self._graphs[oldest]                        # its memory returns to the graphs' pool
            self._shape_seen.pop(oldest, None)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, pool=self._graph_pool):
            logits = self._forward(ctx)
        if self._graph_pool is None:
            self._graph_pool = graph.pool()
        self._graphs[key] = _DecodeGraph(inputs, graph, logits)
        graph.replay()
        self.graph_replays += 1
        return logits if borrow_logits else logits.clone()

    def decode_greedy(self, requests: Sequence[Hashable], tokens: Sequence[int]) -> List[int]:
        """One decode step for requests that each bring one token; returns each one's next token (argmax)."""
        from ..kernels import api as K
        logits = self.step([StepEntry(r, [int(t)], [0]) for r, t in zip(requests, tokens)])
        out = torch.empty(logits.shape[0], dtype=torch.int32, device=logits.device)
        K.argmax(logits, out)
        return out.tolist()

    def end(self, request: Hashable) -> None:
        """The request is finished: its pages and its state slot are given back."""
        if self.cache.has(request):
            self.cache.release(request)
