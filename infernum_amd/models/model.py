"""A decoder built from a :class:`ModelSpec`: the parts, their weights' names,
and the forward pass of one step over the schedule of layer runs.

This file holds no architecture: which parts a model has, and in which order
its layers run, is data (the reference builds the same sequence as a graph,
infernum-llama/src/graph_builder.rs:399-549 for whole prompts and :756-921 for
batched decoding; here one forward serves both).
"""
from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import torch

from ..parts.base import (Block, CacheSpec, CacheView, ModelSpec, Part, PartSpec, Runtime, StateSpec, StepContext,
                          WeightSpec, block_factory, make_part)


def _needs(part: Part) -> Tuple[Optional[CacheSpec], Optional[StateSpec]]:
    return (part.cache_spec() if hasattr(part, "cache_spec") else None,
            part.state_spec() if hasattr(part, "state_spec") else None)


class DecoderModel:
    def __init__(self, spec: ModelSpec, rt: Runtime):
        self.spec = spec
        self.rt = rt
        self._parts: List[Tuple[str, Part]] = []        # (prefix, part) of everything that has weights
        self.embedding = self._make("embedding", spec.embedding)
        self.blocks: List[Block] = []
        for ls in spec.layers:
            mixer = self._make("mixer", ls.mixer)
            ff = self._make("feed_forward", ls.feed_forward) if ls.feed_forward is not None else None
            n1 = self._make("norm", ls.mixer_norm) if ls.mixer_norm is not None else None
            n2 = self._make("norm", ls.feed_forward_norm) if ls.feed_forward_norm is not None else None
            extra = {name: (self._make("norm", ps) if isinstance(ps, PartSpec) else self._make(*ps))
                     for name, ps in ls.extra.items()}
            self.blocks.append(block_factory(ls.block)(rt, mixer, ff, n1, n2, extra))
        self.final_norm = self._make("norm", spec.final_norm) if spec.final_norm is not None else None
        self.head = self._make("head", spec.head)
        self._check_schedule()

    def _make(self, category: str, ps: PartSpec) -> Part:
        part = make_part(category, ps, self.rt)
        self._parts.append((ps.prefix, part))
        return part

    def _check_schedule(self) -> None:
        n_layers = len(self.spec.layers)
        for i, e in enumerate(self.spec.schedule):
            if not 0 <= e.layer < n_layers:
                raise ValueError(f"schedule entry {i} names layer {e.layer}, but there are {n_layers} layers")
            if e.cache_of is not None:
                if not 0 <= e.cache_of < i:
                    raise ValueError(f"schedule entry {i} reads the cache of entry {e.cache_of}, which does not run before it")
                if self.spec.schedule[e.cache_of].cache_of is not None:
                    raise ValueError(f"schedule entry {i} reads entry {e.cache_of}, which has no cache of its own")
                a = {n: _needs(p) for n, p in self.blocks[e.layer].cached_parts().items()}
                b = {n: _needs(p) for n, p in self.blocks[self.spec.schedule[e.cache_of].layer].cached_parts().items()}
                if a != b:
                    raise ValueError(f"schedule entry {i} cannot read the cache of entry {e.cache_of}: {a} != {b}")

    def graph_safe(self) -> bool:
        """True when every part may be recorded into a HIP graph (it launches kernels on the current stream
        and reads nothing back from the device on the host)."""
        return all(getattr(part, "graph_safe", False) for _, part in self._parts) and \
            all(getattr(b, "graph_safe", False) for b in self.blocks)

    # ---- weights -------------------------------------------------------------
    def expected_weights(self) -> Dict[str, WeightSpec]:
        """Full tensor name -> what is expected of it."""
        out: Dict[str, WeightSpec] = {}
        for prefix, part in self._parts:
            for local, ws in part.weights().items():
                name = prefix + local
                if name in out and out[name] != ws:
                    raise ValueError(f"two parts want tensor {name!r} differently")
                out[name] = ws
        return out

    def load_weights(self, tensors: Dict[str, torch.Tensor]) -> None:
        """``tensors``: full name -> device tensor, already checked and converted."""
        for prefix, part in self._parts:
            wanted = part.weights()
            if wanted:
                part.load({local: tensors[prefix + local] for local in wanted})

    def step_needs(self) -> Dict[str, set]:
        """What the parts want packed with every step: kind of array -> the set of its parameters."""
        out: Dict[str, set] = {}
        for _, part in self._parts:
            for kind, param in part.step_needs().items():
                out.setdefault(kind, set()).add(param)
        return out

    # ---- cache needs ---------------------------------------------------------
    def _cached(self) -> List[Tuple[int, str, Part]]:
        """(schedule entry, name, part) of every part that keeps something between steps, in the schedule's order."""
        return [(i, name, part) for i, e in enumerate(self.spec.schedule)
                for name, part in self.blocks[e.layer].cached_parts().items()]

    def cache_needs(self) -> List[Tuple[Optional[CacheSpec], Optional[StateSpec]]]:
        """Per cached part of every schedule entry (mostly one: the mixer): the pages and the per-request state it
        wants (None, None for an entry that reads another entry's)."""
        return [(None, None) if self.spec.schedule[i].cache_of is not None else _needs(part)
                for i, _, part in self._cached()]

    def cache_sources(self) -> List[Optional[int]]:
        """Per cached part: the index (in ``cache_needs``) of the part whose pages and state it reads, or None for
        its own."""
        index = {(i, name): k for k, (i, name, _) in enumerate(self._cached())}
        return [None if self.spec.schedule[i].cache_of is None else index[(self.spec.schedule[i].cache_of, name)]
                for i, name, _ in self._cached()]

    def entry_views(self, views: List[CacheView]) -> List[CacheView]:
        """From the cache manager's views (one per cached part) the view of each schedule entry: the mixer's,
        with the layer's further cached parts under their names in ``others``."""
        per_entry: List[Dict[str, CacheView]] = [{} for _ in self.spec.schedule]
        for (i, name, _), view in zip(self._cached(), views):
            per_entry[i][name] = view
        out = []
        for named in per_entry:
            main = named.pop("mixer", None) or CacheView()
            main.others = named
            out.append(main)
        return out

    # ---- the step as a program ------------------------------------------------------
    def native(self, program, views: List[CacheView]) -> None:
        """Every part writes its operations into ``program`` (engine/program.StepProgram), in the order in which
        ``_forward`` below calls the parts' ``forward``."""
        self.embedding.native(program, None)
        for e, view in zip(self.spec.schedule, views):
            self.blocks[e.layer].native(program, view)
        if self.final_norm is not None:
            self.final_norm.native(program, None, rows=True)
        else:
            pending, H, dt = program.pending, self.spec.hidden_size, self.rt.dtype

            def wanted_rows(ctx: StepContext) -> None:
                from ..kernels import api as K
                n, rows = ctx.num_tokens, ctx.logit_rows
                if rows.numel() == 0:
                    return
                h, delta = program.h.view(torch.float32, n, H), program.read(pending, n)
                if delta is not None:
                    K.residual_add(h, delta.joined(dt) if isinstance(delta, K.SplitSum) else delta)
                program.x.view(dt, rows.numel(), H).copy_(h.index_select(0, rows.long()))
            program.python(wanted_rows, "wanted rows")
            program.pending = None
        self.head.native(program, None)

    # ---- one step --------------------------------------------------------------
    def forward(self, ctx: StepContext, views: List[CacheView]) -> torch.Tensor:
        """Runs the tokens of ``ctx`` and returns fp32 logits [R, V] at ctx.logit_rows."""
        from ..kernels.api import on_current_stream
        with on_current_stream():
            return self._forward(ctx, views)

    def _forward(self, ctx: StepContext, views: List[CacheView]) -> torch.Tensor:
        h = self.embedding.forward(ctx)
        pending: Optional[torch.Tensor] = None
        for e, view in zip(self.spec.schedule, views):
            pending = self.blocks[e.layer].forward(h, pending, ctx, view)
        rows = ctx.logit_rows
        if rows.numel() == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=h.device)
        if self.final_norm is not None:
            f = self.final_norm.forward(h, pending, rows=rows)
        else:
            from ..kernels import api as K
            if pending is not None:
                K.residual_add(h, pending.joined(self.rt.dtype) if isinstance(pending, K.SplitSum) else pending)
            f = h.index_select(0, rows.long()).to(self.rt.dtype)
        return self.head.forward(f)
