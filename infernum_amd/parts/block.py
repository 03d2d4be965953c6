"""Arrangements of a layer's parts around the fp32 residual stream.

``prenorm``: h' = h + mixer(norm1(h)); h'' = h' + feed_forward(norm2(h'))
(infernum-llama/src/graph_builder.rs:453-507).  Each add is carried as a pending
delta into the next norm, which adds and normalises in one pass over the row
(the reference's add_rmsnorm fusion, infernum/src/graph/optimizer.rs:105-174,
there limited to adds with one consumer).
"""
from __future__ import annotations

from typing import Optional

import torch

from .base import Block, CacheView, StepContext, register_part


class PreNormBlock(Block):
    graph_safe = True
    def forward(self, h: torch.Tensor, pending: Optional[torch.Tensor], ctx: StepContext,
                cache: CacheView) -> torch.Tensor:
        n = self.mixer_norm.forward(h, pending)
        a = self.mixer.forward(n, ctx, cache)
        n = self.feed_forward_norm.forward(h, a)
        return self.feed_forward.forward(n, ctx)

    def native(self, program, view: CacheView) -> bool:
        if type(self) is not PreNormBlock or self.extra or None in (self.feed_forward, self.mixer_norm,
                                                                    self.feed_forward_norm):
            return False
        return (self.mixer_norm.native(program, None) and self.mixer.native(program, view)
                and self.feed_forward_norm.native(program, None) and self.feed_forward.native(program, None))


register_part("block", "prenorm", PreNormBlock)
