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

    def native(self, program, view: CacheView) -> None:
        if type(self).forward is not PreNormBlock.forward:
            return super().native(program, view)
        self.mixer_norm.native(program, None)
        self.mixer.native(program, view)
        self.feed_forward_norm.native(program, None)
        self.feed_forward.native(program, None)


register_part("block", "prenorm", PreNormBlock)
