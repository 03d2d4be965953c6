"""Token embedding and output head.

h[t] = E[ids[t]] without scaling (infernum-llama/src/graph_builder.rs:442);
logits = f W^T for the wanted rows only, in fp32 straight from the fp32
accumulators (:533-536).  When the file has no head matrix, the embedding
matrix stands in: the reference decides that by the file's contents, not by
``tie_word_embeddings`` (infernum-cuda/src/inner/cuda_graph_engine.rs:225-232);
the two then share one buffer here.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import api as K
from .base import Embedding, Head, Runtime, StepContext, WeightSpec, register_part
from .linear import emit_linear, linear


class TokenEmbedding(Embedding):
    graph_safe = True
    def __init__(self, rt: Runtime, vocab_size: int, hidden_size: int, init_std: float = 0.02):
        super().__init__(rt)
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.init_std = init_std
        self.table: Optional[torch.Tensor] = None

    def weights(self) -> Dict[str, WeightSpec]:
        return {"weight": WeightSpec((self.vocab_size, self.hidden_size), ("normal", self.init_std))}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.table = tensors["weight"].contiguous()

    def forward(self, ctx: StepContext) -> torch.Tensor:
        h = torch.empty((ctx.num_tokens, self.hidden_size), dtype=torch.float32, device=self.table.device)
        return K.embed(self.table, ctx.token_ids, h)

    def native(self, program, view=None) -> None:
        if type(self).forward is not TokenEmbedding.forward:
            return super().native(program, view)
        from ..engine.program import STREAM
        program.op("core", "ia_embed", [self.table, K.DTYPE_CODE[self.table.dtype], program.token_ids, program.h,
                                        program.N, self.hidden_size, self.vocab_size, STREAM])
        program.pending = None


class LinearHead(Head):
    graph_safe = True
    def __init__(self, rt: Runtime, vocab_size: int, hidden_size: int, fallback: Optional[str] = None,
                 tied: bool = False, init_std: float = 0.02):
        super().__init__(rt)
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.fallback, self.tied, self.init_std = fallback, bool(tied), init_std
        self.weight: Optional[torch.Tensor] = None

    def weights(self) -> Dict[str, WeightSpec]:
        return {"weight": WeightSpec((self.vocab_size, self.hidden_size), ("normal", self.init_std),
                                     fallback=self.fallback, write_when_random=not self.tied)}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        # no second copy laid out for the weight-streaming kernel: since that kernel's tiles of rows walk K from
        # starts of their own, the file's layout serves the head as well (128,256 x 4,096 on an MI355X: 187.1 against
        # 187.6 us at 8 rows, 190.0 against 189.0 at 16), and a copy would be another gigabyte
        self.weight = tensors["weight"]

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return linear(x, self.weight, out_dtype=torch.float32, kernels=self.rt.kernels)

    def native(self, program, view=None) -> None:
        if type(self).forward is not LinearHead.forward:
            return super().native(program, view)
        emit_linear(program, program.x, program.R, self.weight, torch.float32, None, False, program.logits, "head")


register_part("embedding", "token", TokenEmbedding)
register_part("head", "linear", LinearHead)
