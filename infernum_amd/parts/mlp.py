"""SwiGLU feed-forward: down( silu(x Wg^T) * (x Wu^T) ), no bias, exact SiLU.

infernum-llama/src/graph_builder.rs:498-507; infernum-cuda/kernels/silu.cu:36-40.
Gate and up are one [2I, H] matrix, so one product makes both.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import FeedForward, Runtime, StepContext, WeightSpec, register_part
from .linear import emit_linear, linear, prepare_weights


class SwiGLUFeedForward(FeedForward):
    graph_safe = True
    def __init__(self, rt: Runtime, hidden_size: int, intermediate_size: int, init_std: float = 0.02):
        super().__init__(rt)
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.init_std = init_std
        self.w_gate_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None

    def weights(self) -> Dict[str, WeightSpec]:
        H, I = self.hidden_size, self.intermediate_size
        init = ("normal", self.init_std)
        return {
            "gate_proj.weight": WeightSpec((I, H), init),
            "up_proj.weight": WeightSpec((I, H), init),
            "down_proj.weight": WeightSpec((H, I), init),
        }

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.w_gate_up = torch.cat([tensors["gate_proj.weight"], tensors["up_proj.weight"]], dim=0).contiguous()
        self.w_down = tensors["down_proj.weight"].contiguous()
        prepare_weights(self.rt, [(self.w_gate_up, "swiglu", False), (self.w_down, None, True)])

    def forward(self, x: torch.Tensor, ctx: Optional[StepContext] = None):
        act = linear(x, self.w_gate_up, epilogue="swiglu", kernels=self.rt.kernels)
        return linear(act, self.w_down, keep_split=True, kernels=self.rt.kernels)

    def native(self, program, view=None) -> None:
        if type(self).forward is not SwiGLUFeedForward.forward:
            return super().native(program, view)
        dt = self.rt.dtype
        act = emit_linear(program, program.x, program.N, self.w_gate_up, dt, "swiglu", False, "swiglu.act", "swiglu.gate_up")
        program.pending = emit_linear(program, act.tensor(), program.N, self.w_down, dt, None, True, "swiglu.out",
                                      "swiglu.down")


register_part("feed_forward", "swiglu", SwiGLUFeedForward)
