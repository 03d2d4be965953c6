"""RMSNorm on the fp32 residual stream, with the residual add fused in.

out = s * (1 / sqrt(mean(s^2) + eps)) * w with s = h + delta: eps inside the
root, the weight multiplies (infernum-cuda/kernels/rmsnorm.cu:79-80,89-93; fused
add: kernels/add_rmsnorm.cu:53-109).  The sum stays fp32 here, where the
reference rounds it to bf16 between the add and the norm.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import api as K
from .base import Norm, Runtime, WeightSpec, register_part


class RMSNorm(Norm):
    graph_safe = True
    def __init__(self, rt: Runtime, size: int, eps: float, init: tuple = ("ones",)):
        super().__init__(rt)
        self.size = int(size)
        self.eps = float(eps)
        self.init = tuple(init)
        self.weight: Optional[torch.Tensor] = None

    def weights(self) -> Dict[str, WeightSpec]:
        # a norm weight stored in fp32 stays fp32; the kernel reads either
        return {"weight": WeightSpec((self.size,), init=self.init, follows_compute_dtype=False)}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.weight = tensors["weight"].contiguous()

    def forward(self, h: torch.Tensor, delta, out: Optional[torch.Tensor] = None,
                rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        n = rows.numel() if rows is not None else h.shape[0]
        if out is None:
            out = torch.empty((n, self.size), dtype=self.rt.dtype, device=h.device)
        return K.add_rmsnorm(h, delta, self.weight, self.eps, out, rows)


    def native(self, program, view=None, rows: bool = False) -> None:
        """One launch per form the pending delta can have (none, a tensor, partial sums of a split product)."""
        if type(self).forward is not RMSNorm.forward:
            return super().native(program, view, rows)          # a subclass that computes something else
        from ..engine.program import ALWAYS, STREAM, Guard
        base = Guard.between(program.R, 1) if rows else ALWAYS
        for alt in (program.pending.alts if program.pending is not None else [None]):
            delta, code, splits, when = None, program.act_code, 1, base
            if alt is not None:
                if not alt.splits and alt.dtype != self.rt.dtype:
                    raise K.KernelError("add_rmsnorm: the delta must have the activations' dtype")
                delta, when = alt.where, base & alt.when
                code, splits = (K.DTYPE_CODE[torch.float32], alt.splits) if alt.splits else (program.act_code, 1)
            program.op("core", "ia_add_rmsnorm",
                       [program.h, delta, code, splits, program.N, program.act_code, self.weight,
                        K.DTYPE_CODE[self.weight.dtype], program.x, program.logit_rows if rows else None,
                        program.R if rows else program.N, self.size, float(self.eps), STREAM], when)
        program.pending = None


register_part("norm", "rmsnorm", RMSNorm)
