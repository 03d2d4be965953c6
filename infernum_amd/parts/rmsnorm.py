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


    def native(self, program, view, final: bool = False) -> bool:
        if type(self) is not RMSNorm:
            return False
        program.add_norm(self.weight, self.eps, final=final)
        return True


register_part("norm", "rmsnorm", RMSNorm)
