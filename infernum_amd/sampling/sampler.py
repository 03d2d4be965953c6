"""Choice of the next token of every wanted row of a step, on the device.

Greedy rows take the argmax kernel (lowest index wins a tie; the reference leaves
ties open, infernum-cuda/kernels/argmax.cu:14-86).  Sampled rows go through the
repetition penalty, temperature, softmax, nucleus and inverse CDF of
infernum-cuda/src/inner/cuda/ops/sample.rs:94-159, which the reference runs on the
host over a downloaded row; here the row stays on the device and one int32 per row
comes back.  Three stated differences: the nucleus takes every token that ties with
the one that crosses ``top_p``; the CDF walks the nucleus in the order of the
vocabulary rather than by falling probability (no sort of the vocabulary); and
masses are added as integers, exp((x - max) / T) * 2^31 rounded down, so that sums
do not depend on their order: a token whose probability is below 5e-10 of the
likeliest one's is never drawn.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Sequence

import torch

from ..kernels import api as K
from .params import SamplingParams
from .rng import token_uniform


@dataclass
class RowRequest:
    """What is needed to choose the token of one row of logits."""

    sampling: Optional[SamplingParams]          # None: greedy
    generated_before: int = 0                   # tokens the request has generated so far
    history: Sequence[int] = ()                 # prompt and generated tokens so far (for the penalty)


class Sampler:
    def __init__(self, device: torch.device):
        self.device = device

    def select(self, logits: torch.Tensor, rows: Sequence[RowRequest]) -> List[int]:
        """logits fp32 [R, V] on the device (left unchanged); one token per row."""
        R, V = logits.shape
        if R != len(rows):
            raise ValueError(f"{R} rows of logits for {len(rows)} requests")
        if R == 0:
            return []
        sampled = [i for i, r in enumerate(rows) if r.sampling is not None]
        out = torch.empty(R, dtype=torch.int32, device=logits.device)
        if len(sampled) < R:
            K.argmax(logits, out)
        if not sampled:
            return out.tolist()
        # sampled rows are worked on in a copy: the penalty changes logits in place
        idx = torch.tensor(sampled, dtype=torch.long, device=logits.device)
        work_logits = logits.index_select(0, idx).contiguous()
        S = len(sampled)
        params = [rows[i].sampling for i in sampled]
        if any(abs(p.repetition_penalty - 1.0) > 1.1920929e-07 for p in params):
            W = max(1, max(min(p.repetition_penalty_window, len(rows[i].history)) for p, i in zip(params, sampled)))
            recent = torch.zeros((S, W), dtype=torch.int32)
            counts = torch.zeros(S, dtype=torch.int32)
            for s, (p, i) in enumerate(zip(params, sampled)):
                n = min(p.repetition_penalty_window, len(rows[i].history))
                if n:
                    recent[s, :n] = torch.tensor(list(rows[i].history[-n:]), dtype=torch.int32)
                counts[s] = n
            pen = torch.tensor([p.repetition_penalty for p in params], dtype=torch.float32)
            K.repetition_penalty(work_logits, recent.to(logits.device), counts.to(logits.device),
                                 pen.to(logits.device))
        host = torch.tensor([[p.temperature for p in params], [p.top_p for p in params],
                             [token_uniform(p.seed, rows[i].generated_before) for p, i in zip(params, sampled)]],
                            dtype=torch.float32).to(logits.device)
        picked = torch.empty(S, dtype=torch.int32, device=logits.device)
        K.sample(work_logits, torch.empty_like(work_logits), host[0], host[1], host[2], picked)
        out.index_copy_(0, idx, picked)
        return out.tolist()
