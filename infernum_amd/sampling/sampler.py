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

import numpy as np
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
    pending_row: int = -1                       # >= 0: the request's newest token is this entry of ``previous``


class Sampler:
    # a request's newest token may still be on the device (``RowRequest.pending_row``, ``previous``): the penalty
    # finds it there, so a generation loop need not wait for a step's tokens before it launches the next
    history_on_device = True

    def __init__(self, device: torch.device):
        self.device = device
        self._staging = None

    def _to_device(self, host: np.ndarray) -> torch.Tensor:
        """A small host array to the device without waiting for what the GPU still has to do."""
        if torch.device(self.device).type != "cuda":
            return torch.from_numpy(host).to(self.device)
        if self._staging is None:
            from ..kernels.staging import PinnedUpload
            self._staging = PinnedUpload(torch.device(self.device), buffers=8)
        return self._staging.upload(host)

    @staticmethod
    def needs_history(sampling: Optional[SamplingParams]) -> bool:
        """Whether a request's choice looks at the tokens it has generated (the repetition penalty does)."""
        return sampling is not None and abs(sampling.repetition_penalty - 1.0) > 1.1920929e-07 \
            and sampling.repetition_penalty_window > 0

    def select(self, logits: torch.Tensor, rows: Sequence[RowRequest]) -> List[int]:
        """logits fp32 [R, V] on the device (left unchanged); one token per row."""
        return self.select_on_device(logits, rows).tolist()

    def select_on_device(self, logits: torch.Tensor, rows: Sequence[RowRequest],
                         previous: Optional[torch.Tensor] = None) -> torch.Tensor:
        """The same, with the tokens left on the device: int32 [R].  ``previous``: the tokens an earlier call left
        on the device, for rows whose ``pending_row`` names one of them as their newest token."""
        R, V = logits.shape
        if R != len(rows):
            raise ValueError(f"{R} rows of logits for {len(rows)} requests")
        out = torch.empty(R, dtype=torch.int32, device=logits.device)
        if R == 0:
            return out
        sampled = [i for i, r in enumerate(rows) if r.sampling is not None]
        if len(sampled) < R:
            K.argmax(logits, out)
        if not sampled:
            return out
        S = len(sampled)
        params = [rows[i].sampling for i in sampled]
        penalised = any(abs(p.repetition_penalty - 1.0) > 1.1920929e-07 for p in params)
        # one block of host numbers for all rows, one copy: temperature, top_p, draw, penalty
        nums = np.empty((4, S), dtype=np.float32)
        for s, (p, i) in enumerate(zip(params, sampled)):
            nums[0, s], nums[1, s] = p.temperature, p.top_p
            nums[2, s] = token_uniform(p.seed, rows[i].generated_before)
            nums[3, s] = p.repetition_penalty
        dev_nums = self._to_device(nums)
        if S == R and not penalised and logits.is_contiguous():
            work_logits = logits                     # nothing changes the logits: no copy
            idx = None
        else:
            # sampled rows are worked on in a copy: the penalty changes logits in place
            idx = self._to_device(np.asarray(sampled, dtype=np.int32)).long() if S < R else None
            work_logits = (logits.index_select(0, idx) if idx is not None else logits.clone()).contiguous()
        if penalised:
            tails = []
            for p, i in zip(params, sampled):
                h = rows[i].history
                n = min(p.repetition_penalty_window, len(h))
                tails.append(list(h[len(h) - n:]) if n else [])
            W = max(1, max(len(t) for t in tails))
            # the rows' tokens, how many of each row count, and which token on the device is a row's newest
            ints = np.zeros(S * W + 2 * S, dtype=np.int32)
            pending = False
            for s, (t, i) in enumerate(zip(tails, sampled)):
                ints[s * W:s * W + len(t)] = t
                ints[S * W + s] = len(t)
                ints[S * W + S + s] = rows[i].pending_row
                pending = pending or rows[i].pending_row >= 0
            if pending and previous is None:
                raise ValueError("a row's newest token is said to be on the device, but no tokens were given")
            dev_ints = self._to_device(ints)
            K.repetition_penalty(work_logits, dev_ints[:S * W].view(S, W), dev_ints[S * W:S * W + S], dev_nums[3],
                                 previous if pending else None, dev_ints[S * W + S:] if pending else None)
        picked = out if idx is None else torch.empty(S, dtype=torch.int32, device=logits.device)
        K.sample(work_logits, torch.empty_like(work_logits), dev_nums[0], dev_nums[1], dev_nums[2], picked)
        if idx is not None:
            out.index_copy_(0, idx, picked)
        return out
