"""The uniform number behind a request's next sampled token.

It depends on the request's seed and on how many tokens the request has generated
so far, and on nothing else: not on the batch, not on the step, not on whether the
request was set back and recomputed.  The arithmetic is the reference's: the
per-token state is one xorshift64 round over ``seed ^ generated_before``
(infernum-runtime/src/engine.rs:283,406,491-494); the draw adds one, runs four
more rounds and divides by 2^64 - 1 in 32-bit floats
(infernum-cuda/src/inner/cuda/ops/sample.rs:141-147).
"""
from __future__ import annotations

import numpy as np

_MASK = (1 << 64) - 1


def _round(s: int) -> int:
    s ^= (s << 13) & _MASK
    s ^= s >> 7
    s ^= (s << 17) & _MASK
    return s


def token_uniform(seed: int, generated_before: int) -> float:
    """u in [0, 1] for the token that follows ``generated_before`` generated tokens."""
    state = _round((seed ^ generated_before) & _MASK)
    state = (state + 1) & _MASK
    for _ in range(4):
        state = _round(state)
    return float(np.float32(state) / np.float32(_MASK))
