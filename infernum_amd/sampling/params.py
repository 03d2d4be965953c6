"""Options of a generation and of sampling, with the reference's names, meanings
and defaults (infernum/src/sampling.rs:5-60)."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional


@dataclass(frozen=True)
class SamplingParams:
    """Nucleus sampling.  ``temperature`` > 0 scales the logits; ``top_p`` in (0, 1]
    keeps the most probable tokens whose mass reaches it; the same ``seed`` and the
    same input give the same output; ``repetition_penalty`` > 1 weakens tokens that
    stand among the last ``repetition_penalty_window`` tokens (1.0: off)."""

    temperature: float = 0.7
    top_p: float = 0.9
    seed: int = 42
    repetition_penalty: float = 1.0
    repetition_penalty_window: int = 64

    def __post_init__(self) -> None:
        if not self.temperature > 0.0:
            raise ValueError(f"temperature must be > 0, got {self.temperature} (greedy decoding: sampling=None)")
        if not 0.0 < self.top_p <= 1.0:
            raise ValueError(f"top_p must be in (0, 1], got {self.top_p}")
        if not self.repetition_penalty > 0.0:
            raise ValueError(f"repetition_penalty must be > 0, got {self.repetition_penalty}")
        if self.repetition_penalty_window < 0:
            raise ValueError("repetition_penalty_window must be >= 0")
        if not 0 <= self.seed < (1 << 64):
            raise ValueError("seed must fit 64 unsigned bits")


@dataclass(frozen=True)
class GenerateOptions:
    """``sampling`` None means greedy decoding (argmax, the lowest index among equal
    maxima).  ``eos_token_id`` None never stops on a token.  ``use_kv_cache`` False
    recomputes the whole sequence for every new token (a slow check of the cache)."""

    max_new_tokens: int = 100
    eos_token_id: Optional[int] = None
    sampling: Optional[SamplingParams] = None
    use_kv_cache: bool = True

    def __post_init__(self) -> None:
        if self.max_new_tokens < 0:
            raise ValueError("max_new_tokens must be >= 0")
