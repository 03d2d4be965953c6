"""Rotary position encoding: the table of inverse frequencies.

f_i = theta^(-2i/d) for i < d/2; the angle of position p is p * f_i and pairs are
half-split, (x[i], x[i + d/2]) (infernum/src/rope.rs:19-30,
infernum-cuda/kernels/rope.cu:25-41).  The rotation itself runs in the kernel
that also writes keys and values to their pages; this part owns the
frequencies only, which is all that differs between encodings of this family.

``llama3`` scaling is not in the reference's Llama path.  It has the form of
the reference's YaRN bands (infernum/src/rope.rs:91-120) with the band edges
taken from the configuration: with wavelength L = 2 pi / f and the original
context n, L < n/high keeps f, L > n/low gives f/factor, and between them
f' = (1-r) f/factor + r f with r = (n/L - low) / (high - low).  There is no
magnitude correction.

Frequencies are formed and kept in float64; the rotation kernel forms the angle
position * frequency in float64 too and brings it into [-pi, pi] before it takes
the fp32 sine and cosine, so that the angle is as good at position 100,000 as at
position 1 (a table of fp32 frequencies, which a position encoding may also give,
is multiplied in fp32: off by up to position * 2^-24 rad).
"""
from __future__ import annotations

import math
from typing import Any, Mapping, Optional

import torch

from .base import PositionEncoding, Runtime, register_part


def rope_inverse_frequencies(rotary_dim: int, theta: float, scaling: Optional[Mapping[str, Any]] = None) -> torch.Tensor:
    """float64 [rotary_dim / 2] on the CPU."""
    if rotary_dim <= 0 or rotary_dim % 2:
        raise ValueError(f"rotary size must be even and positive, got {rotary_dim}")
    half = rotary_dim // 2
    freqs = []
    for i in range(half):
        f = float(theta) ** (-2.0 * i / rotary_dim)
        if scaling is not None:
            kind = scaling.get("rope_type")
            if kind != "llama3":
                raise ValueError(f"rope scaling of type {kind!r} is not supported")
            factor = float(scaling["factor"])
            low = float(scaling["low_freq_factor"])
            high = float(scaling["high_freq_factor"])
            n = float(scaling["original_max_position_embeddings"])
            wavelen = 2.0 * math.pi / f
            if wavelen < n / high:
                pass
            elif wavelen > n / low:
                f = f / factor
            else:
                r = (n / wavelen - low) / (high - low)
                f = (1.0 - r) * f / factor + r * f
        freqs.append(f)
    return torch.tensor(freqs, dtype=torch.float64)


class RotaryEmbedding(PositionEncoding):
    """Half-split rotary encoding of the first ``rotary_dim`` values of a head."""
    graph_safe = True

    def __init__(self, rt: Runtime, head_dim: int, theta: float, scaling: Optional[Mapping[str, Any]] = None,
                 rotary_dim: Optional[int] = None):
        super().__init__(rt)
        self.head_dim = int(head_dim)
        self.rotary_dim = int(rotary_dim) if rotary_dim is not None else self.head_dim
        if self.rotary_dim > self.head_dim:
            raise ValueError("rotary_dim larger than the head size")
        self.inv_freq = rope_inverse_frequencies(self.rotary_dim, theta, scaling).to(rt.device)


class NoPositionEncoding(PositionEncoding):
    """Queries and keys are used as they are."""
    graph_safe = True

    def __init__(self, rt: Runtime, **_: Any):
        super().__init__(rt)
        self.inv_freq = None
        self.rotary_dim = 0


register_part("position", "rope", RotaryEmbedding)
register_part("position", "none", NoPositionEncoding)
