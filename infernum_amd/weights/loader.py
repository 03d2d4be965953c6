"""Weights by tensor name from a model folder onto the device.

The model says what it expects (full name, shape); the folder says what it has.
All differences are gathered into one :class:`WeightError`: missing tensors,
unexpected tensors and wrong shapes.  (The reference reports only the first
missing name, ``WeightNotFound``, infernum-cuda/src/inner/weights/safetensors.rs:
124-127, and does not check shapes.)

Matrices follow the compute dtype (bf16 when serving in bf16, fp32 in the 32-bit
path; file values are widened or rounded once).  A tensor that does not follow
it stays as stored: fp32 stays fp32, integer tables become int32.
"""
from __future__ import annotations

import fnmatch
from typing import Callable, Dict, Hashable, List

import torch

from ..parts.base import Runtime, WeightSpec
from .safetensors_io import TensorEntry, open_model_tensors

# Buffers that older checkpoints carry and no part reads.
IGNORED_TENSORS = ("*.rotary_emb.inv_freq",)


class WeightError(ValueError):
    def __init__(self, where: str, missing: List[str], unexpected: List[str], wrong_shape: List[str]):
        self.missing, self.unexpected, self.wrong_shape = missing, unexpected, wrong_shape
        lines = [f"weights in {where} do not fit the model:"]
        if missing:
            lines.append(f"  missing ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong_shape:
            lines.append(f"  wrong shape ({len(wrong_shape)}): " + "; ".join(wrong_shape))
        super().__init__("\n".join(lines))


def _convert(t: torch.Tensor, spec: WeightSpec, rt: Runtime) -> torch.Tensor:
    if not t.dtype.is_floating_point:
        return t.to(device=rt.device, dtype=torch.int32)
    if spec.follows_compute_dtype or rt.dtype == torch.float32:
        target = rt.dtype
    elif t.dtype in (torch.float32, torch.float64):
        target = torch.float32
    else:
        target = torch.bfloat16
    # on the device, so that a large matrix is converted there and the host copy stays mapped
    t = t.to(device=rt.device).contiguous()
    if t.dtype == target:
        return t
    if t.is_cuda and t.dtype in (torch.float32, torch.bfloat16):
        from ..kernels import api as K
        return K.cast(t, target)
    return t.to(target).contiguous()                # float16 and float64 files, and hosts without a GPU


def check_against(expected: Dict[str, WeightSpec], found: Dict[str, tuple], where: str) -> Dict[str, str]:
    """Compare names and shapes; returns expected name -> name to read it from."""
    missing, wrong = [], []
    source: Dict[str, str] = {}
    used = set()
    for name, spec in expected.items():
        src = name
        if src not in found and spec.fallback is not None and spec.fallback in found:
            src = spec.fallback
        if src not in found:
            missing.append(name)
            continue
        used.add(src)
        if tuple(found[src]) != tuple(spec.shape):
            wrong.append(f"{name}: expected {list(spec.shape)} got {list(found[src])}")
        source[name] = src
    unexpected = sorted(n for n in found if n not in used and n not in expected
                        and not any(fnmatch.fnmatch(n, pat) for pat in IGNORED_TENSORS))
    if missing or unexpected or wrong:
        raise WeightError(where, sorted(missing), unexpected, wrong)
    return source


class LazyTensors:
    """name -> tensor, made when a part asks for it: a model's parts are loaded one after the other, and what a part
    does not keep (the three projections it has put into one matrix) is gone before the next part's tensors come, so
    that loading needs the memory of the model and of one part's tensors, not twice the model's.  Names that share a
    key share one tensor (a tied head and its embedding): ``make(name, key)`` is called once, for the name that asks
    first, and the tensor is kept until the last of them has asked."""

    def __init__(self, keys: Dict[str, Hashable], make: Callable[[str, Hashable], torch.Tensor]):
        self._keys, self._make = dict(keys), make
        self._left: Dict[Hashable, int] = {}
        for key in self._keys.values():
            self._left[key] = self._left.get(key, 0) + 1
        self._kept: Dict[Hashable, torch.Tensor] = {}

    def __contains__(self, name: str) -> bool:
        return name in self._keys

    def __getitem__(self, name: str) -> torch.Tensor:
        key = self._keys[name]
        t = self._kept.get(key)
        if t is None:
            t = self._make(name, key)
        self._left[key] -= 1
        if self._left[key] > 0:
            self._kept[key] = t
        else:
            self._kept.pop(key, None)
        return t


def load_weights(model, model_dir: str) -> None:
    """Read every tensor the model expects from ``model_dir`` and hand them to its parts, part by part."""
    rt: Runtime = model.rt
    expected = model.expected_weights()
    entries: Dict[str, TensorEntry] = open_model_tensors(model_dir)
    source = check_against(expected, {n: e.shape for n, e in entries.items()}, model_dir)
    # a tied head shares the embedding's buffer: one key for both
    keys = {name: (source[name], spec.follows_compute_dtype) for name, spec in expected.items()}
    model.load_weights(LazyTensors(keys, lambda name, key: _convert(entries[key[0]].read(), expected[name], rt)))
