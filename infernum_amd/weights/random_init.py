"""Random weights from a configuration and a seed.

Every tensor is a function of (seed, tensor name, element index) alone, so
values depend neither on the order in which tensors are made nor on the device
that makes them: a model filled on the GPU and a folder written on the host
from the same seed hold the same numbers.  Matrices and
the embedding are N(0, std), norm weights are what the spec says (ones, or a
uniform range).  ``write_random_model`` writes a model folder (config.json,
model.safetensors) that loads like any other; ``random_weights_on_device``
fills a model directly, for runs whose weights are too large to write first.
The reference has no such mode (its tests download checkpoints).
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Any, Dict, Iterator, Optional, Tuple

import torch

from ..parts.base import Runtime, WeightSpec


def _tensor_seed(seed: int, name: str) -> int:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(digest[:8], "little") & 0x7FFFFFFFFFFFFFFF


# ---- one generator for the CPU and the GPU -------------------------------------------------------------
# Element i of a tensor gets the 32-bit number hash(key of (seed, name), i): integer operations only, which
# give the same bits on every device.  A normal deviate is read from a table of 65,537 quantiles of the
# standard normal distribution (made once on the host, without a device's mathematical functions) with a
# linear step between two entries: a gather, a subtraction, a product by a multiple of 2^-16 and an addition
# in fp32, each rounded the same way everywhere.  The distribution is the normal one with a density that is
# constant within each 1/65,536 of probability, cut at 4.9 standard deviations.
_MASK32 = 0xFFFFFFFF
_CHUNK = 1 << 24                      # elements made at a time (bounds the temporaries)
_quantiles: Dict[torch.device, torch.Tensor] = {}


def _mix32(x: torch.Tensor) -> torch.Tensor:
    """A 32-bit integer hash on values kept in int64 (the low 32 bits of a product survive its wrap)."""
    x = x ^ (x >> 16)
    x = (x * 0x7FEB352D) & _MASK32
    x = x ^ (x >> 15)
    x = (x * 0x846CA68B) & _MASK32
    return x ^ (x >> 16)


def _uniform_bits(n: int, first: int, key: int, device: torch.device) -> torch.Tensor:
    """32 random bits (int64 in [0, 2^32)) for elements first .. first+n-1 of the tensor with this key."""
    k0, k1 = key & _MASK32, (key >> 32) & _MASK32
    i = torch.arange(first, first + n, dtype=torch.int64, device=device)
    x = _mix32((i & _MASK32) ^ k0)
    x = _mix32(((x + k1) & _MASK32) ^ (i >> 32))
    return x


def _normal_quantiles(device: torch.device) -> torch.Tensor:
    t = _quantiles.get(device)
    if t is None:
        from statistics import NormalDist
        inv = NormalDist().inv_cdf
        n = 65536
        q = [inv(1.0 / (16 * n))] + [inv(k / n) for k in range(1, n)] + [-inv(1.0 / (16 * n))]
        t = _quantiles[device] = torch.tensor(q, dtype=torch.float64).to(torch.float32).to(device)
    return t


def _standard_normal(n: int, first: int, key: int, device: torch.device) -> torch.Tensor:
    u = _uniform_bits(n, first, key, device)
    table = _normal_quantiles(device)
    idx = u >> 16
    frac = (u & 0xFFFF).to(torch.float32) * (1.0 / 65536.0)
    lo = table[idx]
    step = table[idx + 1] - lo
    step.mul_(frac)                     # a product, then a sum: two roundings, never a fused one
    return lo.add_(step)


def draw(spec: WeightSpec, seed: int, name: str, device: torch.device) -> torch.Tensor:
    """An fp32 tensor of the spec's shape on ``device``: the same bits on every device."""
    kind = spec.init[0]
    if kind == "ones":
        return torch.ones(spec.shape, dtype=torch.float32, device=device)
    if kind == "zeros":
        return torch.zeros(spec.shape, dtype=torch.float32, device=device)
    if kind not in ("normal", "uniform"):
        raise ValueError(f"unknown init {spec.init!r} for {name}")
    key = _tensor_seed(seed, name)
    out = torch.empty(spec.shape, dtype=torch.float32, device=device)
    flat = out.view(-1)
    for first in range(0, flat.numel(), _CHUNK):
        n = min(_CHUNK, flat.numel() - first)
        if kind == "normal":
            z = _standard_normal(n, first, key, device)
            flat[first:first + n] = z.mul_(float(spec.init[1]))
        else:
            lo, hi = float(spec.init[1]), float(spec.init[2])
            u = (_uniform_bits(n, first, key, device) >> 8).to(torch.float32) * (1.0 / (1 << 24))   # exact in fp32
            flat[first:first + n] = u.mul_(hi - lo).add_(lo)
    return out


def _cpu_model(config: Any, dtype: torch.dtype, **spec_kw: Any):
    from ..config.registry import model_spec_for
    from ..models.model import DecoderModel
    spec = model_spec_for(config, **spec_kw)
    return DecoderModel(spec, Runtime(torch.device("cpu"), dtype))


def random_tensors(config: Any, seed: int, dtype: torch.dtype = torch.bfloat16, made_on: Any = "cpu",
                   **spec_kw: Any) -> Iterator[Tuple[str, torch.Tensor]]:
    """(name, CPU tensor) for every tensor a file of this model holds; matrices in ``dtype``.
    ``made_on``: the device that works the numbers out (the same numbers on any; a GPU makes a large
    model's in seconds where the host takes minutes)."""
    model = _cpu_model(config, dtype, **spec_kw)
    for name, spec in sorted(model.expected_weights().items()):
        if not spec.write_when_random:
            continue
        t = draw(spec, seed, name, torch.device(made_on))
        yield name, t.to(dtype).cpu()


def write_random_model(config: Any, out_dir: str, seed: int, dtype: torch.dtype = torch.bfloat16,
                       made_on: Any = "cpu", **spec_kw: Any) -> str:
    """Write ``out_dir/config.json`` and ``out_dir/model.safetensors``; returns out_dir."""
    from .safetensors_io import write_safetensors
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, "config.json"), "w") as f:
        json.dump(config.to_dict(), f, indent=2)
    write_safetensors(os.path.join(out_dir, "model.safetensors"), random_tensors(config, seed, dtype, made_on, **spec_kw))
    return out_dir


def random_weights_on_device(model, seed: int, stored_as: Optional[torch.dtype] = None) -> None:
    """Fill a model with random weights made on its own device (nothing is written): the model that loading
    the folder of ``write_random_model(dtype=stored_as)`` would give; ``stored_as`` defaults to the model's
    compute type (a 32-bit model with ``stored_as=torch.bfloat16`` holds the numbers of the bfloat16 one)."""
    rt: Runtime = model.rt
    expected = model.expected_weights()
    from .loader import LazyTensors
    # a tied head shares its fallback's buffer: the fallback's name is the key of both
    keys = {name: spec.fallback if not spec.write_when_random and spec.fallback is not None else name
            for name, spec in expected.items()}

    def make(name: str, key: str) -> torch.Tensor:
        # what loading the folder that write_random_model(dtype=rt.dtype) writes would give: every tensor
        # rounded to that type once, also those that do not follow the compute type
        return draw(expected[key], seed, key, rt.device).to(stored_as or rt.dtype).to(rt.dtype)

    model.load_weights(LazyTensors(keys, make))


def main(argv: Optional[list] = None) -> int:
    """python -m infernum_amd.weights.random_init --config CONFIG.json --seed S --out DIR [--dtype bfloat16|float32]"""
    import argparse
    from ..config.registry import config_from_dict
    from ..config.base import read_config_json
    from .. import models  # noqa: F401  (registers the architectures)
    ap = argparse.ArgumentParser(prog="random_init", description="write a model folder (config.json, "
                                 "model.safetensors) with random weights from a configuration and a seed")
    ap.add_argument("--config", required=True, help="a config.json (or a folder that holds one)")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--out", required=True)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--norm-init", default="ones", choices=["ones", "uniform"],
                    help="norm weights: 1.0, or uniform in [0.5, 1.5]")
    a = ap.parse_args(argv)
    config = config_from_dict(read_config_json(a.config), where=a.config)
    kw = {"norm_init": ("uniform", 0.5, 1.5)} if a.norm_init == "uniform" else {}
    out = write_random_model(config, a.out, a.seed, {"bfloat16": torch.bfloat16, "float32": torch.float32}[a.dtype],
                             **kw)
    print(f"wrote {out}")
    return 0


if __name__ == "__main__":
    import sys
    sys.exit(main())
