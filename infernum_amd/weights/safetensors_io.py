"""Reading and writing of safetensors files: an 8-byte little-endian length, a
JSON header {name: {dtype, shape, data_offsets}}, then the raw bytes.

All ``*.safetensors`` files of a folder are read, in sorted order, through a
memory map; an index file is not consulted (as the reference,
infernum-cuda/src/inner/weights/safetensors.rs:99-120).
"""
from __future__ import annotations

import glob
import json
import mmap
import os
import struct
from typing import Dict, Iterable, List, Tuple

import torch

_DTYPES = {
    "F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8,
    "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class TensorEntry:
    """Where one tensor lies in a file, and how to get it."""

    __slots__ = ("name", "dtype", "shape", "path", "begin", "end", "_owner")

    def __init__(self, name, dtype, shape, path, begin, end, owner):
        self.name, self.dtype, self.shape, self.path, self.begin, self.end, self._owner = \
            name, dtype, shape, path, begin, end, owner

    def read(self) -> torch.Tensor:
        """A CPU tensor that shares the file's memory map (read-only: copy before writing)."""
        n = 1
        for s in self.shape:
            n *= s
        if n == 0:
            return torch.empty(self.shape, dtype=self.dtype)
        buf = self._owner.buffer()
        t = torch.frombuffer(buf, dtype=self.dtype, count=n, offset=self._owner.data_start + self.begin)
        return t.reshape(self.shape)


class SafetensorsFile:
    def __init__(self, path: str):
        self.path = path
        self._mm = None
        try:
            with open(path, "rb") as f:
                head = f.read(8)
                if len(head) != 8:
                    raise SafetensorsError(f"{path}: shorter than a safetensors header")
                (n,) = struct.unpack("<Q", head)
                size = os.path.getsize(path)
                if n > size - 8 or n > (100 << 20):
                    raise SafetensorsError(f"{path}: header length {n} does not fit the file")
                try:
                    meta = json.loads(f.read(n).decode("utf-8"))
                except (UnicodeDecodeError, json.JSONDecodeError) as e:
                    raise SafetensorsError(f"{path}: header is not JSON: {e}") from e
        except OSError as e:
            raise SafetensorsError(f"cannot read {path}: {e}") from e
        self.data_start = 8 + n
        self.entries: Dict[str, TensorEntry] = {}
        data_len = size - self.data_start
        for name, info in meta.items():
            if name == "__metadata__":
                continue
            dt = _DTYPES.get(info.get("dtype"))
            if dt is None:
                raise SafetensorsError(f"{path}: tensor {name!r} has unsupported dtype {info.get('dtype')!r}")
            shape = tuple(int(s) for s in info["shape"])
            b, e = (int(x) for x in info["data_offsets"])
            count = 1
            for s in shape:
                count *= s
            if not (0 <= b <= e <= data_len) or (e - b) != count * torch.empty((), dtype=dt).element_size():
                raise SafetensorsError(f"{path}: tensor {name!r} has offsets that do not fit its shape or the file")
            self.entries[name] = TensorEntry(name, dt, shape, path, b, e, self)

    def buffer(self):
        if self._mm is None:
            with open(self.path, "rb") as f:
                self._mm = mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_COPY)   # private: torch wants a writable buffer
        return self._mm


def open_model_tensors(model_dir: str) -> Dict[str, TensorEntry]:
    """name -> entry over every ``*.safetensors`` of the folder."""
    paths = sorted(glob.glob(os.path.join(model_dir, "*.safetensors")))
    if not paths:
        raise SafetensorsError(f"No .safetensors files found in {model_dir}")
    out: Dict[str, TensorEntry] = {}
    for p in paths:
        for name, e in SafetensorsFile(p).entries.items():
            if name in out:
                raise SafetensorsError(f"tensor {name!r} is in both {out[name].path} and {p}")
            out[name] = e
    return out


def write_safetensors(path: str, tensors: Iterable[Tuple[str, torch.Tensor]]) -> None:
    """Write (name, tensor) pairs; tensors are taken one at a time, so a generator keeps memory low."""
    items: List[Tuple[str, torch.Tensor]] = []
    header: Dict[str, dict] = {}
    offset = 0
    # two passes would need the tensors twice; sizes are known from shapes, so collect metas first
    staged = []
    for name, t in tensors:
        t = t.detach().to("cpu").contiguous()
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"cannot store dtype {t.dtype}")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
        staged.append(t)
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for t in staged:
            if t.numel():
                f.write(t.view(torch.uint8).numpy().tobytes() if t.dtype != torch.bool else t.numpy().tobytes())
    os.replace(tmp, path)
