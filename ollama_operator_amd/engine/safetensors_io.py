"""Minimal safetensors reader / writer (no third-party loader on the serving path).

File layout: 8-byte little-endian header length, that many bytes of JSON (name -> dtype, shape,
data_offsets relative to the end of the header), then the raw little-endian tensor data. The file is
memory-mapped; tensors are handed out as torch views of the map (bfloat16 through its uint16 bits), so a
tensor's pages are only read when it is copied to the device.
"""
from __future__ import annotations

import json
import struct

import numpy as np
import torch

_NP = {"F32": np.float32, "F16": np.float16, "BF16": np.uint16, "I32": np.int32, "I64": np.int64, "U8": np.uint8,
       "F64": np.float64, "I8": np.int8, "I16": np.int16}
_TORCH_NAME = {torch.float32: "F32", torch.float16: "F16", torch.bfloat16: "BF16", torch.int32: "I32",
               torch.int64: "I64", torch.uint8: "U8", torch.float64: "F64"}


class SafetensorsFile:
    def __init__(self, path: str):
        self.path = path
        with open(path, "rb") as f:
            (n,) = struct.unpack("<Q", f.read(8))
            if n <= 0 or n > (1 << 30):
                raise ValueError(f"{path}: implausible safetensors header length {n}")
            self.header = json.loads(f.read(n))
        self.header.pop("__metadata__", None)
        self._base = 8 + n
        self._map = np.memmap(path, dtype=np.uint8, mode="r")
        for name, t in self.header.items():
            if t["dtype"] not in _NP:
                raise ValueError(f"{path}: tensor {name} has unsupported dtype {t['dtype']}")
            a, b = t["data_offsets"]
            want = int(np.prod(t["shape"], dtype=np.int64)) * np.dtype(_NP[t["dtype"]]).itemsize
            if not (0 <= a <= b and self._base + b <= self._map.size and b - a == want):
                raise ValueError(f"{path}: tensor {name} has bad offsets")

    def names(self) -> list[str]:
        return list(self.header)

    def has(self, name: str) -> bool:
        return name in self.header

    def shape(self, name: str) -> tuple[int, ...]:
        return tuple(self.header[name]["shape"])

    def tensor(self, name: str) -> torch.Tensor:
        """A CPU tensor in the file's dtype (a copy, so the map can go away)."""
        t = self.header[name]
        a, b = t["data_offsets"]
        arr = np.frombuffer(self._map[self._base + a:self._base + b].tobytes(), dtype=_NP[t["dtype"]]).reshape(t["shape"])
        out = torch.from_numpy(arr.copy())
        return out.view(torch.bfloat16) if t["dtype"] == "BF16" else out


def write_safetensors(path: str, tensors: dict[str, torch.Tensor]) -> None:
    header, blobs, at = {}, [], 0
    for name, t in tensors.items():
        t = t.detach().cpu().contiguous()
        raw = (t.view(torch.uint16) if t.dtype == torch.bfloat16 else t).numpy().tobytes()
        header[name] = dict(dtype=_TORCH_NAME[t.dtype], shape=list(t.shape), data_offsets=[at, at + len(raw)])
        blobs.append(raw)
        at += len(raw)
    h = json.dumps(header, separators=(",", ":")).encode()
    h += b" " * (-len(h) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(h)))
        f.write(h)
        for b in blobs:
            f.write(b)
