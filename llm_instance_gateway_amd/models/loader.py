"""Checkpoint reading: safetensors files, memory-mapped.

Layout of a safetensors file: an 8-byte little-endian header length, that
many bytes of JSON (tensor name -> dtype, shape, data_offsets relative to the
end of the header), then the raw little-endian tensor data.  Nothing in the
file is executed; tensors are views of one read-only mmap and are copied to
their device by whoever consumes them.
"""

from __future__ import annotations

import json
import mmap
import struct
from typing import Dict

import torch

_DTYPES = {
    "BF16": torch.bfloat16,
    "F16": torch.float16,
    "F32": torch.float32,
    "F64": torch.float64,
    "I64": torch.int64,
    "I32": torch.int32,
    "I16": torch.int16,
    "I8": torch.int8,
    "U8": torch.uint8,
    "BOOL": torch.bool,
}


def read_safetensors_shapes(path: str) -> Dict[str, list]:
    """Tensor name -> shape from the header alone (no tensor data is read)."""
    with open(path, "rb") as f:
        (hlen,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(hlen).decode("utf-8"))
    return {k: list(v["shape"]) for k, v in header.items() if k != "__metadata__"}


def read_safetensors(path: str) -> Dict[str, torch.Tensor]:
    with open(path, "rb") as f:
        mm = mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_COPY)
    (hlen,) = struct.unpack("<Q", mm[:8])
    if hlen > len(mm) - 8:
        raise ValueError(f"{path}: header length {hlen} exceeds the file")
    header = json.loads(bytes(mm[8 : 8 + hlen]).decode("utf-8"))
    base = 8 + hlen
    buf = memoryview(mm)
    out: Dict[str, torch.Tensor] = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        if info["dtype"] not in _DTYPES:
            raise ValueError(f"{path}: tensor {name} has unsupported dtype {info['dtype']}")
        dt = _DTYPES[info["dtype"]]
        lo, hi = info["data_offsets"]
        shape = list(info["shape"])
        n = 1
        for d in shape:
            n *= d
        if hi - lo != n * torch.empty((), dtype=dt).element_size() or base + hi > len(mm):
            raise ValueError(f"{path}: tensor {name} does not fit its offsets")
        if n == 0:
            out[name] = torch.empty(shape, dtype=dt)
        else:
            out[name] = torch.frombuffer(buf, dtype=dt, count=n, offset=base + lo).view(shape)
    return out
