"""Checkpoint reading: safetensors files, memory-mapped, no code executed.

A safetensors file is an 8-byte little-endian header length, that many bytes
of JSON ({name: {dtype, shape, data_offsets}}), then the raw tensor data.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterator, Tuple

import numpy as np
import torch

_DTYPES = {
    "BF16": torch.bfloat16, "F16": torch.float16, "F32": torch.float32,
    "F64": torch.float64, "I64": torch.int64, "I32": torch.int32,
    "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8,
    "BOOL": torch.bool,
}


def iter_safetensors(path: str) -> Iterator[Tuple[str, torch.Tensor]]:
    """Yield (name, tensor) pairs; tensors are copies (the map is closed
    when the iterator ends)."""
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(n))
        base = 8 + n
        mm = mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_READ)
        try:
            for name, info in header.items():
                if name == "__metadata__":
                    continue
                dt = _DTYPES[info["dtype"]]
                a, b = info["data_offsets"]
                shape = tuple(info["shape"])
                if b == a:
                    yield name, torch.empty(shape, dtype=dt)
                    continue
                raw = np.frombuffer(mm, dtype=np.uint8, count=b - a,
                                    offset=base + a)
                t = torch.from_numpy(raw.copy()).view(dt).reshape(shape)
                del raw                      # release the map's export
                yield name, t
        finally:
            mm.close()


def safetensors_shapes(path: str) -> Dict[str, Tuple[int, ...]]:
    """{name: shape} of every tensor in a model folder, from the file
    headers alone."""
    out: Dict[str, Tuple[int, ...]] = {}
    for fn in sorted(os.listdir(path)):
        if not fn.endswith(".safetensors"):
            continue
        with open(os.path.join(path, fn), "rb") as f:
            (n,) = struct.unpack("<Q", f.read(8))
            header = json.loads(f.read(n))
        for name, info in header.items():
            if name != "__metadata__":
                out[name] = tuple(info["shape"])
    return out


def load_model_dir_tensors(path: str) -> Dict[str, torch.Tensor]:
    """All tensors of every *.safetensors file in a model folder."""
    out: Dict[str, torch.Tensor] = {}
    files = sorted(f for f in os.listdir(path) if f.endswith(".safetensors"))
    if not files:
        raise FileNotFoundError(f"no .safetensors file in {path}")
    for fn in files:
        for name, t in iter_safetensors(os.path.join(path, fn)):
            out[name] = t
    return out
