"""Reads a model directory's safetensors file onto a device through the library's reader ring (csrc/stloader.hip).

A safetensors file is an 8-byte little-endian header length, that many bytes of JSON (name -> dtype, shape, data_offsets), then the
data; only the header is parsed on the host, the tensor bytes go file -> pinned ring -> device without a host tensor in between."""
from __future__ import annotations

import json
import os
import struct

import torch

_DTYPES = {"BF16": torch.bfloat16, "F16": torch.float16, "F32": torch.float32, "I32": torch.int32, "I16": torch.int16,
           "I64": torch.int64, "U8": torch.uint8, "I8": torch.int8, "BOOL": torch.bool}


def read_header(path: str):
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        if n <= 0 or n > 1 << 30:
            raise RuntimeError(f"{path}: implausible safetensors header length {n}")
        header = json.loads(f.read(n))
    header.pop("__metadata__", None)
    return header, 8 + n


def load_tensors(path: str, device, ext, names=None) -> dict:
    """name -> tensor on `device` in the stored dtype"""
    header, base = read_header(path)
    size = os.path.getsize(path)
    out = {}
    for name, info in header.items():
        if names is not None and name not in names:
            continue
        if info["dtype"] not in _DTYPES:
            raise RuntimeError(f"{path}: tensor {name} has unsupported dtype {info['dtype']}")
        lo, hi = info["data_offsets"]
        t = torch.empty(tuple(info["shape"]), dtype=_DTYPES[info["dtype"]], device=device)
        if hi - lo != t.numel() * t.element_size() or base + hi > size:
            raise RuntimeError(f"{path}: tensor {name}: data range does not match its shape")
        ext.stloader_read(path, base + lo, hi - lo, t)
        out[name] = t
    return out
