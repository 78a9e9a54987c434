"""The single-file container (llmquant/packing/format.py), byte for byte:

    b"LLMQUANT" | uint64-LE header length | JSON header | tensor bytes

The JSON header is {"version": 1, "meta": {...}, "tensors": {name: {dtype, shape, offset,
nbytes}}} as json.dumps writes it by default; offsets are relative to the first byte after
the header and every tensor starts on a 64-byte boundary. bfloat16 travels as its raw 16
bits. dtypes: uint8, int8, float32, bfloat16.
"""

from __future__ import annotations

import json
import struct
from pathlib import Path

import numpy as np
import torch

MAGIC = b"LLMQUANT"
VERSION = 1
ALIGNMENT = 64
HEADER_LENGTH_BYTES = 8

_DTYPES = {"uint8": torch.uint8, "int8": torch.int8, "float32": torch.float32,
           "bfloat16": torch.bfloat16}


def _raw_bytes(tensor: torch.Tensor) -> bytes:
    host = tensor.detach().cpu().contiguous()
    if host.dtype == torch.bfloat16:
        host = host.view(torch.uint16)
    return host.numpy().tobytes()


def _tensor_at(data: np.ndarray, entry: dict) -> torch.Tensor:
    window = data[entry["offset"]: entry["offset"] + entry["nbytes"]]
    name = entry["dtype"]
    if name == "bfloat16":
        words = np.frombuffer(window, dtype=np.uint16).copy()
        return torch.from_numpy(words).view(torch.bfloat16).reshape(entry["shape"])
    values = np.frombuffer(window, dtype=np.dtype(name)).copy()
    return torch.from_numpy(values).reshape(entry["shape"])


def write_packed(path, tensors: dict, meta: dict) -> Path:
    """Write `tensors` (name -> tensor, in order) and a metadata dict. Returns the path."""
    path = Path(path)
    path.parent.mkdir(parents=True, exist_ok=True)
    table, chunks, cursor = {}, [], 0
    for name, tensor in tensors.items():
        gap = -cursor % ALIGNMENT
        if gap:
            chunks.append(bytes(gap))
            cursor += gap
        payload = _raw_bytes(tensor)
        table[name] = {
            "dtype": str(tensor.dtype).removeprefix("torch."),
            "shape": list(tensor.shape),
            "offset": cursor,
            "nbytes": len(payload),
        }
        chunks.append(payload)
        cursor += len(payload)
    header = json.dumps({"version": VERSION, "meta": meta, "tensors": table}).encode("utf-8")
    with open(path, "wb") as out:
        out.write(MAGIC + struct.pack("<Q", len(header)) + header)
        out.writelines(chunks)
    return path


def _read_header_and_start(path):
    with open(path, "rb") as src:
        if src.read(len(MAGIC)) != MAGIC:
            raise ValueError(f"{path} is not a llmquant weight file")
        (length,) = struct.unpack("<Q", src.read(HEADER_LENGTH_BYTES))
        header = json.loads(src.read(length).decode("utf-8"))
    if header["version"] != VERSION:
        raise ValueError(f"unsupported file version {header['version']}, expected {VERSION}")
    return header, len(MAGIC) + HEADER_LENGTH_BYTES + length


def read_header(path) -> dict:
    """The JSON header alone: enough to inspect a file without touching the weights."""
    return _read_header_and_start(path)[0]


def read_packed(path):
    """(tensors, meta). The data region is memory-mapped and each tensor copied out once."""
    header, start = _read_header_and_start(path)
    if not header["tensors"]:
        return {}, header["meta"]
    data = np.memmap(path, dtype=np.uint8, mode="r", offset=start)
    return {name: _tensor_at(data, entry) for name, entry in header["tensors"].items()}, header["meta"]
