"""Reading and writing safetensors files without any library.

Layout (as the reference's converter reads it,
/root/reference/tools/convert_to_gguf.py:282-291, 323-343): an 8-byte
little-endian header length, a JSON header {name: {dtype, shape,
data_offsets}}, then the payload; offsets are relative to the payload start.
Tensors are returned as torch views into a private copy-on-write mapping of
the file, so nothing is read until it is used.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Tuple

import torch

_DTYPES = {
    "F64": (torch.float64, 8), "F32": (torch.float32, 4), "F16": (torch.float16, 2),
    "BF16": (torch.bfloat16, 2), "I64": (torch.int64, 8), "I32": (torch.int32, 4),
    "I16": (torch.int16, 2), "I8": (torch.int8, 1), "U8": (torch.uint8, 1),
    "BOOL": (torch.bool, 1),
}
_NAMES = {v[0]: k for k, v in _DTYPES.items()}
_MAX_HEADER = 100 * 1024 * 1024


class SafetensorsError(ValueError):
    pass


def read_header(path: str) -> Tuple[dict, int, int]:
    """(header dict without __metadata__, payload offset, file size)."""
    size = os.path.getsize(path)
    with open(path, "rb") as f:
        head = f.read(8)
        if len(head) != 8:
            raise SafetensorsError(f"{path}: truncated before the header length")
        (n,) = struct.unpack("<Q", head)
        if n > _MAX_HEADER or 8 + n > size:
            raise SafetensorsError(f"{path}: header length {n} does not fit the file ({size} bytes)")
        raw = f.read(n)
    if len(raw) != n:
        raise SafetensorsError(f"{path}: truncated header")
    try:
        header = json.loads(raw.decode("utf-8"))
    except (UnicodeDecodeError, json.JSONDecodeError) as e:
        raise SafetensorsError(f"{path}: header is not valid JSON: {e}") from e
    if not isinstance(header, dict):
        raise SafetensorsError(f"{path}: header must be a JSON object")
    header.pop("__metadata__", None)
    return header, 8 + n, size


def read_file(path: str) -> Dict[str, torch.Tensor]:
    """All tensors of one file, by name, as views into a mapping of it."""
    header, base, size = read_header(path)
    payload = size - base
    with open(path, "rb") as f:
        mapping = mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_COPY) if size else None
    out: Dict[str, torch.Tensor] = {}
    spans = []
    for name, info in header.items():
        try:
            dtype_name, shape, (begin, end) = info["dtype"], info["shape"], info["data_offsets"]
        except (KeyError, TypeError, ValueError) as e:
            raise SafetensorsError(f"{path}: entry {name!r} is malformed") from e
        if dtype_name not in _DTYPES:
            raise SafetensorsError(f"{path}: tensor {name!r} has unsupported dtype {dtype_name!r}")
        dtype, width = _DTYPES[dtype_name]
        if not all(isinstance(s, int) and s >= 0 for s in shape):
            raise SafetensorsError(f"{path}: tensor {name!r} has a bad shape {shape!r}")
        count = 1
        for s in shape:
            count *= s
        if not (isinstance(begin, int) and isinstance(end, int) and 0 <= begin <= end <= payload):
            raise SafetensorsError(f"{path}: tensor {name!r} lies outside the file")
        if end - begin != count * width:
            raise SafetensorsError(
                f"{path}: tensor {name!r} spans {end - begin} bytes but shape {shape} of {dtype_name} needs {count * width}")
        spans.append((begin, end, name))
        if count == 0:
            out[name] = torch.empty(shape, dtype=dtype)
        else:
            out[name] = torch.frombuffer(mapping, dtype=dtype, count=count, offset=base + begin).reshape(shape)
    spans.sort()
    for (b0, e0, n0), (b1, e1, n1) in zip(spans, spans[1:]):
        if b1 < e0:
            raise SafetensorsError(f"{path}: tensors {n0!r} and {n1!r} overlap")
    return out


def write_file(path: str, tensors: Dict[str, torch.Tensor], metadata: Dict[str, str] | None = None) -> None:
    """Write tensors (CPU, any supported dtype) in name order."""
    header = {}
    if metadata:
        header["__metadata__"] = dict(metadata)
    offset = 0
    order = sorted(tensors)
    for name in order:
        t = tensors[name]
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"tensor {name!r}: dtype {t.dtype} cannot be stored")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    raw = json.dumps(header, separators=(",", ":")).encode("utf-8")
    raw += b" " * (-(8 + len(raw)) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(raw)))
        f.write(raw)
        for name in order:
            t = tensors[name].detach().contiguous().cpu()
            if t.numel():
                f.write(t.view(torch.uint8).numpy().tobytes() if t.dim() else t.reshape(1).view(torch.uint8).numpy().tobytes())
    os.replace(tmp, path)
