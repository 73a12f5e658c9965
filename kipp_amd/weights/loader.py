"""Weights by tensor name from a model folder.

`read_model_tensors(dir)` maps every tensor of `model.safetensors` (or of the
shards named by `model.safetensors.index.json`,
/root/reference/tools/convert_to_gguf.py:297-314) without reading it.
`check_tensors` compares what the file holds with what the model's parts
declare and raises ONE error that lists every missing tensor, every unexpected
tensor and every wrong shape or type (the reference stops at the first:
/root/reference/src/kipp.c:859-906, 997-1002).
"""
from __future__ import annotations

import json
import os
from typing import Dict

import torch

from ..parts.base import ParamSpec
from .safetensors_io import SafetensorsError, read_file

_FLOATS = (torch.float32, torch.bfloat16, torch.float16)
_INTS = (torch.int64, torch.int32, torch.int16, torch.int8, torch.uint8)


class WeightError(ValueError):
    """The model folder does not hold what the configuration needs."""

    def __init__(self, where, missing, unexpected, wrong):
        self.missing, self.unexpected, self.wrong = list(missing), list(unexpected), list(wrong)
        lines = [f"weights in {where} do not match the configuration:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong:
            lines.append(f"  wrong shape or type ({len(self.wrong)}): " + "; ".join(self.wrong))
        super().__init__("\n".join(lines))


def read_model_tensors(model_dir: str) -> Dict[str, torch.Tensor]:
    index = os.path.join(model_dir, "model.safetensors.index.json")
    single = os.path.join(model_dir, "model.safetensors")
    if os.path.exists(index):
        with open(index, "r", encoding="utf-8") as f:
            weight_map = json.load(f).get("weight_map")
        if not isinstance(weight_map, dict):
            raise SafetensorsError(f"{index}: no weight_map")
        out: Dict[str, torch.Tensor] = {}
        for shard in sorted(set(weight_map.values())):
            tensors = read_file(os.path.join(model_dir, shard))
            for name, t in tensors.items():
                if weight_map.get(name) == shard:
                    out[name] = t
        listed_but_absent = [n for n in weight_map if n not in out]
        if listed_but_absent:
            raise SafetensorsError(f"{index}: tensors listed but absent from their shard: {', '.join(listed_but_absent)}")
        return out
    if os.path.exists(single):
        return read_file(single)
    raise SafetensorsError(f"{model_dir}: neither model.safetensors nor model.safetensors.index.json")


def check_tensors(where: str, found: Dict[str, torch.Tensor], expected: Dict[str, ParamSpec]) -> None:
    missing = [n for n in expected if n not in found]
    unexpected = [n for n in found if n not in expected]
    wrong = []
    for name, spec in expected.items():
        t = found.get(name)
        if t is None:
            continue
        if tuple(t.shape) != tuple(spec.shape):
            wrong.append(f"{name}: shape {tuple(t.shape)}, expected {tuple(spec.shape)}")
        elif spec.kind == "float" and t.dtype not in _FLOATS:
            wrong.append(f"{name}: type {t.dtype}, expected bfloat16, float16 or float32")
        elif spec.kind == "int" and t.dtype not in _INTS:
            wrong.append(f"{name}: type {t.dtype}, expected an integer type")
    if missing or unexpected or wrong:
        raise WeightError(where, sorted(missing), sorted(unexpected), wrong)
