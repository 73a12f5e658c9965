"""Random weights: a model folder (config.json, model.safetensors) from a
configuration and a seed.

Each tensor has its own stream, seeded by (seed, tensor name), so the values
do not depend on the order of creation.  Matrices and the embedding are
N(0, std), norm weights 1 + N(0, std), with the std that the part declares.
Values are drawn in float32 and stored as `dtype` (bfloat16: round to nearest
even).
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Dict

import torch

from ..config import parse_config
from ..parts.base import ParamSpec
from .safetensors_io import write_file


def tensor_seed(seed: int, name: str) -> int:
    digest = hashlib.sha256(f"{seed}:{name}".encode("utf-8")).digest()
    return int.from_bytes(digest[:8], "little") & ((1 << 63) - 1)


def random_tensor(seed: int, name: str, spec: ParamSpec, dtype: torch.dtype = torch.bfloat16,
                  device: str = "cpu") -> torch.Tensor:
    gen = torch.Generator(device=device)
    gen.manual_seed(tensor_seed(seed, name))
    if spec.kind == "int":
        return torch.zeros(spec.shape, dtype=torch.int32, device=device)
    how, std = spec.init
    t = torch.empty(spec.shape, dtype=torch.float32, device=device).normal_(0.0, std, generator=gen)
    if how == "one_plus_normal":
        t += 1.0
    elif how != "normal":
        raise ValueError(f"unknown init {how!r} for {name}")
    return t.to(dtype)


def random_tensors(expected: Dict[str, ParamSpec], seed: int, dtype: torch.dtype = torch.bfloat16,
                   device: str = "cpu") -> Dict[str, torch.Tensor]:
    return {name: random_tensor(seed, name, spec, dtype, device) for name, spec in expected.items()}


def write_random_model(model_dir: str, config: dict, seed: int, dtype: str = "bfloat16") -> str:
    """Write config.json and model.safetensors for `config` (a config.json dict)."""
    from ..engine.model import model_params
    _, cfg = parse_config(config)
    expected = model_params(cfg.model_spec())
    torch_dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype]
    os.makedirs(model_dir, exist_ok=True)
    out = dict(config)
    out["torch_dtype"] = dtype
    with open(os.path.join(model_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(out, f, indent=2, sort_keys=True)
        f.write("\n")
    write_file(os.path.join(model_dir, "model.safetensors"), random_tensors(expected, seed, torch_dtype),
               metadata={"format": "pt", "seed": str(seed)})
    return model_dir
