"""Typed configurations and the architecture registry.

`load_config(model_dir)` reads config.json, looks `architectures[0]` up in the
registry and returns (family, typed config).  A family is what an architecture
registers: how to read its config.json keys and how to turn the typed config
into a `ModelSpec` (the decoder as data).
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Callable, Dict

from .specs import (AttentionSpec, ConfigError, EmbeddingSpec, GatedMLPSpec,
                    HeadSpec, LayerRun, LayerSpec, ModelSpec, NoPositionSpec,
                    RMSNormSpec, RopeSpec)


@dataclass(frozen=True)
class Family:
    """One architecture: `parse(dict) -> config` and `config.model_spec()`."""
    name: str
    parse: Callable[[dict], object]


_ARCHITECTURES: Dict[str, Family] = {}


def register_architecture(name: str, parse: Callable[[dict], object]) -> Family:
    """Register `name` (the string in config.json `architectures[0]`).  `parse`
    takes the config.json dict and returns a typed config with `model_spec()`
    and `to_dict()`."""
    family = Family(name, parse)
    _ARCHITECTURES[name] = family
    return family


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def get_architecture(name: str) -> Family:
    if name not in _ARCHITECTURES:
        known = ", ".join(sorted(_ARCHITECTURES)) or "(none)"
        raise ConfigError(f"architecture {name!r} is not in the registry; known: {known}")
    return _ARCHITECTURES[name]


def parse_config(d: dict):
    """(family, typed config) of a config.json dict."""
    if not isinstance(d, dict):
        raise ConfigError("config.json must hold a JSON object")
    archs = d.get("architectures")
    if not isinstance(archs, list) or len(archs) != 1 or not isinstance(archs[0], str):
        raise ConfigError("config.json architectures: expected a list with one name")
    family = get_architecture(archs[0])
    return family, family.parse(d)


def load_config(model_dir: str):
    path = os.path.join(model_dir, "config.json")
    try:
        with open(path, "r", encoding="utf-8") as f:
            d = json.load(f)
    except OSError as e:
        raise ConfigError(f"cannot read {path}: {e}") from e
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path} is not valid JSON: {e}") from e
    return parse_config(d)


def shape_names():
    """Names of the shapes shipped under config/shapes/."""
    here = os.path.join(os.path.dirname(__file__), "shapes")
    return sorted(f[:-5] for f in os.listdir(here) if f.endswith(".json"))


def shape_config(name: str) -> dict:
    """config.json dict of a named shape shipped under config/shapes/."""
    here = os.path.join(os.path.dirname(__file__), "shapes")
    path = os.path.join(here, name + ".json")
    if not os.path.exists(path):
        known = sorted(f[:-5] for f in os.listdir(here) if f.endswith(".json"))
        raise ConfigError(f"unknown shape {name!r}; known: {', '.join(known)}")
    with open(path, "r", encoding="utf-8") as f:
        return json.load(f)


from . import qwen3 as _qwen3  # noqa: E402

register_architecture(_qwen3.ARCHITECTURE, _qwen3.Qwen3Config.from_dict)
Qwen3Config = _qwen3.Qwen3Config
