"""What every part has in common: its parameters as data, and the registries.

A part class is registered under the `kind` of its spec in the registry of its
category (mixer, feed_forward, norm, position, block).  `params(spec)` lists
its tensors by local name without touching a device; the file name of a
tensor is `spec.prefix + local_name`.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict, Tuple


@dataclass(frozen=True)
class ParamSpec:
    """A tensor a part needs.  kind "float": a matrix or vector of reals;
    "int": an integer table (kept as int32).  `init` is how the random-weights
    mode fills it: ("normal", std) or ("one_plus_normal", std)."""
    shape: Tuple[int, ...]
    kind: str = "float"
    init: Tuple[str, float] = ("normal", 0.02)


CATEGORIES = ("mixer", "feed_forward", "norm", "position", "block", "embedding", "head")
_REGISTRY: Dict[str, Dict[str, type]] = {c: {} for c in CATEGORIES}


def register(category: str, kind: str) -> Callable[[type], type]:
    """Class decorator: `@register("mixer", "attention")`."""
    if category not in _REGISTRY:
        raise KeyError(f"unknown part category {category!r}; one of {CATEGORIES}")

    def deco(cls: type) -> type:
        _REGISTRY[category][kind] = cls
        return cls
    return deco


def unregister(category: str, kind: str) -> None:
    _REGISTRY[category].pop(kind, None)


def part_class(category: str, kind: str) -> type:
    try:
        return _REGISTRY[category][kind]
    except KeyError:
        known = ", ".join(sorted(_REGISTRY[category])) or "(none)"
        raise KeyError(f"no {category} part registered for kind {kind!r}; known: {known}") from None


def build_part(category: str, spec, runtime):
    return part_class(category, spec.kind)(spec, runtime)


def part_params(category: str, spec) -> Dict[str, ParamSpec]:
    """Full tensor names of one part."""
    cls = part_class(category, spec.kind)
    prefix = getattr(spec, "prefix", "")
    return {prefix + name: p for name, p in cls.params(spec).items()}
