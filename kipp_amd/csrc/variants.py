"""Which libraries a model needs, and the list that `build()` compiles ahead
of time.

A library is a `.hip` file, or a `.hip` file with constants (a kernel compiled
for one head size, say).  The files every model launches are listed here; a part
whose kernels are specialised says which builds it needs itself, through a
static method of its class

    variants(spec, dtype) -> [(file name without .hip, {constant: value} or None), ...]

so that a new part brings its own builds with it.
"""
from __future__ import annotations

from typing import List, Optional, Tuple

Spec = Tuple[str, Optional[dict]]

GENERIC: List[Spec] = [(name, None) for name in
                       ("elementwise", "rope_kv", "attention_generic", "gemm_f32", "gemm_skinny", "gemm_rows", "gemm_tiles", "sampling")]


def _add(out: List[Spec], more) -> None:
    for v in more:
        if v not in out:
            out.append(v)


def model_variants(spec, dtype: str) -> List[Spec]:
    """Everything the model `spec` launches under `dtype`: the common files and what its parts declare."""
    from ..parts import part_class
    out = list(GENERIC)
    owners = [("embedding", spec.embedding), ("norm", spec.final_norm), ("head", spec.head)]
    if getattr(spec, "input_position", None) is not None:
        owners.append(("position", spec.input_position))
    for layer in spec.layers:
        block = part_class("block", layer.block)
        _add(out, getattr(block, "variants", lambda s, d: [])(layer, dtype))
        owners.extend((category, layer.part(role)) for role, category in block.roles)
    for category, part_spec in owners:
        declare = getattr(part_class(category, part_spec.kind), "variants", None)
        if declare is not None:
            _add(out, declare(part_spec, dtype))
    return out


def prebuilt() -> List[Spec]:
    """What `build()` compiles ahead: everything the named shapes under `config/shapes` launch, in both
    precisions, and the read-bandwidth yardstick of `python -m kipp_amd.workloads hbm`."""
    from ..config import parse_config, shape_config, shape_names
    out = list(GENERIC)
    for name in shape_names():
        _, cfg = parse_config(shape_config(name))
        for dtype in ("bfloat16", "float32"):
            _add(out, model_variants(cfg.model_spec(), dtype))
    out.append(("probe", None))
    return out


# Kernel builds beyond what the named shapes launch: head sizes and head groupings at which the kernels are checked
# alone and in small models, and builds of the decode attention whose thresholds are lowered so that a check can
# reach the kernels for long contexts and many sequences with inputs it can verify.  `build()` compiles them ahead
# together with `prebuilt()`; whoever finds one missing compiles it then.
ATTENTION = [(128, 16), (128, 1), (16, 3), (48, 3), (64, 1), (32, 16), (256, 4), (80, 3), (256, 2), (16, 1), (32, 2), (16, 6)]   # (head size, group)
EARLY_STREAM = [(128, 4), (48, 3), (16, 2)]      # the kernel for long contexts takes over at 1,024 keys
WHOLE_CONTEXTS = [(128, 4), (128, 16)]           # the whole-context kernel at few sequences


def check_builds() -> List[Spec]:
    """Builds beyond the named shapes' own that the checks of the kernels and of small models launch."""
    out = []
    for head_dim, group in ATTENTION:
        out.append(("attention_prefill", {"HEAD_DIM": head_dim}))
        out.append(("attention_decode", {"HEAD_DIM": head_dim, "GROUP": group}))
    for head_dim, group in EARLY_STREAM:
        out.append(("attention_decode", {"HEAD_DIM": head_dim, "GROUP": group, "STREAM_FROM": 1024}))
    for head_dim, group in WHOLE_CONTEXTS:
        out.append(("attention_decode", {"HEAD_DIM": head_dim, "GROUP": group, "RING_FROM_PAIRS": 1}))
    seen, unique = set(), []
    for name, defines in out:
        key = (name, tuple(sorted(defines.items())))
        if key not in seen:
            seen.add(key)
            unique.append((name, defines))
    return unique

