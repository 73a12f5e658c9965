"""Which libraries a model needs, and the list that `build()` compiles ahead
of time (the sizes of the benchmark, of the tests and of the smoke run)."""
from __future__ import annotations

from typing import List, Optional, Tuple

Spec = Tuple[str, Optional[dict]]

GENERIC: List[Spec] = [(name, None) for name in
                       ("elementwise", "rope_kv", "attention_generic", "gemm_f32", "gemm_skinny", "gemm_rows", "sampling")]


def attention_variants(head_dim: int, group: int) -> List[Spec]:
    out: List[Spec] = [("attention_prefill", {"HEAD_DIM": head_dim})]
    if group <= 16:
        out.append(("attention_decode", {"HEAD_DIM": head_dim, "GROUP": group}))
    return out


def model_variants(spec, dtype: str) -> List[Spec]:
    """Everything the model `spec` launches under `dtype`."""
    out = list(GENERIC)
    if dtype == "bfloat16":
        for layer in spec.layers:
            for _, part in layer.parts:
                if getattr(part, "kind", None) == "attention":
                    for v in attention_variants(part.head_dim, part.num_heads // part.num_kv_heads):
                        if v not in out:
                            out.append(v)
    return out


# (head_dim, query heads per key/value head) of the shapes under config/shapes,
# the tiny configurations, the toy model of the tests and the kernel tests
PREBUILT_ATTENTION = [(128, 4), (128, 8), (128, 16), (128, 1), (16, 2), (32, 4), (16, 3), (48, 3), (64, 1), (32, 16), (256, 4), (80, 3), (256, 2), (16, 1)]


# builds of the decode attention in which the kernel for long contexts takes over at 1,024 keys
# already, so that a kernel test can reach it with contexts it can check
PREBUILT_WHOLE_CONTEXTS = [(128, 4), (128, 16)]    # tests: the whole-context decode kernel at few sequences
PREBUILT_EARLY_STREAM = [(128, 4), (48, 3), (16, 2)]


def prebuilt() -> List[Spec]:
    out = list(GENERIC)
    for head_dim, group in PREBUILT_ATTENTION:
        for v in attention_variants(head_dim, group):
            if v not in out:
                out.append(v)
    for head_dim, group in PREBUILT_EARLY_STREAM:
        out.append(("attention_decode", {"HEAD_DIM": head_dim, "GROUP": group, "STREAM_FROM": 1024}))
    for head_dim, group in PREBUILT_WHOLE_CONTEXTS:
        out.append(("attention_decode", {"HEAD_DIM": head_dim, "GROUP": group, "RING_FROM_PAIRS": 1}))
    out.append(("probe", None))       # the read-bandwidth yardstick of `python -m kipp_amd.workloads hbm`
    return out
