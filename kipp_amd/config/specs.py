"""Architecture-neutral description of a decoder as data.

A model is a `ModelSpec`: sizes, a tuple of `LayerSpec`s and the order in
which they run.  Every layer names its block arrangement and gives one spec
for each part of it (mixer, feed-forward, norms); a mixer spec carries its
position-encoding spec.  A spec is a frozen dataclass whose `kind` names the
part class registered for it in `kipp_amd.parts`; all sizes and constants of
a part are fields of its spec, so no part needs to know the model it sits in.

Tensor names: a spec has a `prefix`; the part declares local parameter names
and the file name of a tensor is `prefix + local_name`.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional, Tuple


class ConfigError(ValueError):
    """A configuration that cannot be built: says which key and why."""


@dataclass(frozen=True)
class RMSNormSpec:
    """y = x * rsqrt(mean(x^2) + eps) * w over the last axis of `width`."""
    width: int
    eps: float
    prefix: str = ""
    kind: str = "rms_norm"


@dataclass(frozen=True)
class RopeSpec:
    """Rotary position encoding over the first `rotary_dim` dims of a head.

    pairing "half": dim i rotates with dim i + rotary_dim/2 (the reference's
    pairing, /root/reference/src/kipp.c:2368-2382); "interleaved": dim 2i with dim 2i + 1.
    """
    head_dim: int
    theta: float
    rotary_dim: Optional[int] = None
    pairing: str = "half"
    kind: str = "rope"

    def __post_init__(self):
        rd = self.head_dim if self.rotary_dim is None else self.rotary_dim
        if rd <= 0 or rd % 2 or rd > self.head_dim:
            raise ConfigError(f"rotary_dim {rd} must be even and in (0, head_dim={self.head_dim}]")
        if not self.theta > 0:
            raise ConfigError(f"rope theta must be positive, got {self.theta}")
        if self.pairing not in ("half", "interleaved"):
            raise ConfigError(f"rope pairing {self.pairing!r} is not one of half, interleaved")


@dataclass(frozen=True)
class NoPositionSpec:
    """No position encoding inside the mixer."""
    kind: str = "none"


@dataclass(frozen=True)
class AttentionSpec:
    """Causal grouped-query attention over a paged key/value cache.

    `window` None keeps every key; W keeps the last W keys (the query's own
    position included).  `qk_norm_eps` None means no per-head norm of q and k.
    `scale` None means 1/sqrt(head_dim).  `page_size` None keeps its keys in pages
    of the engine's size; P asks for pages of P tokens (a short window is served
    better by small pages), in a pool of their own.
    """
    hidden_size: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    position: object = NoPositionSpec()
    qk_norm_eps: Optional[float] = None
    window: Optional[int] = None
    scale: Optional[float] = None
    prefix: str = ""
    kind: str = "attention"
    page_size: Optional[int] = None

    def __post_init__(self):
        if self.num_heads <= 0 or self.num_kv_heads <= 0:
            raise ConfigError("attention needs at least one query head and one key/value head")
        if self.num_heads % self.num_kv_heads:
            raise ConfigError(
                f"num_attention_heads {self.num_heads} is not a multiple of "
                f"num_key_value_heads {self.num_kv_heads}")
        # any head size up to 256 runs (the float32 path and the generic kernel take it); the matrix-core attention
        # kernels of the bfloat16 path take multiples of 16 and the mixer falls back to the generic one otherwise
        if self.head_dim <= 0 or self.head_dim > 256:
            raise ConfigError(
                f"head_dim {self.head_dim} unsupported: the attention kernels take head sizes from 1 to 256")
        if self.window is not None and self.window <= 0:
            raise ConfigError(f"attention window must be positive, got {self.window}")
        if self.page_size is not None and self.page_size <= 0:
            raise ConfigError(f"attention page_size must be positive, got {self.page_size}")

    @property
    def q_dim(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.num_kv_heads * self.head_dim


@dataclass(frozen=True)
class GatedMLPSpec:
    """down(act(gate(x)) * up(x)); `activation` is "silu"."""
    hidden_size: int
    intermediate_size: int
    activation: str = "silu"
    prefix: str = ""
    kind: str = "gated_mlp"

    def __post_init__(self):
        if self.intermediate_size <= 0:
            raise ConfigError("intermediate_size must be positive")
        if self.activation != "silu":
            raise ConfigError(f"activation {self.activation!r} unsupported (silu only)")


@dataclass(frozen=True)
class LayerSpec:
    """One block: `block` names the arrangement, `parts` its parts by role.

    The "pre_norm" arrangement has the roles mixer_norm, mixer, ffn_norm, ffn
    and computes x += mixer(mixer_norm(x)); x += ffn(ffn_norm(x)).
    """
    parts: Tuple[Tuple[str, object], ...]
    block: str = "pre_norm"

    @property
    def kind(self) -> str:
        return self.block

    def part(self, role: str):
        for name, spec in self.parts:
            if name == role:
                return spec
        raise KeyError(role)


@dataclass(frozen=True)
class LayerRun:
    """One entry of the run order: run `layer`; `cache_of` names an earlier
    entry of the order (by index) whose cache this run reads instead of
    writing its own."""
    layer: int
    cache_of: Optional[int] = None


@dataclass(frozen=True)
class EmbeddingSpec:
    vocab_size: int
    hidden_size: int
    prefix: str = "model.embed_tokens."
    kind: str = "embedding"


@dataclass(frozen=True)
class HeadSpec:
    """Output head: logits = W x.  `tied` aliases the embedding table."""
    vocab_size: int
    hidden_size: int
    tied: bool
    prefix: str = "lm_head."
    kind: str = "lm_head"


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    hidden_size: int
    vocab_size: int
    max_position: int
    embedding: EmbeddingSpec
    layers: Tuple[LayerSpec, ...]
    order: Tuple[LayerRun, ...]
    final_norm: object
    head: HeadSpec
    stop_tokens: Tuple[int, ...] = field(default_factory=tuple)
    input_position: Optional[object] = None   # a position part applied to the residual stream after the embedding (None: none)

    def __post_init__(self):
        for index, run in enumerate(self.order):
            if not 0 <= run.layer < len(self.layers):
                raise ConfigError(f"order[{index}] names layer {run.layer} of {len(self.layers)}")
            if run.cache_of is not None:
                if not 0 <= run.cache_of < index:
                    raise ConfigError(f"order[{index}] reads the cache of entry {run.cache_of}, which is not earlier")
                if self.order[run.cache_of].cache_of is not None:
                    raise ConfigError(f"order[{index}] reads the cache of an entry that has none of its own")
