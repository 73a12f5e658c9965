"""Typed configuration of the Qwen3 dense decoder, read from config.json keys.

The reference takes these numbers from GGUF metadata that its converter wrote
from the same config.json keys (/root/reference/tools/convert_to_gguf.py:471-488)
and checks them against a compiled-in registry
(/root/reference/src/kipp.c:756-809).  Here every size is a field; nothing is
fixed in code.  Keys whose non-default value would change the computation and
that this engine does not implement are refused, never ignored.
"""
from __future__ import annotations

from dataclasses import dataclass, asdict
from typing import Tuple

from .specs import (AttentionSpec, ConfigError, EmbeddingSpec, GatedMLPSpec,
                    HeadSpec, LayerRun, LayerSpec, ModelSpec, RMSNormSpec,
                    RopeSpec)

ARCHITECTURE = "Qwen3ForCausalLM"

_REQUIRED = ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
             "num_attention_heads", "num_key_value_heads", "rms_norm_eps",
             "rope_theta", "max_position_embeddings")


def _as_int(d, key, minimum=1):
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, int):
        raise ConfigError(f"config.json {key}: expected an integer, got {v!r}")
    if v < minimum:
        raise ConfigError(f"config.json {key}: must be >= {minimum}, got {v}")
    return v


def _as_float(d, key):
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"config.json {key}: expected a number, got {v!r}")
    return float(v)


@dataclass(frozen=True)
class Qwen3Config:
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rms_norm_eps: float
    rope_theta: float
    max_position_embeddings: int
    tie_word_embeddings: bool
    stop_tokens: Tuple[int, ...] = ()

    @classmethod
    def from_dict(cls, d: dict) -> "Qwen3Config":
        missing = [k for k in _REQUIRED if k not in d]
        if missing:
            raise ConfigError("config.json lacks required keys: " + ", ".join(missing))
        if d.get("model_type", "qwen3") != "qwen3":
            raise ConfigError(f"config.json model_type: expected 'qwen3', got {d['model_type']!r}")
        if d.get("hidden_act", "silu") != "silu":
            raise ConfigError(f"config.json hidden_act: only 'silu' is implemented, got {d['hidden_act']!r}")
        if d.get("attention_bias", False):
            raise ConfigError("config.json attention_bias: projections with bias are not implemented")
        if d.get("rope_scaling") is not None:
            raise ConfigError("config.json rope_scaling: scaled rotary frequencies are not implemented")
        if d.get("use_sliding_window", False):
            raise ConfigError("config.json use_sliding_window: this architecture is run with full attention only")
        hidden = _as_int(d, "hidden_size")
        heads = _as_int(d, "num_attention_heads")
        if "head_dim" in d and d["head_dim"] is not None:
            head_dim = _as_int(d, "head_dim")
        else:
            if hidden % heads:
                raise ConfigError("config.json head_dim absent and hidden_size is not a multiple of num_attention_heads")
            head_dim = hidden // heads
        eps = _as_float(d, "rms_norm_eps")
        if not eps >= 0:
            raise ConfigError(f"config.json rms_norm_eps: must be >= 0, got {eps}")
        tied = d.get("tie_word_embeddings", False)
        if not isinstance(tied, bool):
            raise ConfigError(f"config.json tie_word_embeddings: expected true or false, got {tied!r}")
        stops = d.get("eos_token_id", ())
        if stops is None:
            stops = ()
        if isinstance(stops, int):
            stops = (stops,)
        vocab = _as_int(d, "vocab_size")
        for tok in stops:
            if isinstance(tok, bool) or not isinstance(tok, int) or not 0 <= tok < vocab:
                raise ConfigError(f"config.json eos_token_id: {tok!r} is not a token of the vocabulary")
        cfg = cls(
            vocab_size=vocab,
            hidden_size=hidden,
            intermediate_size=_as_int(d, "intermediate_size"),
            num_hidden_layers=_as_int(d, "num_hidden_layers"),
            num_attention_heads=heads,
            num_key_value_heads=_as_int(d, "num_key_value_heads"),
            head_dim=head_dim,
            rms_norm_eps=eps,
            rope_theta=_as_float(d, "rope_theta"),
            max_position_embeddings=_as_int(d, "max_position_embeddings"),
            tie_word_embeddings=tied,
            stop_tokens=tuple(stops),
        )
        cfg.model_spec()  # validates the part sizes (head_dim, groups, ...)
        return cfg

    def to_dict(self) -> dict:
        d = asdict(self)
        stops = d.pop("stop_tokens")
        d["architectures"] = [ARCHITECTURE]
        d["model_type"] = "qwen3"
        d["hidden_act"] = "silu"
        d["attention_bias"] = False
        d["rope_scaling"] = None
        d["use_sliding_window"] = False
        if stops:
            d["eos_token_id"] = list(stops) if len(stops) > 1 else stops[0]
        return d

    @property
    def q_dim(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.num_key_value_heads * self.head_dim

    def model_spec(self) -> ModelSpec:
        """The decoder as data: per layer input RMSNorm, attention with
        per-head q/k RMSNorm and rotary encoding, post-attention RMSNorm and a
        SwiGLU feed-forward (layer order of /root/reference/src/kipp.c:2588-2655)."""
        layers = []
        for i in range(self.num_hidden_layers):
            p = f"model.layers.{i}."
            mixer = AttentionSpec(
                hidden_size=self.hidden_size,
                num_heads=self.num_attention_heads,
                num_kv_heads=self.num_key_value_heads,
                head_dim=self.head_dim,
                position=RopeSpec(head_dim=self.head_dim, theta=self.rope_theta),
                qk_norm_eps=self.rms_norm_eps,
                window=None,
                prefix=p + "self_attn.",
            )
            layers.append(LayerSpec(block="pre_norm", parts=(
                ("mixer_norm", RMSNormSpec(self.hidden_size, self.rms_norm_eps, p + "input_layernorm.")),
                ("mixer", mixer),
                ("ffn_norm", RMSNormSpec(self.hidden_size, self.rms_norm_eps, p + "post_attention_layernorm.")),
                ("ffn", GatedMLPSpec(self.hidden_size, self.intermediate_size, "silu", p + "mlp.")),
            )))
        return ModelSpec(
            architecture=ARCHITECTURE,
            hidden_size=self.hidden_size,
            vocab_size=self.vocab_size,
            max_position=self.max_position_embeddings,
            embedding=EmbeddingSpec(self.vocab_size, self.hidden_size),
            layers=tuple(layers),
            order=tuple(LayerRun(i) for i in range(self.num_hidden_layers)),
            final_norm=RMSNormSpec(self.hidden_size, self.rms_norm_eps, "model.norm."),
            head=HeadSpec(self.vocab_size, self.hidden_size, self.tie_word_embeddings),
            stop_tokens=self.stop_tokens,
        )
