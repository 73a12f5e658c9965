import json

import pytest

from kipp_amd.config import (ConfigError, Qwen3Config, get_architecture, load_config, parse_config,
                             register_architecture, shape_config, unregister_architecture)
from kipp_amd.config.specs import AttentionSpec, RopeSpec


def test_tiny_configurations_differ_in_every_size_and_option(tiny_configs):
    a, b = (parse_config(tiny_configs[k])[1] for k in "ab")
    for field in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers", "num_key_value_heads",
                  "head_dim", "rms_norm_eps", "rope_theta", "max_position_embeddings", "tie_word_embeddings"):
        assert getattr(a, field) != getattr(b, field), field
    assert a.num_attention_heads // a.num_key_value_heads != b.num_attention_heads // b.num_key_value_heads
    assert a.q_dim == a.hidden_size and b.q_dim != b.hidden_size
    for n in (b.hidden_size, b.intermediate_size, b.vocab_size):
        assert n & (n - 1)   # no power of two


def test_model_spec_is_data(tiny_configs):
    family, cfg = parse_config(tiny_configs["b"])
    assert family.name == "Qwen3ForCausalLM"
    spec = cfg.model_spec()
    assert len(spec.layers) == 3 and [r.layer for r in spec.order] == [0, 1, 2]
    mixer = spec.layers[1].part("mixer")
    assert (mixer.num_heads, mixer.num_kv_heads, mixer.head_dim, mixer.window) == (4, 1, 32, None)
    assert mixer.qk_norm_eps == 1e-5 and mixer.position.theta == 1e6 and mixer.prefix == "model.layers.1.self_attn."
    assert spec.layers[0].part("ffn").intermediate_size == 200
    assert not spec.head.tied and spec.final_norm.eps == 1e-5
    assert Qwen3Config.from_dict(cfg.to_dict()) == cfg


def test_head_dim_defaults_to_hidden_over_heads(tiny_configs):
    d = dict(tiny_configs["a"])
    del d["head_dim"]
    assert parse_config(d)[1].head_dim == 16
    d["hidden_size"] = 66
    with pytest.raises(ConfigError, match="head_dim"):
        parse_config(d)


@pytest.mark.parametrize("key,value,match", [
    ("rope_scaling", {"type": "yarn", "factor": 4}, "rope_scaling"),
    ("attention_bias", True, "attention_bias"),
    ("hidden_act", "gelu", "hidden_act"),
    ("use_sliding_window", True, "use_sliding_window"),
    ("model_type", "llama", "model_type"),
    ("num_key_value_heads", 3, "multiple"),
    ("head_dim", 260, "head_dim"),
    ("head_dim", 23, "rotary_dim"),
    ("vocab_size", "256", "vocab_size"),
    ("num_hidden_layers", 0, "num_hidden_layers"),
    ("rms_norm_eps", -1.0, "rms_norm_eps"),
    ("tie_word_embeddings", "yes", "tie_word_embeddings"),
    ("eos_token_id", 99999, "eos_token_id"),
])
def test_refused_values(tiny_configs, key, value, match):
    d = dict(tiny_configs["a"])
    d[key] = value
    with pytest.raises(ConfigError, match=match):
        parse_config(d)


def test_missing_keys_are_listed_together(tiny_configs):
    d = dict(tiny_configs["a"])
    del d["rope_theta"], d["rms_norm_eps"]
    with pytest.raises(ConfigError) as e:
        parse_config(d)
    assert "rope_theta" in str(e.value) and "rms_norm_eps" in str(e.value)


def test_registry(tiny_configs, tmp_path):
    d = dict(tiny_configs["a"], architectures=["NoSuchModel"])
    with pytest.raises(ConfigError, match="not in the registry"):
        parse_config(d)
    register_architecture("NoSuchModel", Qwen3Config.from_dict)
    try:
        assert parse_config(d)[0].name == "NoSuchModel"
    finally:
        unregister_architecture("NoSuchModel")
    with pytest.raises(ConfigError):
        get_architecture("NoSuchModel")
    with pytest.raises(ConfigError, match="architectures"):
        parse_config({k: v for k, v in d.items() if k != "architectures"})
    (tmp_path / "config.json").write_text(json.dumps(tiny_configs["b"]))
    assert load_config(str(tmp_path))[1].vocab_size == 509
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="JSON"):
        load_config(str(tmp_path))
    with pytest.raises(ConfigError, match="cannot read"):
        load_config(str(tmp_path / "absent"))


def test_eos_token_becomes_stop_tokens(tiny_configs):
    assert parse_config(dict(tiny_configs["a"], eos_token_id=[5, 9]))[1].model_spec().stop_tokens == (5, 9)
    assert parse_config(dict(tiny_configs["a"], eos_token_id=7))[1].stop_tokens == (7,)


def test_part_specs_check_their_sizes():
    with pytest.raises(ConfigError):
        AttentionSpec(64, 4, 2, 272)
    assert AttentionSpec(64, 4, 2, 20).q_dim == 80      # no multiple of 16: the generic attention kernel runs it
    with pytest.raises(ConfigError):
        AttentionSpec(64, 4, 2, 16, window=0)
    with pytest.raises(ConfigError):
        RopeSpec(16, 1e4, rotary_dim=7)
    assert shape_config("qwen3-4b")["num_hidden_layers"] == 36
    with pytest.raises(ConfigError):
        shape_config("nope")
