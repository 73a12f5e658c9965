"""The pins of the plain implementation can fail: each plausible mistake below, made in a copy of
`tests/plain/qwen3_plain.py`, is caught by at least one test of `tests/test_plain.py` (after the
reference's seeded-fault runs, /root/reference/src/kipp.c:2814-2880: a gate that no fault can fail
proves nothing)."""
import os
import types

import pytest

import tests.test_plain as pins

SOURCE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "plain", "qwen3_plain.py")

MISTAKES = {
    "q_norm and k_norm weights exchanged": (
        'weights[p + "self_attn.q_norm.weight"], eps)\n        k = head_norm(k, n_kv, d, weights[p + "self_attn.k_norm.weight"]',
        'weights[p + "self_attn.k_norm.weight"], eps)\n        k = head_norm(k, n_kv, d, weights[p + "self_attn.q_norm.weight"]'),
    "the up side through SiLU instead of the gate": (
        "linear(silu(linear(x, w_gate)) * linear(x, w_up), w_down)",
        "linear(silu(linear(x, w_up)) * linear(x, w_gate), w_down)"),
    "the feed-forward normed with the attention's norm weight": (
        'n = rms_norm(x, weights[p + "post_attention_layernorm.weight"], eps)',
        'n = rms_norm(x, weights[p + "input_layernorm.weight"], eps)'),
    "the feed-forward reads the residual before the attention's delta": (
        '        x = x + linear(a, weights[p + "self_attn.o_proj.weight"])\n'
        '        n = rms_norm(x, weights[p + "post_attention_layernorm.weight"], eps)',
        '        n = rms_norm(x, weights[p + "post_attention_layernorm.weight"], eps)\n'
        '        x = x + linear(a, weights[p + "self_attn.o_proj.weight"])'),
    "rotation before the per-head norm": (
        '        q = head_norm(q, n_q, d, weights[p + "self_attn.q_norm.weight"], eps)\n'
        '        k = head_norm(k, n_kv, d, weights[p + "self_attn.k_norm.weight"], eps)\n'
        '        q = rope(q, n_q, d, positions, theta)\n        k = rope(k, n_kv, d, positions, theta)',
        '        q = rope(q, n_q, d, positions, theta)\n        k = rope(k, n_kv, d, positions, theta)\n'
        '        q = head_norm(q, n_q, d, weights[p + "self_attn.q_norm.weight"], eps)\n'
        '        k = head_norm(k, n_kv, d, weights[p + "self_attn.k_norm.weight"], eps)'),
    "interleaved rotary pairs": (
        "first, second = heads[..., :half], heads[..., half:]\n    out = np.concatenate([first * cos - second * sin, second * cos + first * sin], axis=-1)",
        "first, second = heads[..., 0::2], heads[..., 1::2]\n    out = np.stack([first * cos - second * sin, second * cos + first * sin], axis=-1).reshape(heads.shape)"),
    "the rotation's sign": ("first * cos - second * sin, second * cos + first * sin", "first * cos + second * sin, second * cos - first * sin"),
    "eps outside the root": ("1.0 / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)", "1.0 / (np.sqrt(np.mean(x * x, axis=-1, keepdims=True)) + eps)"),
    "norm weight as 1 + w": ("return x * scale * np.asarray(weight, dtype=DTYPE)", "return x * scale * (1.0 + np.asarray(weight, dtype=DTYPE))"),
    "query head h reads key/value head h % n_kv": ("kv = head // per_kv", "kv = head % n_kv"),
    "no 1/sqrt(d)": ("scale = 1.0 / np.sqrt(np.float64(head_dim))", "scale = 1.0"),
    "a token sees the next one": ("scores = (kh[first:token + 1, kv, :]", "scores = (kh[first:min(t, token + 2), kv, :]"),
    "the embedding scaled by sqrt(hidden)": (
        "return np.asarray(table, dtype=DTYPE)[np.asarray(tokens, dtype=np.int64)]",
        "return np.asarray(table, dtype=DTYPE)[np.asarray(tokens, dtype=np.int64)] * np.sqrt(np.asarray(table).shape[1])"),
    "no final norm": ('n = rms_norm(x, weights["model.norm.weight"], eps)\n    head', 'n = x\n    head'),
}


@pytest.mark.parametrize("mistake", sorted(MISTAKES))
def test_a_mistake_in_the_plain_implementation_is_caught(mistake, monkeypatch):
    old, new = MISTAKES[mistake]
    with open(SOURCE, "r", encoding="utf-8") as f:
        source = f.read()
    assert source.count(old) == 1, f"the text to change is not there once: {old!r}"
    mutant = types.ModuleType("qwen3_plain_mutant")
    exec(compile(source.replace(old, new), "qwen3_plain_mutant", "exec"), mutant.__dict__)
    monkeypatch.setattr(pins, "P", mutant)
    caught = []
    for name in sorted(dir(pins)):
        test = getattr(pins, name)
        if not name.startswith("test_") or getattr(test, "__code__", None) is None or test.__code__.co_argcount:
            continue          # tests that take fixtures compare two implementations with each other
        try:
            test()
        except AssertionError:
            caught.append(name)
        except Exception:     # a mistake may also break a shape
            caught.append(name)
    assert caught, f"no pin notices: {mistake}"
