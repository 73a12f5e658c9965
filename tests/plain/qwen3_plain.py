"""The plain implementation: the Qwen3 dense decoder over whole sequences, no
cache, no pages, no batching, one function for each part, written from the
reference's formulas.  It shares no code with `kipp_amd`: it reads the model
folder with the `safetensors` package and computes with NumPy.

All functions compute in `DTYPE` (float64 by default, so that the float32
engine is compared against something more exact than itself).  The rotation
angle alone is formed in float32, as the reference does (`(float)position *
frequency`), because at large positions the rounding of that product is part
of the formula's result.
"""
from __future__ import annotations

import json
import os

import numpy as np

DTYPE = np.float64


# ----------------------------------------------------------------------------- parts

def bf16_round(x):
    """Round float32 values to bfloat16 (nearest even) and widen back.
    /root/reference/src/kipp.c:2181-2186 (float_to_bf16), :2174-2179 (bf16_to_float)."""
    bits = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    rounding = 0x7FFF + ((bits >> 16) & 1)
    out = (((bits + rounding) >> 16) << 16).astype(np.uint32)
    return out.view(np.float32)


def bf16_bits(x):
    """The 16 stored bits.  /root/reference/src/kipp.c:2181-2186."""
    bits = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    rounding = 0x7FFF + ((bits >> 16) & 1)
    return ((bits + rounding) >> 16).astype(np.uint16)


def embed(table, tokens):
    """x[t] = E[token_t], a plain row gather without scaling.
    /root/reference/src/kipp.c:2579-2585."""
    return np.asarray(table, dtype=DTYPE)[np.asarray(tokens, dtype=np.int64)]


def rms_norm(x, weight, eps):
    """y = x * (1 / sqrt(mean(x^2) + eps)) * w over the last axis; eps inside the
    root, the weight a plain multiplier.  /root/reference/src/kipp.c:2221-2231."""
    x = np.asarray(x, dtype=DTYPE)
    scale = 1.0 / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)
    return x * scale * np.asarray(weight, dtype=DTYPE)


def linear(x, weight):
    """y[o] = sum_i W[o, i] x[i]; W is [out][in], no bias.
    /root/reference/src/kipp.c:2233-2244."""
    return np.asarray(x, dtype=DTYPE) @ np.asarray(weight, dtype=DTYPE).T


def head_norm(states, n_heads, head_dim, weight, eps):
    """RMSNorm of every head vector of [tokens, n_heads * head_dim] with one
    weight [head_dim] shared by all heads.  /root/reference/src/kipp.c:2480-2500."""
    t = states.shape[0]
    heads = np.asarray(states, dtype=DTYPE).reshape(t, n_heads, head_dim)
    return rms_norm(heads, weight, eps).reshape(t, n_heads * head_dim)


def rope(states, n_heads, head_dim, positions, theta):
    """Rotate dim i with dim i + head_dim/2 by angle pos * theta^(-2i/head_dim):
    (a, b) -> (a cos - b sin, b cos + a sin).  /root/reference/src/kipp.c:2368-2382
    (rope_head), :2502-2512 (apply_rope)."""
    t = states.shape[0]
    half = head_dim // 2
    heads = np.asarray(states, dtype=DTYPE).reshape(t, n_heads, head_dim)
    freq = np.power(np.float64(theta), -(2.0 * np.arange(half, dtype=np.float64)) / head_dim).astype(np.float32)
    angle = (np.asarray(positions, dtype=np.float32)[:, None] * freq[None, :]).astype(np.float32).astype(np.float64)
    cos, sin = np.cos(angle)[:, None, :], np.sin(angle)[:, None, :]
    first, second = heads[..., :half], heads[..., half:]
    out = np.concatenate([first * cos - second * sin, second * cos + first * sin], axis=-1)
    return out.reshape(t, n_heads * head_dim)


def softmax(scores):
    """exp(x - max) / sum over the last axis.  /root/reference/src/kipp.c:2384-2400."""
    e = np.exp(scores - np.max(scores, axis=-1, keepdims=True))
    return e * (1.0 / np.sum(e, axis=-1, keepdims=True))


def causal_gqa(q, k, v, n_q, n_kv, head_dim, window=None):
    """Token t of query head h attends to sources s <= t of key/value head
    h // (n_q / n_kv); score = (q . k) * (1 / sqrt(head_dim)); softmax; weighted
    values.  /root/reference/src/kipp.c:2520-2562.  `window` W (not in the reference)
    keeps only sources s > t - W."""
    t = q.shape[0]
    scale = 1.0 / np.sqrt(np.float64(head_dim))
    per_kv = n_q // n_kv
    qh = np.asarray(q, dtype=DTYPE).reshape(t, n_q, head_dim)
    kh = np.asarray(k, dtype=DTYPE).reshape(t, n_kv, head_dim)
    vh = np.asarray(v, dtype=DTYPE).reshape(t, n_kv, head_dim)
    out = np.zeros((t, n_q, head_dim), dtype=DTYPE)
    for token in range(t):
        first = 0 if window is None else max(0, token - window + 1)
        for head in range(n_q):
            kv = head // per_kv
            scores = (kh[first:token + 1, kv, :] @ qh[token, head, :]) * scale
            out[token, head, :] = softmax(scores) @ vh[first:token + 1, kv, :]
    return out.reshape(t, n_q * head_dim)


def silu(x):
    """x / (1 + exp(-x)).  /root/reference/src/kipp.c:2402-2404."""
    return x / (1.0 + np.exp(-x))


def swiglu_mlp(x, w_gate, w_up, w_down):
    """down(silu(gate(x)) * up(x)).  /root/reference/src/kipp.c:2633-2653."""
    return linear(silu(linear(x, w_gate)) * linear(x, w_up), w_down)


# ----------------------------------------------------------------------------- the model

def load_folder(model_dir):
    """(config dict, {name: float64 array}) of a model folder."""
    from safetensors.torch import load_file
    with open(os.path.join(model_dir, "config.json"), "r", encoding="utf-8") as f:
        config = json.load(f)
    tensors = load_file(os.path.join(model_dir, "model.safetensors"))
    return config, {name: t.float().numpy().astype(DTYPE) for name, t in tensors.items()}


def forward_whole(config, weights, tokens, kv_round=None, return_hidden=False, position_offset=0):
    """Logits [len(tokens), vocab] of one whole sequence.
    Layer order of /root/reference/src/kipp.c:2588-2655 (cpu_forward): input norm, q/k/v,
    per-head q and k norm, rotation, attention, output projection and residual,
    post-attention norm, SwiGLU and residual; then the final norm and the head
    (:2657-2661), here for every position, not only the last.
    `kv_round`: a function applied to keys and values before attention (the
    reference rounds them to bfloat16 there, :2614-2615; the float32 engine keeps
    them in float32, so its reference passes None).  `position_offset` shifts every
    position (the result must not change: only distances count)."""
    n_q = config["num_attention_heads"]
    n_kv = config["num_key_value_heads"]
    d = config.get("head_dim") or config["hidden_size"] // n_q
    eps = config["rms_norm_eps"]
    theta = config["rope_theta"]
    positions = np.arange(len(tokens)) + position_offset
    x = embed(weights["model.embed_tokens.weight"], tokens)
    for layer in range(config["num_hidden_layers"]):
        p = f"model.layers.{layer}."
        n = rms_norm(x, weights[p + "input_layernorm.weight"], eps)
        q = linear(n, weights[p + "self_attn.q_proj.weight"])
        k = linear(n, weights[p + "self_attn.k_proj.weight"])
        v = linear(n, weights[p + "self_attn.v_proj.weight"])
        q = head_norm(q, n_q, d, weights[p + "self_attn.q_norm.weight"], eps)
        k = head_norm(k, n_kv, d, weights[p + "self_attn.k_norm.weight"], eps)
        q = rope(q, n_q, d, positions, theta)
        k = rope(k, n_kv, d, positions, theta)
        if kv_round is not None:
            k, v = kv_round(k).astype(DTYPE), kv_round(v).astype(DTYPE)
        a = causal_gqa(q, k, v, n_q, n_kv, d)
        x = x + linear(a, weights[p + "self_attn.o_proj.weight"])
        n = rms_norm(x, weights[p + "post_attention_layernorm.weight"], eps)
        x = x + swiglu_mlp(n, weights[p + "mlp.gate_proj.weight"], weights[p + "mlp.up_proj.weight"],
                           weights[p + "mlp.down_proj.weight"])
    n = rms_norm(x, weights["model.norm.weight"], eps)
    head = weights["model.embed_tokens.weight"] if config.get("tie_word_embeddings", False) else weights["lm_head.weight"]
    logits = linear(n, head)
    return (logits, x) if return_hidden else logits


def nmse(a, r):
    """sum((a - r)^2) / sum(r^2) in float64.  /root/reference/tests/kipp_test.c:1117-1127."""
    a = np.asarray(a, dtype=np.float64)
    r = np.asarray(r, dtype=np.float64)
    return float(np.sum((a - r) ** 2) / np.sum(r ** 2))
