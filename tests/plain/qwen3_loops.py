"""A second plain implementation of the Qwen3 dense decoder, written on its own from the
reference's formulas and sharing nothing with `qwen3_plain.py` (no import, no helper): scalar
loops over tokens, heads and source positions in float64, a running cache of keys and values as
the reference's token-by-token path keeps one, the rotation as a complex product.  The two
implementations check each other; a mistake would have to be made twice in different code.

The one float32 value is the rotation angle, `(float)position * frequency` with a float32
frequency (/root/reference/src/kipp.c:2368-2382).
"""
import json
import math
import os

import numpy as np


def _matvec(weight, x):
    """y[o] = sum_i W[o][i] x[i]  (/root/reference/src/kipp.c:2233-2244)."""
    return [float(np.dot(weight[o], x)) for o in range(weight.shape[0])]


def _norm(x, weight, eps):
    """/root/reference/src/kipp.c:2221-2231: sum of squares, 1 / sqrt(mean + eps), times weight."""
    total = 0.0
    for v in x:
        total += v * v
    scale = 1.0 / math.sqrt(total / len(x) + eps)
    return [x[i] * scale * float(weight[i]) for i in range(len(x))]


def _rotate(head, position, theta):
    """/root/reference/src/kipp.c:2368-2382: pair (i, i + d/2) turned by position * theta^(-2i/d)."""
    d = len(head)
    half = d // 2
    out = [0.0] * d
    for i in range(half):
        frequency = np.float32(math.pow(theta, -(2.0 * i) / d))
        angle = float(np.float32(position) * frequency)
        z = complex(head[i], head[i + half]) * complex(math.cos(angle), math.sin(angle))
        out[i], out[i + half] = z.real, z.imag
    return out


def forward(config, weights, tokens):
    """float64 logits [len(tokens), vocab]; the tokens are run one after another, each over the
    keys and values of the tokens before it (/root/reference/src/kipp.c:2924-3020, the cached
    path, without its rounding of the cache to bfloat16)."""
    layers = config["num_hidden_layers"]
    n_q = config["num_attention_heads"]
    n_kv = config["num_key_value_heads"]
    d = config.get("head_dim") or config["hidden_size"] // n_q
    eps = config["rms_norm_eps"]
    theta = config["rope_theta"]
    share = n_q // n_kv
    w = {k: np.asarray(v, dtype=np.float64) for k, v in weights.items()}
    head = w["model.embed_tokens.weight"] if config.get("tie_word_embeddings", False) else w["lm_head.weight"]
    keys = [[] for _ in range(layers)]       # keys[layer][position][kv head] -> list of d
    values = [[] for _ in range(layers)]
    logits = []
    for position, token in enumerate(tokens):
        x = [float(v) for v in w["model.embed_tokens.weight"][token]]
        for layer in range(layers):
            p = f"model.layers.{layer}."
            h = np.array(_norm(x, w[p + "input_layernorm.weight"], eps))
            q = _matvec(w[p + "self_attn.q_proj.weight"], h)
            k = _matvec(w[p + "self_attn.k_proj.weight"], h)
            v = _matvec(w[p + "self_attn.v_proj.weight"], h)
            q_heads = [_rotate(_norm(q[a * d:(a + 1) * d], w[p + "self_attn.q_norm.weight"], eps), position, theta)
                       for a in range(n_q)]
            k_heads = [_rotate(_norm(k[a * d:(a + 1) * d], w[p + "self_attn.k_norm.weight"], eps), position, theta)
                       for a in range(n_kv)]
            keys[layer].append(k_heads)
            values[layer].append([v[a * d:(a + 1) * d] for a in range(n_kv)])
            attended = []
            for a in range(n_q):
                g = a // share
                scores = []
                for s in range(position + 1):
                    dot = 0.0
                    for j in range(d):
                        dot += q_heads[a][j] * keys[layer][s][g][j]
                    scores.append(dot * (1.0 / math.sqrt(d)))
                top = max(scores)
                e = [math.exp(sc - top) for sc in scores]
                z = 0.0
                for ev in e:
                    z += ev
                out = [0.0] * d
                for s in range(position + 1):
                    prob = e[s] * (1.0 / z)
                    for j in range(d):
                        out[j] += prob * values[layer][s][g][j]
                attended.extend(out)
            delta = _matvec(w[p + "self_attn.o_proj.weight"], np.array(attended))
            x = [x[i] + delta[i] for i in range(len(x))]
            h = np.array(_norm(x, w[p + "post_attention_layernorm.weight"], eps))
            gate = _matvec(w[p + "mlp.gate_proj.weight"], h)
            up = _matvec(w[p + "mlp.up_proj.weight"], h)
            act = np.array([(gate[i] / (1.0 + math.exp(-gate[i]))) * up[i] for i in range(len(gate))])
            delta = _matvec(w[p + "mlp.down_proj.weight"], act)
            x = [x[i] + delta[i] for i in range(len(x))]
        logits.append(_matvec(head, np.array(_norm(x, w["model.norm.weight"], eps))))
    return np.array(logits, dtype=np.float64)


def read_folder(model_dir):
    """(config, {name: float64 array}) with the framework's own file reader left out of it too:
    the safetensors header is parsed here (8 bytes of length, JSON, raw little-endian data)."""
    with open(os.path.join(model_dir, "config.json"), "r", encoding="utf-8") as f:
        config = json.load(f)
    tensors = {}
    with open(os.path.join(model_dir, "model.safetensors"), "rb") as f:
        size = int.from_bytes(f.read(8), "little")
        header = json.loads(f.read(size))
        data = f.read()
    for name, info in header.items():
        if name == "__metadata__":
            continue
        begin, end = info["data_offsets"]
        raw = data[begin:end]
        if info["dtype"] == "F32":
            values = np.frombuffer(raw, dtype="<f4").astype(np.float64)
        elif info["dtype"] == "BF16":
            values = (np.frombuffer(raw, dtype="<u2").astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        else:
            raise ValueError(f"{name}: type {info['dtype']} is not read here")
        tensors[name] = values.reshape(info["shape"])
    return config, tensors
