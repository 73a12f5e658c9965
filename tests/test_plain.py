"""Pins of the plain implementation: vectors the reference's own tests hold,
special cases that reduce to a library routine, and invariants, each chosen so
that a plausible mistake (a wrong sign or pairing, a norm in the wrong place, a
wrong head mapping) fails it."""
import math

import numpy as np
import torch

from tests.plain import qwen3_plain as P


def test_bf16_vectors():
    # /root/reference/tests/kipp_test.c:56-62
    assert P.bf16_bits(np.float32(1.0)) == 0x3F80
    assert P.bf16_bits(np.float32(-2.0)) == 0xC000
    assert P.bf16_round(np.float32(1.00390625)) == np.float32(1.0)      # tie goes to the even mantissa
    assert P.bf16_round(np.float32(1.01171875)) == np.float32(1.015625)  # tie goes up to the even one
    x = np.random.default_rng(0).normal(size=4096).astype(np.float32) * 37
    assert np.array_equal(P.bf16_round(x), torch.tensor(x).bfloat16().float().numpy())
    assert np.array_equal(P.bf16_round(P.bf16_round(x)), P.bf16_round(x))


def test_rms_norm_vectors():
    # /root/reference/tests/kipp_test.c:88-96
    got = P.rms_norm(np.array([3.0, 4.0]), np.ones(2), 0.0)
    assert np.allclose(got, np.array([3.0, 4.0]) / math.sqrt(12.5), rtol=1e-12)
    # /root/reference/src/cuda/kipp_cuda.cu:964-970
    assert np.allclose(P.rms_norm(np.ones(128), np.ones(128), 1e-6), 1 / math.sqrt(1 + 1e-6), rtol=1e-12)
    # eps sits inside the root: a zero row stays zero and finite
    assert np.array_equal(P.rms_norm(np.zeros(8), np.ones(8), 1e-6), np.zeros(8))
    # the weight is a plain multiplier, not 1 + w
    assert np.allclose(P.rms_norm(np.array([3.0, 4.0]), np.zeros(2), 0.0), 0.0)
    x = np.random.default_rng(1).normal(size=(5, 33))
    assert np.allclose(np.sqrt(np.mean(P.rms_norm(x, np.ones(33), 0.0) ** 2, axis=-1)), 1.0)
    assert np.allclose(P.rms_norm(7.5 * x, np.ones(33), 0.0), P.rms_norm(x, np.ones(33), 0.0))
    ref = torch.nn.functional.rms_norm(torch.tensor(x), (33,), torch.ones(33, dtype=torch.float64), 1e-5).numpy()
    assert np.allclose(P.rms_norm(x, np.ones(33), 1e-5), ref, rtol=1e-12)


def test_linear_vector():
    # /root/reference/tests/kipp_test.c:98-108
    got = P.linear(np.array([2.0, -1.0, 0.5]), np.array([[1, 2, 3], [-1, 0.5, 0]]))
    assert np.allclose(got, [1.5, -2.5])
    assert np.allclose(P.linear(np.arange(4.0), np.eye(4)), np.arange(4.0))


def test_rope_vector_and_invariants():
    # /root/reference/tests/kipp_test.c:110-123: pins the half-split pairing (0,2),(1,3) and theta^(-2i/d)
    got = P.rope(np.array([[1.0, 2.0, 3.0, 4.0]]), 1, 4, [1], 10000.0)[0]
    c, s, c2, s2 = math.cos(1.0), math.sin(1.0), math.cos(0.01), math.sin(0.01)
    assert np.allclose(got, [c - 3 * s, 2 * c2 - 4 * s2, 3 * c + s, 4 * c2 + 2 * s2], rtol=1e-6)
    rng = np.random.default_rng(2)
    x = rng.normal(size=(1, 3 * 16))
    assert np.allclose(P.rope(x, 3, 16, [0], 1e6), x)                          # position 0 is the identity
    y = P.rope(x, 3, 16, [9], 1e6).reshape(3, 16)
    xh = x.reshape(3, 16)
    assert np.allclose(xh[:, :8] ** 2 + xh[:, 8:] ** 2, y[:, :8] ** 2 + y[:, 8:] ** 2)   # each pair keeps its length
    # it is the complex product (x_i + i x_{i+d/2}) * exp(i pos theta^(-2i/d))
    z = (xh[:, :8] + 1j * xh[:, 8:]) * np.exp(1j * 9 * np.power(1e6, -2.0 * np.arange(8) / 16))
    assert np.allclose(np.concatenate([z.real, z.imag], axis=1), y, rtol=1e-5)
    # scores depend on the distance only: <R_m q, R_n k> = <R_{m+7} q, R_{n+7} k>
    q, k = rng.normal(size=(1, 16)), rng.normal(size=(1, 16))
    a = P.rope(q, 1, 16, [5], 1e4) @ P.rope(k, 1, 16, [2], 1e4).T
    b = P.rope(q, 1, 16, [12], 1e4) @ P.rope(k, 1, 16, [9], 1e4).T
    assert np.allclose(a, b, rtol=1e-5)


def test_head_norm():
    # /root/reference/src/cuda/kipp_cuda.cu:959-992
    assert np.allclose(P.head_norm(np.ones((2, 3 * 8)), 3, 8, np.ones(8), 1e-6), 1 / math.sqrt(1 + 1e-6))
    rng = np.random.default_rng(3)
    x, w = rng.normal(size=(4, 3 * 8)), rng.normal(size=8)
    got = P.head_norm(x, 3, 8, w, 1e-5).reshape(4, 3, 8)
    for h in range(3):   # every head is normed on its own with the same weight
        assert np.allclose(got[:, h], P.rms_norm(x.reshape(4, 3, 8)[:, h], w, 1e-5))
    # norm before rotation: the other order gives another result when w is not constant
    a = P.rope(P.head_norm(x, 3, 8, w, 1e-5), 3, 8, np.arange(4), 1e4)
    b = P.head_norm(P.rope(x, 3, 8, np.arange(4), 1e4), 3, 8, w, 1e-5)
    assert not np.allclose(a, b)


def test_softmax_and_silu():
    # /root/reference/tests/kipp_test.c:125-132
    p = P.softmax(np.array([1.0, 2.0, 3.0]))
    assert abs(p.sum() - 1) < 1e-12 and p[0] < p[1] < p[2]
    assert np.allclose(P.softmax(np.array([1.0, 2.0, 3.0]) + 100), p)
    assert np.allclose(P.softmax(np.array([1000.0, 1000.0])), [0.5, 0.5])
    assert P.silu(np.float64(0.0)) == 0.0
    assert abs(P.silu(np.float64(1.0)) - 0.7310586) < 1e-7
    assert abs(P.silu(np.float64(1.0)) * 2 - 1.4621172) < 1e-6
    x = np.linspace(-5, 5, 11)
    assert np.allclose(P.silu(x), x * torch.sigmoid(torch.tensor(x)).numpy())


def test_causal_gqa_vector():
    # /root/reference/tests/kipp_test.c:135-175: q = k = 0, v0 = 1, v1 = 3 -> 1.0 then 2.0
    n_q, n_kv, d = 32, 8, 128
    q = np.zeros((2, n_q * d))
    k = np.zeros((2, n_kv * d))
    v = np.concatenate([np.ones((1, n_kv * d)), 3 * np.ones((1, n_kv * d))])
    out = P.causal_gqa(q, k, v, n_q, n_kv, d)
    assert np.allclose(out[0], 1.0) and np.allclose(out[1], 2.0)


def test_causal_gqa_special_cases():
    rng = np.random.default_rng(4)
    t, n_q, n_kv, d = 9, 6, 3, 16
    q, k, v = rng.normal(size=(t, n_q * d)), rng.normal(size=(t, n_kv * d)), rng.normal(size=(t, n_kv * d)) + 1
    out = P.causal_gqa(q, k, v, n_q, n_kv, d).reshape(t, n_q, d)
    # the library routine: dense causal attention with K and V heads repeated per group
    kk = torch.tensor(k).reshape(t, n_kv, d).repeat_interleave(n_q // n_kv, dim=1).transpose(0, 1)
    vv = torch.tensor(v).reshape(t, n_kv, d).repeat_interleave(n_q // n_kv, dim=1).transpose(0, 1)
    qq = torch.tensor(q).reshape(t, n_q, d).transpose(0, 1)
    ref = torch.nn.functional.scaled_dot_product_attention(qq, kk, vv, is_causal=True).transpose(0, 1).numpy()
    assert np.allclose(out, ref, rtol=1e-10, atol=1e-12)
    # consecutive query heads share a key/value head: h // (n_q / n_kv), not h % n_kv
    v2 = np.zeros((t, n_kv, d))
    v2[:, 1, :] = 1.0
    out2 = P.causal_gqa(q, k, v2.reshape(t, -1), n_q, n_kv, d).reshape(t, n_q, d)
    assert np.allclose(out2[:, [2, 3]], 1.0) and np.allclose(out2[:, [0, 1, 4, 5]], 0.0)
    # q = 0: the running mean of V; one token: V itself
    mean = P.causal_gqa(np.zeros_like(q), k, v, n_q, n_kv, d).reshape(t, n_q, d)
    vh = v.reshape(t, n_kv, d)
    assert np.allclose(mean[4, 0], vh[:5, 0].mean(axis=0)) and np.allclose(out[0, 5], vh[0, 2])
    # a token does not see later tokens
    k3, v3 = k.copy(), v.copy()
    k3[6:] += 5
    v3[6:] -= 3
    assert np.array_equal(P.causal_gqa(q, k3, v3, n_q, n_kv, d)[:6], out.reshape(t, -1)[:6])
    # a window of W keeps the last W sources, the token itself included
    w = P.causal_gqa(q, k, v, n_q, n_kv, d, window=3).reshape(t, n_q, d)
    ref_w = P.causal_gqa(q[5:8], k[5:8], v[5:8], n_q, n_kv, d).reshape(3, n_q, d)
    assert np.allclose(w[7], ref_w[2]) and np.allclose(w[1], out[1])


def _tiny(seed=0, tied=True):
    cfg = dict(vocab_size=50, hidden_size=24, intermediate_size=40, num_hidden_layers=2, num_attention_heads=3,
               num_key_value_heads=1, head_dim=16, rms_norm_eps=1e-5, rope_theta=100.0, tie_word_embeddings=tied)
    rng = np.random.default_rng(seed)
    w = {"model.embed_tokens.weight": rng.normal(size=(50, 24)) * 0.5, "model.norm.weight": 1 + 0.1 * rng.normal(size=24)}
    if not tied:
        w["lm_head.weight"] = rng.normal(size=(50, 24)) * 0.5
    for i in range(2):
        p = f"model.layers.{i}."
        w[p + "input_layernorm.weight"] = 1 + 0.1 * rng.normal(size=24)
        w[p + "post_attention_layernorm.weight"] = 1 + 0.1 * rng.normal(size=24)
        w[p + "self_attn.q_proj.weight"] = rng.normal(size=(48, 24)) * 0.3
        w[p + "self_attn.k_proj.weight"] = rng.normal(size=(16, 24)) * 0.3
        w[p + "self_attn.v_proj.weight"] = rng.normal(size=(16, 24)) * 0.3
        w[p + "self_attn.o_proj.weight"] = rng.normal(size=(24, 48)) * 0.3
        w[p + "self_attn.q_norm.weight"] = 1 + 0.1 * rng.normal(size=16)
        w[p + "self_attn.k_norm.weight"] = 1 + 0.1 * rng.normal(size=16)
        w[p + "mlp.gate_proj.weight"] = rng.normal(size=(40, 24)) * 0.3
        w[p + "mlp.up_proj.weight"] = rng.normal(size=(40, 24)) * 0.3
        w[p + "mlp.down_proj.weight"] = rng.normal(size=(24, 40)) * 0.3
    return cfg, w


def test_whole_model_closed_form_and_invariants():
    cfg, w = _tiny()
    tokens = [3, 17, 3, 44, 9, 21]
    base = P.forward_whole(cfg, w, tokens)
    # with zero output and down projections the residual stays the embedding
    w0 = dict(w)
    for i in range(2):
        w0[f"model.layers.{i}.self_attn.o_proj.weight"] = np.zeros((24, 48))
        w0[f"model.layers.{i}.mlp.down_proj.weight"] = np.zeros((24, 40))
    closed = P.rms_norm(w["model.embed_tokens.weight"][tokens], w["model.norm.weight"], 1e-5) @ w["model.embed_tokens.weight"].T
    assert np.allclose(P.forward_whole(cfg, w0, tokens), closed, rtol=1e-12)
    # causal: a prefix gives the same logits as the same positions of the whole
    assert np.allclose(P.forward_whole(cfg, w, tokens[:4]), base[:4], rtol=1e-10)
    # only distances between positions count
    assert np.allclose(P.forward_whole(cfg, w, tokens, position_offset=37), base, rtol=1e-4, atol=1e-6)
    # equal tokens at different positions give different logits (positions are used at all)
    assert not np.allclose(base[0], base[2])
    # an untied head that equals the embedding is the tied model
    cfg_u, w_u = dict(cfg, tie_word_embeddings=False), dict(w)
    w_u["lm_head.weight"] = w["model.embed_tokens.weight"]
    assert np.array_equal(P.forward_whole(cfg_u, w_u, tokens), base)
    # the reference rounds keys and values to bfloat16; that changes logits a little, not a lot
    rounded = P.forward_whole(cfg, w, tokens, kv_round=P.bf16_round)
    assert 0 < P.nmse(rounded, base) < 1e-4


def test_swiglu_vector_and_which_side_goes_through_silu():
    # /root/reference/tests/kipp_test.c:130-132: gate 1, up 2 -> silu(1) * 2 = 1.4621172, here through 1 x 1 weights
    one = np.ones((1, 1))
    assert abs(P.swiglu_mlp(np.array([[1.0]]), one, 2 * one, one)[0, 0] - 1.4621172) < 1e-6
    # the other way round it would be silu(2) * 1 = 1.7615942
    assert abs(P.swiglu_mlp(np.array([[1.0]]), 2 * one, one, one)[0, 0] - 1.7615942) < 1e-6
    # the delta is linear in W_up and not in W_gate
    rng = np.random.default_rng(5)
    x, wg, wu, wd = rng.normal(size=(3, 6)), rng.normal(size=(10, 6)), rng.normal(size=(10, 6)), rng.normal(size=(6, 10))
    base = P.swiglu_mlp(x, wg, wu, wd)
    assert np.allclose(P.swiglu_mlp(x, wg, 2 * wu, wd), 2 * base, rtol=1e-12)
    assert not np.allclose(P.swiglu_mlp(x, 2 * wg, wu, wd), 2 * base, rtol=1e-3)
    # a gate of zero closes the unit whatever the up side holds
    assert np.array_equal(P.swiglu_mlp(x, np.zeros_like(wg), wu, wd), np.zeros((3, 6)))


def test_block_arrangement():
    """Which norm feeds which half of a block, and that the residual itself is never normed."""
    cfg, w = _tiny(seed=3)
    cfg = dict(cfg, num_hidden_layers=1)
    tokens = [3, 17, 3, 44, 9, 21]
    p = "model.layers.0."
    emb = w["model.embed_tokens.weight"][tokens]
    _, hidden = P.forward_whole(cfg, w, tokens, return_hidden=True)
    # input_layernorm feeds the attention and nothing else: with its weight at zero q, k and v are zero, so is
    # the attention's delta, and what is left is x + mlp(norm(x, post_attention_layernorm)) of the plain embedding
    w_in0 = dict(w)
    w_in0[p + "input_layernorm.weight"] = np.zeros(24)
    _, h_in0 = P.forward_whole(cfg, w_in0, tokens, return_hidden=True)
    mlp_only = emb + P.swiglu_mlp(P.rms_norm(emb, w[p + "post_attention_layernorm.weight"], 1e-5),
                                  w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    assert np.allclose(h_in0, mlp_only, rtol=1e-12)
    # post_attention_layernorm feeds the feed-forward and nothing else: with its weight at zero the feed-forward's
    # delta is zero (silu(0) * 0), and the hidden state is the one of the same model with a zero down projection
    w_post0, w_down0 = dict(w), dict(w)
    w_post0[p + "post_attention_layernorm.weight"] = np.zeros(24)
    w_down0[p + "mlp.down_proj.weight"] = np.zeros((24, 40))
    _, h_post0 = P.forward_whole(cfg, w_post0, tokens, return_hidden=True)
    _, h_down0 = P.forward_whole(cfg, w_down0, tokens, return_hidden=True)
    assert np.array_equal(h_post0, h_down0) and not np.allclose(h_post0, emb)     # the attention's delta is still there
    # the feed-forward reads the residual AFTER the attention's delta was added: its own delta differs from the
    # one it would give on the embedding alone
    assert not np.allclose(hidden - h_down0, mlp_only - emb, rtol=1e-3)
    # pre-norm: a norm's weight reaches the residual only through its half's delta.  Scaling post_attention_layernorm
    # by c is the same as scaling the columns of W_gate and W_up by c (the delta is linear in W_up's input side)
    w_c, w_cols = dict(w), dict(w)
    w_c[p + "post_attention_layernorm.weight"] = 1.7 * w[p + "post_attention_layernorm.weight"]
    w_cols[p + "mlp.gate_proj.weight"] = 1.7 * w[p + "mlp.gate_proj.weight"]
    w_cols[p + "mlp.up_proj.weight"] = 1.7 * w[p + "mlp.up_proj.weight"]
    assert np.allclose(P.forward_whole(cfg, w_c, tokens), P.forward_whole(cfg, w_cols, tokens), rtol=1e-12)
    # ... and scaling input_layernorm by c is the same as scaling W_q, W_k and W_v by c
    w_c, w_cols = dict(w), dict(w)
    w_c[p + "input_layernorm.weight"] = 0.6 * w[p + "input_layernorm.weight"]
    for name in ("q_proj", "k_proj", "v_proj"):
        w_cols[p + f"self_attn.{name}.weight"] = 0.6 * w[p + f"self_attn.{name}.weight"]
    assert np.allclose(P.forward_whole(cfg, w_c, tokens), P.forward_whole(cfg, w_cols, tokens), rtol=1e-12)
    # the final norm is applied once, after the last block, with model.norm.weight
    assert np.allclose(P.forward_whole(cfg, w, tokens), P.rms_norm(hidden, w["model.norm.weight"], 1e-5)
                       @ w["model.embed_tokens.weight"].T, rtol=1e-12)


def test_q_norm_and_k_norm_are_not_interchangeable():
    """q_norm.weight belongs to the queries.  With it at zero on the upper half of a head, the upper halves of
    the (normed) queries vanish, so flipping the sign of those rows of W_q changes nothing (a sign leaves the
    norm's scale alone), while the same flip in W_k does; were the two weights applied the other way round,
    it would be the flip in W_q that shows."""
    cfg, w = _tiny(seed=4)
    cfg = dict(cfg, num_hidden_layers=1)
    tokens = [7, 1, 30, 30, 12, 5, 48]
    p = "model.layers.0.self_attn."
    rng = np.random.default_rng(6)
    w = dict(w)
    w[p + "q_norm.weight"] = np.concatenate([1 + 0.3 * rng.normal(size=8), np.zeros(8)])
    w[p + "k_norm.weight"] = 1 + 0.3 * rng.normal(size=16)
    base = P.forward_whole(cfg, w, tokens)
    upper = np.tile(np.concatenate([np.ones(8), -np.ones(8)]), 3)        # 3 query heads of 16
    flipped_q, flipped_k = dict(w), dict(w)
    flipped_q[p + "q_proj.weight"] = w[p + "q_proj.weight"] * upper[:, None]
    flipped_k[p + "k_proj.weight"] = w[p + "k_proj.weight"] * upper[:16, None]
    assert np.allclose(P.forward_whole(cfg, flipped_q, tokens), base, rtol=1e-12)
    assert not np.allclose(P.forward_whole(cfg, flipped_k, tokens), base, rtol=1e-3)
    # and the mirror image pins k_norm.weight to the keys
    w[p + "q_norm.weight"], w[p + "k_norm.weight"] = w[p + "k_norm.weight"], w[p + "q_norm.weight"]
    base = P.forward_whole(cfg, w, tokens)
    flipped_q, flipped_k = dict(w), dict(w)
    flipped_q[p + "q_proj.weight"] = w[p + "q_proj.weight"] * upper[:, None]
    flipped_k[p + "k_proj.weight"] = w[p + "k_proj.weight"] * upper[:16, None]
    assert np.allclose(P.forward_whole(cfg, flipped_k, tokens), base, rtol=1e-12)
    assert not np.allclose(P.forward_whole(cfg, flipped_q, tokens), base, rtol=1e-3)


def test_the_second_plain_implementation_agrees(model_folders):
    """Scalar loops over tokens, heads and sources with a running cache, written on its own
    (`tests/plain/qwen3_loops.py`), against the whole-sequence NumPy form, on both tiny configurations
    (float32 and bfloat16 files): relative difference below 1e-12 at every logit's scale."""
    from tests.plain import qwen3_loops as L
    for (key, dtype), folder in sorted(model_folders.items()):
        cfg, weights = P.load_folder(folder)
        cfg2, weights2 = L.read_folder(folder)
        assert cfg2 == cfg and sorted(weights2) == sorted(weights)
        assert all(np.array_equal(weights[name], weights2[name]) for name in weights)
        vocab = cfg["vocab_size"]
        tokens = [int(t) for t in np.random.default_rng(11).integers(0, vocab, size=19)]
        a, b = P.forward_whole(cfg, weights, tokens), L.forward(cfg2, weights2, tokens)
        assert a.shape == b.shape == (19, vocab)
        assert np.abs(a - b).max() <= 1e-12 * np.abs(a).max(), (key, dtype, np.abs(a - b).max(), np.abs(a).max())
    # and on the hand-made model of these tests, whose norm weights differ more from one
    cfg, w = _tiny(seed=9, tied=False)
    tokens = [3, 17, 3, 44, 9, 21, 0, 49]
    a, b = P.forward_whole(cfg, w, tokens), L.forward(cfg, w, tokens)
    assert np.abs(a - b).max() <= 1e-12 * np.abs(a).max()
