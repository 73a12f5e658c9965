"""The framework is open: a mixer with state of its own, a windowed attention
layer, a layer named twice and a layer that reads another layer's cache are
defined HERE, registered, built and stepped without a change to the
framework's files.  None of this is a model of anyone's."""
from dataclasses import dataclass

import numpy as np
import pytest
import torch

from tests import helpers as H
from tests.plain import qwen3_plain as plain

pytestmark = pytest.mark.gpu

HIDDEN, VOCAB, HEADS, KV, D, INNER, EPS, THETA, WINDOW, DECAY = 48, 97, 3, 1, 16, 56, 1e-5, 500.0, 11, 0.75


@dataclass(frozen=True)
class DecaySpec:
    hidden_size: int
    decay: float
    prefix: str = ""
    kind: str = "toy_decay"


def _register():
    from kipp_amd.cache import StateNeed
    from kipp_amd.config import register_architecture
    from kipp_amd.config.specs import (AttentionSpec, EmbeddingSpec, GatedMLPSpec, HeadSpec, LayerRun, LayerSpec,
                                       ModelSpec, RMSNormSpec, RopeSpec)
    from kipp_amd.parts import ParamSpec, register

    @register("mixer", "toy_decay")
    class DecayMixer:
        """s_t = decay * s_{t-1} + x_t per request; delta_t = W s_t.  The state s
        lives in the request's slot and is carried across steps."""

        def __init__(self, spec, runtime):
            self.spec, self.rt = spec, runtime

        @staticmethod
        def params(spec):
            return {"mix.weight": ParamSpec((spec.hidden_size, spec.hidden_size))}

        def load(self, tensors):
            self.w = tensors["mix.weight"]

        def cache_need(self):
            return None

        def state_need(self):
            return StateNeed((self.spec.hidden_size,), "float32")

        def forward(self, x, batch, cache, state):
            assert cache is None and state is not None
            out = torch.empty(x.shape, dtype=torch.float32, device=x.device)
            slots = batch.slots.cpu().tolist()
            for start, n, slot in zip(batch.host["q_start"], batch.host["q_len"], slots):
                s = state[slot]
                for t in range(start, start + n):
                    s = self.spec.decay * s + x[t].float()
                    out[t] = s
                state[slot] = s
            return self.rt.linear(out.to(x.dtype), self.w)

    class ToyConfig:
        def __init__(self, d):
            self.d = d

        def to_dict(self):
            return dict(self.d)

        def model_spec(self):
            def layer(i, mixer):
                p = f"layers.{i}."
                return LayerSpec(block="pre_norm", parts=(
                    ("mixer_norm", RMSNormSpec(HIDDEN, EPS, p + "n1.")), ("mixer", mixer),
                    ("ffn_norm", RMSNormSpec(HIDDEN, EPS, p + "n2.")), ("ffn", GatedMLPSpec(HIDDEN, INNER, "silu", p + "mlp."))))

            def attn(i, window):
                return AttentionSpec(HIDDEN, HEADS, KV, D, position=RopeSpec(D, THETA), qk_norm_eps=None, window=window,
                                     prefix=f"layers.{i}.attn.")
            layers = (layer(0, attn(0, None)), layer(1, DecaySpec(HIDDEN, DECAY, "layers.1.decay.")), layer(2, attn(2, WINDOW)))
            # layer 0 runs twice (the second time with a cache of its own), and the
            # last run is layer 0 once more reading the cache of the first run
            order = (LayerRun(0), LayerRun(1), LayerRun(2), LayerRun(0), LayerRun(0, cache_of=0))
            return ModelSpec("ToyForTests", HIDDEN, VOCAB, 256, EmbeddingSpec(VOCAB, HIDDEN, "embed."), layers, order,
                             RMSNormSpec(HIDDEN, EPS, "norm."), HeadSpec(VOCAB, HIDDEN, True))

    register_architecture("ToyForTests", ToyConfig)


def _plain_toy(w, tokens):
    """The same toy model over a whole sequence, from plain parts."""
    t = len(tokens)
    pos = np.arange(t)
    x = plain.embed(w["embed.weight"], tokens)
    kv0 = {}

    def attention(i, n, window, reuse=None):
        p = f"layers.{i}.attn."
        q = plain.rope(plain.linear(n, w[p + "q_proj.weight"]), HEADS, D, pos, THETA)
        if reuse is None:
            k = plain.rope(plain.linear(n, w[p + "k_proj.weight"]), KV, D, pos, THETA)
            v = plain.linear(n, w[p + "v_proj.weight"])
        else:
            k, v = reuse
        a = plain.causal_gqa(q, k, v, HEADS, KV, D, window=window)
        return plain.linear(a, w[p + "o_proj.weight"]), (k, v)

    def decay(n):
        s, out = np.zeros(HIDDEN), []
        for row in n:
            s = DECAY * s + row
            out.append(s)
        return plain.linear(np.stack(out), w["layers.1.decay.mix.weight"])

    for run, (layer, reuse) in enumerate([(0, False), (1, False), (2, False), (0, False), (0, True)]):
        p = f"layers.{layer}."
        n = plain.rms_norm(x, w[p + "n1.weight"], EPS)
        if layer == 1:
            delta = decay(n)
        elif layer == 2:
            delta, _ = attention(2, n, WINDOW)
        else:
            delta, kv = attention(0, n, None, reuse=kv0.get("first") if reuse else None)
            kv0.setdefault("first", kv)
        x = x + delta
        n = plain.rms_norm(x, w[p + "n2.weight"], EPS)
        x = x + plain.swiglu_mlp(n, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    return plain.linear(plain.rms_norm(x, w["norm.weight"], EPS), w["embed.weight"])


@pytest.fixture(scope="module")
def toy_folder(tmp_path_factory):
    _register()
    from kipp_amd.weights import write_random_model
    folder = str(tmp_path_factory.mktemp("toy") / "model")
    write_random_model(folder, {"architectures": ["ToyForTests"]}, seed=3, dtype="float32")
    yield folder
    from kipp_amd.config import unregister_architecture
    from kipp_amd.parts import unregister
    unregister_architecture("ToyForTests")
    unregister("mixer", "toy_decay")


@pytest.mark.parametrize("cut", ["whole", "tail", "portions", "mixed"])
def test_toy_model_steps_like_its_plain_form(toy_folder, cut):
    from kipp_amd.engine import Engine
    _, weights = plain.load_folder(toy_folder)
    requests = {f"t{i}": H.random_tokens(i, n, VOCAB) for i, n in enumerate([5, 40, 64, 23, 31])}
    steps = {"whole": H.whole, "tail": H.tail_one_by_one, "portions": H.changing_portions,
             "mixed": lambda r: H.mixed(r, seed=2)}[cut](requests)
    engine = Engine.from_folder(toy_folder, dtype="float32", page_size=4, num_pages=H.peak_pages(requests, steps, 4),
                                max_requests=4)
    cache = engine.cache
    assert len(cache.groups) == 2 and cache.groups[0].runs == [0, 3] and cache.groups[1].runs == [2]
    assert list(cache.states) == [1] and not cache.share
    got = H.replay(engine, requests, steps)
    for rid, toks in requests.items():
        H.assert_close(got[rid], _plain_toy(weights, toks), H.NMSE_F32, f"toy/{cut}/{rid}")
    assert cache.free_pages() == [g.pool.num_pages for g in cache.groups]


def test_window_pages_return_early_and_slots_start_from_zero(toy_folder):
    from kipp_amd.engine import Engine, StepEntry
    _, weights = plain.load_folder(toy_folder)
    engine = Engine.from_folder(toy_folder, dtype="float32", page_size=4, num_pages=20, max_requests=1)
    toks = H.random_tokens(9, 50, VOCAB)
    engine.step([StepEntry("w", toks, [])])
    full, windowed = engine.cache.free_pages()
    assert full == 20 - 13 and windowed == 20 - 3        # only the pages the window still covers are held
    engine.close("w")
    # the one slot is used again: the state of the request before must not leak
    again = H.random_tokens(10, 12, VOCAB)
    got = engine.step([StepEntry("x", again, list(range(12)))]).cpu().numpy()
    H.assert_close(got, _plain_toy(weights, again), H.NMSE_F32, "slot reuse")
