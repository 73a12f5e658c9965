"""The framework is open: a mixer with state of its own, a windowed attention
layer, a layer named twice, a layer that reads another layer's cache, a
feed-forward with routing and another position encoding are defined HERE,
registered, built and stepped without a change to the framework's files.
None of this is a model of anyone's."""
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


# ---------------------------------------------------------------------------------------------------
# A feed-forward with routing and another position encoding, again defined here only.

EXPERTS, R_INNER, STRETCH = 3, 24, 4.0


@dataclass(frozen=True)
class RoutedSpec:
    hidden_size: int
    experts: int
    inner: int
    prefix: str = ""
    kind: str = "toy_routed"


@dataclass(frozen=True)
class StretchedRopeSpec:
    head_dim: int
    theta: float
    stretch: float
    kind: str = "toy_stretched_rope"


def _register_routed():
    from kipp_amd.config import register_architecture
    from kipp_amd.config.specs import (AttentionSpec, EmbeddingSpec, HeadSpec, LayerRun, LayerSpec, ModelSpec, RMSNormSpec)
    from kipp_amd.parts import ParamSpec, register

    @register("feed_forward", "toy_routed")
    class RoutedFFN:
        """Every token goes to the one expert its router logit is largest for;
        delta = p * W2_e silu(W1_e x) with p the softmax weight of that expert
        (router logits and softmax in float32)."""

        def __init__(self, spec, runtime):
            self.spec, self.rt = spec, runtime

        @staticmethod
        def params(spec):
            out = {"router.weight": ParamSpec((spec.experts, spec.hidden_size))}
            for e in range(spec.experts):
                out[f"experts.{e}.w1.weight"] = ParamSpec((spec.inner, spec.hidden_size))
                out[f"experts.{e}.w2.weight"] = ParamSpec((spec.hidden_size, spec.inner))
            return out

        def load(self, tensors):
            self.t = tensors

        def forward(self, x, batch=None):
            logits = self.rt.linear(x, self.t["router.weight"])
            weight, expert = torch.softmax(logits.float(), dim=-1).max(dim=-1)
            delta = torch.zeros(x.shape, dtype=torch.float32, device=x.device)
            for e in range(self.spec.experts):
                rows = (expert == e).nonzero().flatten()
                if rows.numel():
                    h = torch.nn.functional.silu(self.rt.linear(x[rows].contiguous(), self.t[f"experts.{e}.w1.weight"]))
                    delta[rows] = self.rt.linear(h.to(x.dtype).contiguous(), self.t[f"experts.{e}.w2.weight"]) * weight[rows, None]
            return delta

    @register("position", "toy_stretched_rope")
    class StretchedRope:
        """Rotation with every frequency divided by `stretch`.  It gives the mixer its
        table of frequencies and nothing else: the mixer computes the angles itself."""

        def __init__(self, spec, runtime):
            i = torch.arange(spec.head_dim // 2, dtype=torch.float64)
            freq = torch.pow(torch.tensor(float(spec.theta), dtype=torch.float64), -(2.0 * i) / spec.head_dim) / spec.stretch
            self.inv_freq, self.head_dim = freq.to(device=runtime.device, dtype=torch.float32), spec.head_dim

        @staticmethod
        def params(spec):
            return {}

        def load(self, tensors):
            pass

        def rotary_table(self):
            return self.inv_freq, self.head_dim

    class RoutedConfig:
        def __init__(self, d):
            self.d = d

        def to_dict(self):
            return dict(self.d)

        def model_spec(self):
            def layer(i):
                p = f"layers.{i}."
                attn = AttentionSpec(HIDDEN, HEADS, KV, D, position=StretchedRopeSpec(D, THETA, STRETCH), qk_norm_eps=None,
                                     prefix=p + "attn.")
                return LayerSpec(block="pre_norm", parts=(
                    ("mixer_norm", RMSNormSpec(HIDDEN, EPS, p + "n1.")), ("mixer", attn),
                    ("ffn_norm", RMSNormSpec(HIDDEN, EPS, p + "n2.")), ("ffn", RoutedSpec(HIDDEN, EXPERTS, R_INNER, p + "moe."))))
            layers = (layer(0), layer(1))
            return ModelSpec("ToyRoutedForTests", HIDDEN, VOCAB, 256, EmbeddingSpec(VOCAB, HIDDEN, "embed."), layers,
                             (LayerRun(0), LayerRun(1)), RMSNormSpec(HIDDEN, EPS, "norm."), HeadSpec(VOCAB, HIDDEN, True))

    register_architecture("ToyRoutedForTests", RoutedConfig)


def _plain_routed(w, tokens):
    t = len(tokens)
    pos = np.arange(t) / STRETCH                        # dividing the frequencies is dividing the positions
    x = plain.embed(w["embed.weight"], tokens)
    for i in range(2):
        p = f"layers.{i}."
        n = plain.rms_norm(x, w[p + "n1.weight"], EPS)
        q = plain.rope(plain.linear(n, w[p + "attn.q_proj.weight"]), HEADS, D, pos, THETA)
        k = plain.rope(plain.linear(n, w[p + "attn.k_proj.weight"]), KV, D, pos, THETA)
        v = plain.linear(n, w[p + "attn.v_proj.weight"])
        x = x + plain.linear(plain.causal_gqa(q, k, v, HEADS, KV, D), w[p + "attn.o_proj.weight"])
        n = plain.rms_norm(x, w[p + "n2.weight"], EPS)
        probs = plain.softmax(plain.linear(n, w[p + "moe.router.weight"]))
        delta = np.zeros_like(x)
        for row in range(t):
            e = int(probs[row].argmax())
            h = plain.silu(plain.linear(n[row:row + 1], w[p + f"moe.experts.{e}.w1.weight"]))
            delta[row] = probs[row, e] * plain.linear(h, w[p + f"moe.experts.{e}.w2.weight"])[0]
        x = x + delta
    return plain.linear(plain.rms_norm(x, w["norm.weight"], EPS), w["embed.weight"])


@pytest.mark.parametrize("cut", ["whole", "portions", "mixed"])
def test_routed_feed_forward_and_another_position_encoding(tmp_path, cut):
    from kipp_amd.config import unregister_architecture
    from kipp_amd.engine import Engine
    from kipp_amd.parts import unregister
    from kipp_amd.weights import write_random_model
    _register_routed()
    try:
        folder = write_random_model(str(tmp_path / "routed"), {"architectures": ["ToyRoutedForTests"]}, seed=8, dtype="float32")
        _, weights = plain.load_folder(folder)
        requests = {f"r{i}": H.random_tokens(20 + i, n, VOCAB) for i, n in enumerate([7, 45, 30])}
        steps = {"whole": H.whole, "portions": H.changing_portions, "mixed": lambda r: H.mixed(r, seed=5)}[cut](requests)
        engine = Engine.from_folder(folder, dtype="float32", page_size=8, num_pages=H.peak_pages(requests, steps, 8),
                                    max_requests=4)
        assert engine.graphs is None or not engine.graphs.possible          # parts that do not declare graph_safe run eagerly
        got = H.replay(engine, requests, steps)
        for rid, toks in requests.items():
            H.assert_close(got[rid], _plain_routed(weights, toks), H.NMSE_F32, f"routed/{cut}/{rid}")
        assert engine.cache.free_pages() == [engine.cache.groups[0].pool.num_pages]
    finally:
        unregister_architecture("ToyRoutedForTests")
        unregister("feed_forward", "toy_routed")
        unregister("position", "toy_stretched_rope")


# ---------------------------------------------------------------------------------------------
# A norm and a feed-forward of other kinds between the framework's own parts, in bfloat16: with few rows the framework's
# products come back not yet launched and its norm leaves its scale to the next product; a norm that
# knows nothing of either gets tensors, and the parts behind it work as before.

@dataclass(frozen=True)
class MeanAbsNormSpec:
    width: int
    eps: float
    prefix: str = ""
    kind: str = "toy_mean_abs"


@dataclass(frozen=True)
class ReluMLPSpec:
    hidden_size: int
    inner: int
    prefix: str = ""
    kind: str = "toy_relu_mlp"


def _register_mean_abs():
    from kipp_amd.config import register_architecture
    from kipp_amd.config.specs import (AttentionSpec, EmbeddingSpec, GatedMLPSpec, HeadSpec, LayerRun, LayerSpec, ModelSpec,
                                       RMSNormSpec, RopeSpec)
    from kipp_amd.parts import ParamSpec, register

    @register("norm", "toy_mean_abs")
    class MeanAbsNorm:
        """y = x / (mean |x| + eps) * w."""

        def __init__(self, spec, runtime):
            self.spec, self.rt = spec, runtime

        @staticmethod
        def params(spec):
            return {"weight": ParamSpec((spec.width,), "float", ("one_plus_normal", 0.05))}

        @staticmethod
        def placement(spec):
            return {"weight": "float32"}

        def load(self, tensors):
            self.weight = tensors["weight"]

        def forward(self, x, out_dtype):
            return (x / (x.abs().mean(dim=-1, keepdim=True) + self.spec.eps) * self.weight).to(out_dtype)

        def add_forward(self, x, delta, out_dtype):
            assert isinstance(delta, torch.Tensor), "a norm that does not declare fuses_products gets tensors"
            x += delta.sum(dim=0) if delta.dim() == 3 else delta
            return self.forward(x, out_dtype)

    @register("feed_forward", "toy_relu_mlp")
    class ReluMLP:
        """delta = W2 relu(W1 x).  It does not declare `takes_scaled_rows`: the block hands it finished rows."""

        def __init__(self, spec, runtime):
            self.spec, self.rt = spec, runtime

        @staticmethod
        def params(spec):
            return {"w1.weight": ParamSpec((spec.inner, spec.hidden_size)), "w2.weight": ParamSpec((spec.hidden_size, spec.inner))}

        def load(self, tensors):
            self.t = tensors

        def forward(self, x, batch=None):
            assert isinstance(x, torch.Tensor), "a feed-forward that does not declare takes_scaled_rows gets tensors"
            h = torch.relu(self.rt.linear(x, self.t["w1.weight"])).to(x.dtype).contiguous()
            return self.rt.linear(h, self.t["w2.weight"])

    class MeanAbsConfig:
        def __init__(self, d):
            self.d = d

        def to_dict(self):
            return dict(self.d)

        def model_spec(self):
            def layer(i):
                p = f"layers.{i}."
                attn = AttentionSpec(M_HIDDEN, 4, 2, 32, position=RopeSpec(32, THETA), qk_norm_eps=EPS, prefix=p + "attn.")
                if i == 2:      # the framework's norm in front of a feed-forward of another kind
                    return LayerSpec(block="pre_norm", parts=(
                        ("mixer_norm", RMSNormSpec(M_HIDDEN, EPS, p + "n1.")), ("mixer", attn),
                        ("ffn_norm", RMSNormSpec(M_HIDDEN, EPS, p + "n2.")), ("ffn", ReluMLPSpec(M_HIDDEN, M_INNER, p + "mlp."))))
                return LayerSpec(block="pre_norm", parts=(
                    ("mixer_norm", RMSNormSpec(M_HIDDEN, EPS, p + "n1.")), ("mixer", attn),
                    ("ffn_norm", MeanAbsNormSpec(M_HIDDEN, EPS, p + "n2.")), ("ffn", GatedMLPSpec(M_HIDDEN, M_INNER, prefix=p + "mlp."))))
            return ModelSpec("ToyMeanAbsForTests", M_HIDDEN, VOCAB, 256, EmbeddingSpec(VOCAB, M_HIDDEN, "embed."),
                             (layer(0), layer(1), layer(2)), (LayerRun(0), LayerRun(1), LayerRun(2)),
                             MeanAbsNormSpec(M_HIDDEN, EPS, "norm."),
                             HeadSpec(VOCAB, M_HIDDEN, True))

    register_architecture("ToyMeanAbsForTests", MeanAbsConfig)


M_HIDDEN, M_INNER = 64, 96


def _plain_mean_abs(w, tokens):
    def mean_abs(x, weight):
        return x / (np.abs(x).mean(axis=-1, keepdims=True) + EPS) * weight
    pos = np.arange(len(tokens))
    x = plain.embed(w["embed.weight"], tokens)
    for i in range(3):
        p = f"layers.{i}."
        n = plain.rms_norm(x, w[p + "n1.weight"], EPS)
        q = plain.head_norm(plain.linear(n, w[p + "attn.q_proj.weight"]), 4, 32, w[p + "attn.q_norm.weight"], EPS)
        k = plain.head_norm(plain.linear(n, w[p + "attn.k_proj.weight"]), 2, 32, w[p + "attn.k_norm.weight"], EPS)
        q, k = plain.rope(q, 4, 32, pos, THETA), plain.rope(k, 2, 32, pos, THETA)
        v = plain.linear(n, w[p + "attn.v_proj.weight"])
        x = x + plain.linear(plain.causal_gqa(q, k, v, 4, 2, 32), w[p + "attn.o_proj.weight"])
        if i == 2:
            n = plain.rms_norm(x, w[p + "n2.weight"], EPS)
            x = x + plain.linear(np.maximum(plain.linear(n, w[p + "mlp.w1.weight"]), 0.0), w[p + "mlp.w2.weight"])
            continue
        n = mean_abs(x, w[p + "n2.weight"])
        x = x + plain.swiglu_mlp(n, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    return plain.linear(mean_abs(x, w["norm.weight"]), w["embed.weight"])


@pytest.mark.parametrize("cut", ["tail", "mixed"])
def test_another_norm_between_products_that_fuse_theirs(tmp_path, cut):
    from kipp_amd.config import unregister_architecture
    from kipp_amd.engine import Engine
    from kipp_amd.parts import unregister
    from kipp_amd.runtime import Deferred, ScaledRows
    from kipp_amd.weights import write_random_model
    _register_mean_abs()
    try:
        folder = write_random_model(str(tmp_path / "meanabs"), {"architectures": ["ToyMeanAbsForTests"]}, seed=12, dtype="bfloat16")
        _, weights = plain.load_folder(folder)
        requests = {f"r{i}": H.random_tokens(40 + i, n, VOCAB) for i, n in enumerate([37, 52, 44])}
        steps = {"tail": H.tail_one_by_one, "mixed": lambda r: H.mixed(r, seed=6)}[cut](requests)
        engine = Engine.from_folder(folder, dtype="bfloat16", page_size=8, max_tokens=256, max_requests=4)
        # the framework's parts did fuse where they met each other: the second layer's first norm got a product
        # that was not launched yet and handed rows without their scale to the attention
        seen = {"deferred": 0, "scaled": 0, "finished": 0}
        inner_rows = engine.model.rt.rows_of

        def rows_of(h):
            seen["finished"] += isinstance(h, ScaledRows)
            return inner_rows(h)
        engine.model.rt.rows_of = rows_of
        norm1, mixer = engine.model.blocks[1].parts["mixer_norm"], engine.model.blocks[1].parts["mixer"]
        inner_add, inner_mix = norm1.add_forward, mixer.forward

        def add_forward(x, delta, out_dtype):
            seen["deferred"] += isinstance(delta, Deferred)
            return inner_add(x, delta, out_dtype)

        def forward(x, *rest):
            seen["scaled"] += isinstance(x, ScaledRows)
            return inner_mix(x, *rest)
        norm1.add_forward, mixer.forward = add_forward, forward
        got = H.replay(engine, requests, steps)
        for rid, toks in requests.items():
            H.assert_close(got[rid], _plain_mean_abs(weights, toks), H.NMSE_BF16["tiny"], f"mean-abs norm/{cut}/{rid}")
        # and the block finished the rows of the framework's norm for the feed-forward of another kind
        assert seen["deferred"] > 0 and seen["scaled"] > 0 and seen["finished"] > 0, seen
    finally:
        unregister_architecture("ToyMeanAbsForTests")
        unregister("norm", "toy_mean_abs")
        unregister("feed_forward", "toy_relu_mlp")


# ---------------------------------------------------------------------------------------------
# Two attention layers of different geometry in one model (head counts, head sizes, one with a window),
# rotary encodings of both pairings (one over a part of the head only), and a position encoding that is
# no rotation at all: a learned table added to the residual stream after the embedding.  In both
# precisions: under bfloat16 the two geometries take different builds of the attention kernels and
# different workspaces within one step, and pages that the window has passed go back while the
# matrix-core kernels read the rest.

G_HIDDEN, G_INNER, G_WINDOW, G_POSITIONS = 64, 80, 13, 96


@dataclass(frozen=True)
class LearnedPositionSpec:
    positions: int
    hidden_size: int
    prefix: str = ""
    kind: str = "toy_learned_position"


def _register_geometries():
    from kipp_amd.config import register_architecture
    from kipp_amd.config.specs import (AttentionSpec, EmbeddingSpec, GatedMLPSpec, HeadSpec, LayerRun, LayerSpec, ModelSpec,
                                       RMSNormSpec, RopeSpec)
    from kipp_amd.parts import ParamSpec, register

    @register("position", "toy_learned_position")
    class LearnedPosition:
        """x[t] += table[position of t]: applied by the model once, after the embedding."""

        def __init__(self, spec, runtime):
            self.spec, self.rt = spec, runtime

        @staticmethod
        def params(spec):
            return {"table.weight": ParamSpec((spec.positions, spec.hidden_size))}

        @staticmethod
        def placement(spec):
            return {"table.weight": "float32"}

        def load(self, tensors):
            self.table = tensors["table.weight"]

        def forward(self, x, batch):
            return x + self.table[batch.positions.long()]

    class GeometriesConfig:
        def __init__(self, d):
            self.d = d

        def to_dict(self):
            return dict(self.d)

        def model_spec(self):
            def layer(i, attn):
                p = f"layers.{i}."
                return LayerSpec(block="pre_norm", parts=(
                    ("mixer_norm", RMSNormSpec(G_HIDDEN, EPS, p + "n1.")), ("mixer", attn),
                    ("ffn_norm", RMSNormSpec(G_HIDDEN, EPS, p + "n2.")), ("ffn", GatedMLPSpec(G_HIDDEN, G_INNER, prefix=p + "mlp."))))
            wide = AttentionSpec(G_HIDDEN, 4, 2, 32, position=RopeSpec(32, THETA, pairing="interleaved"), qk_norm_eps=EPS,
                                 prefix="layers.0.attn.")
            narrow = AttentionSpec(G_HIDDEN, 6, 1, 16, position=RopeSpec(16, 50.0, rotary_dim=8), qk_norm_eps=None,
                                   window=G_WINDOW, prefix="layers.1.attn.", page_size=self.d.get("narrow_page"))
            return ModelSpec("ToyGeometriesForTests", G_HIDDEN, VOCAB, G_POSITIONS, EmbeddingSpec(VOCAB, G_HIDDEN, "embed."),
                             (layer(0, wide), layer(1, narrow)), (LayerRun(0), LayerRun(1)), RMSNormSpec(G_HIDDEN, EPS, "norm."),
                             HeadSpec(VOCAB, G_HIDDEN, False, "head."),
                             input_position=LearnedPositionSpec(G_POSITIONS, G_HIDDEN, "positions."))

    register_architecture("ToyGeometriesForTests", GeometriesConfig)


def _rotate(states, n_heads, d, rotary, pos, theta, interleaved):
    """Rotation over the first `rotary` dims of every head; pair i is (i, i + rotary/2) or (2i, 2i + 1)."""
    t = states.shape[0]
    heads = np.array(states, dtype=np.float64).reshape(t, n_heads, d)
    half = rotary // 2
    freq = np.power(np.float64(theta), -(2.0 * np.arange(half)) / rotary).astype(np.float32)
    angle = (np.asarray(pos, dtype=np.float32)[:, None] * freq[None, :]).astype(np.float64)
    cos, sin = np.cos(angle)[:, None, :], np.sin(angle)[:, None, :]
    first = np.arange(half) * 2 if interleaved else np.arange(half)
    second = first + 1 if interleaved else first + half
    a, b = heads[..., first].copy(), heads[..., second].copy()
    heads[..., first] = a * cos - b * sin
    heads[..., second] = b * cos + a * sin
    return heads.reshape(t, n_heads * d)


def _plain_geometries(w, tokens):
    pos = np.arange(len(tokens))
    x = plain.embed(w["embed.weight"], tokens) + w["positions.table.weight"][pos]
    for i, (n_q, n_kv, d, rotary, theta, interleaved, window) in enumerate([(4, 2, 32, 32, THETA, True, None),
                                                                           (6, 1, 16, 8, 50.0, False, G_WINDOW)]):
        p = f"layers.{i}."
        n = plain.rms_norm(x, w[p + "n1.weight"], EPS)
        q, k = plain.linear(n, w[p + "attn.q_proj.weight"]), plain.linear(n, w[p + "attn.k_proj.weight"])
        if i == 0:
            q = plain.head_norm(q, n_q, d, w[p + "attn.q_norm.weight"], EPS)
            k = plain.head_norm(k, n_kv, d, w[p + "attn.k_norm.weight"], EPS)
        q, k = _rotate(q, n_q, d, rotary, pos, theta, interleaved), _rotate(k, n_kv, d, rotary, pos, theta, interleaved)
        v = plain.linear(n, w[p + "attn.v_proj.weight"])
        x = x + plain.linear(plain.causal_gqa(q, k, v, n_q, n_kv, d, window=window), w[p + "attn.o_proj.weight"])
        n = plain.rms_norm(x, w[p + "n2.weight"], EPS)
        x = x + plain.swiglu_mlp(n, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    return plain.linear(plain.rms_norm(x, w["norm.weight"], EPS), w["head.weight"])


def test_the_rotation_of_this_file_is_the_plain_one_where_they_meet():
    rng = np.random.default_rng(0)
    x = rng.normal(size=(5, 3 * 16))
    assert np.allclose(_rotate(x, 3, 16, 16, np.arange(5), 100.0, False), plain.rope(x, 3, 16, np.arange(5), 100.0), rtol=1e-12)
    # interleaved pairing is the half pairing of the head with its dims reordered (evens first, then odds)
    order = np.concatenate([np.arange(0, 16, 2), np.arange(1, 16, 2)])
    xh = x.reshape(5, 3, 16)
    ref = plain.rope(xh[..., order].reshape(5, 48), 3, 16, np.arange(5), 100.0).reshape(5, 3, 16)
    got = _rotate(x, 3, 16, 16, np.arange(5), 100.0, True).reshape(5, 3, 16)
    assert np.allclose(got[..., order], ref, rtol=1e-12)
    # a rotation over 8 of 16 dims leaves the other 8 alone
    part = _rotate(x, 3, 16, 8, np.arange(5), 100.0, False).reshape(5, 3, 16)
    assert np.array_equal(part[..., 8:], xh[..., 8:]) and not np.allclose(part[1:, :, :8], xh[1:, :, :8])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cut", ["whole", "tail", "portions", "mixed"])
def test_two_attention_geometries_a_window_and_a_learned_position(tmp_path, dtype, cut):
    from kipp_amd.config import unregister_architecture
    from kipp_amd.engine import Engine
    from kipp_amd.parts import unregister
    from kipp_amd.weights import write_random_model
    _register_geometries()
    try:
        folder = write_random_model(str(tmp_path / "geometries"), {"architectures": ["ToyGeometriesForTests"]}, seed=14, dtype=dtype)
        _, weights = plain.load_folder(folder)
        requests = {f"g{i}": H.random_tokens(60 + i, n, VOCAB) for i, n in enumerate([9, 70, 41, 90, 33])}
        steps = {"whole": H.whole, "tail": H.tail_one_by_one, "portions": H.changing_portions,
                 "mixed": lambda r: H.mixed(r, seed=7)}[cut](requests)
        engine = Engine.from_folder(folder, dtype=dtype, page_size=8, num_pages=H.peak_pages(requests, steps, 8), max_requests=4)
        cache = engine.cache
        assert len(cache.groups) == 2 and not cache.share                   # a window: no shared beginnings
        assert engine.graphs is None or not engine.graphs.possible          # the learned position declares nothing: eager steps
        got = H.replay(engine, requests, steps)
        tol = H.NMSE_F32 if dtype == "float32" else H.NMSE_BF16["tiny"]
        for rid, toks in requests.items():
            H.assert_close(got[rid], _plain_geometries(weights, toks), tol, f"geometries/{dtype}/{cut}/{rid}")
        assert cache.free_pages() == [g.pool.num_pages for g in cache.groups]
        if dtype == "bfloat16":
            assert engine.rt.generic_attention_launches == 0                # both geometries ran on the matrix-core kernels
    finally:
        unregister_architecture("ToyGeometriesForTests")
        unregister("position", "toy_learned_position")


def _peak_window_pages(requests, steps, page, window):
    """Most pages a group with `window` holds over `steps`: a step claims a page for every new block first (a portion's
    early rows still see keys that its late rows have left behind) and gives back, afterwards, the pages that lie wholly
    behind the window of the next query."""
    length, blocks, held = {}, {}, {}
    peak = 0
    for entries, ends in steps:
        for rid, n in entries:
            length[rid] = length.get(rid, 0) + n
            new_blocks = -(-length[rid] // page)
            held.setdefault(rid, set()).update(range(blocks.get(rid, 0), new_blocks))
            blocks[rid] = new_blocks
        peak = max(peak, sum(len(h) for h in held.values()))
        for rid, _ in entries:
            first_needed = max(0, length[rid] - window + 1)
            held[rid] = {b for b in held[rid] if (b + 1) * page > first_needed}
        for rid in ends:
            del length[rid], blocks[rid], held[rid]
    return peak


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cut", ["tail", "mixed"])
def test_cache_groups_with_page_sizes_and_pools_of_their_own(tmp_path, dtype, cut):
    """The same two-geometry model, the windowed layer asking for pages of 4 tokens where the engine's are 8, and the
    two pools sized apart: the full-attention group for the contexts of the live requests, the windowed one for
    their windows only (fewer tokens than the contexts hold).  Block tables, claims and returns go by each group's
    own page size, in a step that launches both geometries."""
    from kipp_amd.config import unregister_architecture
    from kipp_amd.engine import Engine
    from kipp_amd.parts import unregister
    from kipp_amd.weights import write_random_model
    _register_geometries()
    try:
        folder = write_random_model(str(tmp_path / "geometries"), {"architectures": ["ToyGeometriesForTests"], "narrow_page": 4},
                                    seed=15, dtype=dtype)
        _, weights = plain.load_folder(folder)
        requests = {f"g{i}": H.random_tokens(80 + i, n, VOCAB) for i, n in enumerate([9, 70, 41, 90, 33])}
        steps = {"tail": H.tail_one_by_one, "mixed": lambda r: H.mixed(r, seed=8)}[cut](requests)
        full, windowed = H.peak_pages(requests, steps, 8), _peak_window_pages(requests, steps, 4, G_WINDOW)
        assert windowed * 4 < full * 8                                      # the windowed pool holds fewer tokens
        engine = Engine.from_folder(folder, dtype=dtype, page_size=8, num_pages=[full, windowed], max_requests=4)
        cache = engine.cache
        assert [(g.page_size, g.pool.num_pages) for g in cache.groups] == [(8, full), (4, windowed)]
        got = H.replay(engine, requests, steps)
        tol = H.NMSE_F32 if dtype == "float32" else H.NMSE_BF16["tiny"]
        for rid, toks in requests.items():
            H.assert_close(got[rid], _plain_geometries(weights, toks), tol, f"two pools/{dtype}/{cut}/{rid}")
        assert cache.free_pages() == [full, windowed]
    finally:
        unregister_architecture("ToyGeometriesForTests")
        unregister("position", "toy_learned_position")
