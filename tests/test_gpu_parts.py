"""Each part of a layer alone, built from its spec with random weights, against
the plain implementation; then prefix adoption and the step's error paths."""

import numpy as np
import pytest
import torch

from tests import helpers as H
from tests.plain import qwen3_plain as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _runtime(dtype):
    from kipp_amd.runtime import Runtime
    return Runtime(dtype, DEV)


def _weights(cls, spec, seed, dtype):
    from kipp_amd.weights.random_init import random_tensor
    return {name: random_tensor(seed, name, p, dtype) for name, p in cls.params(spec).items()}


def _load(part, cls, spec, tensors, rt):
    forced = getattr(cls, "placement", lambda s: {})(spec)
    part.load({n: rt.place(t, "float", torch.float32 if forced.get(n) == "float32" else None) for n, t in tensors.items()})


def _batch(rt, seq_lens, q_lens, page, n_groups=1):
    """A StepBatch for sequences that hold seq_lens tokens after this step, of
    which the last q_lens are this step's; pages scrambled."""
    from kipp_amd.cache.manager import RequestCache
    from kipp_amd.engine.batch import StepEntry, build_batch
    rng = np.random.default_rng(1)
    blocks = [-(-n // page) for n in seq_lens]
    perm = rng.permutation(sum(blocks) + 2).tolist()
    reqs, entries, at = [], [], 0
    for i, (n, ql) in enumerate(zip(seq_lens, q_lens)):
        pages = perm[at:at + blocks[i]]
        at += blocks[i]
        reqs.append(RequestCache(i, slot=i, length=n - ql, tables=[list(pages) for _ in range(n_groups)]))
        entries.append(StepEntry(i, [0] * ql, list(range(ql))))
    return build_batch(entries, reqs, n_groups, rt.device), sum(blocks) + 2


@pytest.mark.parametrize("dtype,tol", [("float32", 1e-11), ("bfloat16", 2e-5)])
def test_rms_norm_part(dtype, tol):
    from kipp_amd.config.specs import RMSNormSpec
    from kipp_amd.parts import part_class
    rt = _runtime(dtype)
    spec = RMSNormSpec(width=72, eps=3e-5, prefix="n.")
    cls = part_class("norm", spec.kind)
    part = cls(spec, rt)
    w = _weights(cls, spec, 1, torch.float32)
    _load(part, cls, spec, w, rt)
    x = torch.randn(5, 72)
    got = part.forward(x.to(DEV), rt.act_dtype)
    assert got.dtype == rt.act_dtype
    assert plain.nmse(got.float().cpu().numpy(), plain.rms_norm(x.numpy(), w["weight"].numpy(), 3e-5)) < tol
    delta = torch.randn(5, 72)
    xd = x.to(DEV)
    got = part.add_forward(xd, delta.to(DEV), rt.act_dtype)
    assert torch.equal(xd.cpu(), x + delta)
    assert plain.nmse(got.float().cpu().numpy(), plain.rms_norm((x + delta).numpy(), w["weight"].numpy(), 3e-5)) < tol


def test_rope_part_table():
    from kipp_amd.config.specs import RopeSpec
    from kipp_amd.parts import build_part
    rope = build_part("position", RopeSpec(head_dim=48, theta=5e4, rotary_dim=32), _runtime("float32"))
    inv_freq, rotary = rope.rotary_table()
    assert rotary == 32 and inv_freq.dtype == torch.float32
    want = np.power(np.float64(5e4), -(2.0 * np.arange(16)) / 32).astype(np.float32)
    assert np.array_equal(inv_freq.cpu().numpy(), want)
    none = build_part("position", __import__("kipp_amd.config.specs", fromlist=["x"]).NoPositionSpec(), _runtime("float32"))
    assert none.rotary_table() == (None, 0)


@pytest.mark.parametrize("dtype,tol", [("float32", 1e-10), ("bfloat16", 3e-4)])
@pytest.mark.parametrize("n_q,n_kv,d,hidden,window", [(4, 2, 16, 64, None), (6, 2, 48, 72, 13), (4, 1, 32, 80, None)])
def test_attention_part(dtype, tol, n_q, n_kv, d, hidden, window):
    """A mixed step (two portions and two single tokens) on top of an earlier step."""
    from kipp_amd.cache.manager import KVCacheView
    from kipp_amd.config.specs import AttentionSpec, RopeSpec
    from kipp_amd.parts import part_class
    rt = _runtime(dtype)
    spec = AttentionSpec(hidden, n_q, n_kv, d, position=RopeSpec(d, 1e4), qk_norm_eps=1e-5, window=window, prefix="a.")
    cls = part_class("mixer", spec.kind)
    part = cls(spec, rt)
    wdt = torch.float32 if dtype == "float32" else torch.bfloat16
    w = _weights(cls, spec, 2, wdt)
    _load(part, cls, spec, w, rt)
    assert part.cache_need().window == window and part.state_need() is None
    page = 8
    seq_lens, first, second = [40, 21, 9, 30], [33, 20, 8, 2], [7, 1, 1, 28]
    rng = np.random.default_rng(3)
    xs = [torch.tensor(rng.normal(size=(n, hidden)), dtype=torch.float32) for n in seq_lens]
    _, n_pages = _batch(rt, seq_lens, second, page)
    view = KVCacheView(0, torch.zeros(n_pages, n_kv, page, d, dtype=rt.cache_dtype, device=DEV),
                       torch.zeros(n_pages, n_kv, page, d, dtype=rt.cache_dtype, device=DEV), page)
    # the two steps use the same pages: build both batches from one permutation
    b1, _ = _batch(rt, first, first, page)
    b2, _ = _batch(rt, seq_lens, second, page)
    x1 = torch.cat([x[:n] for x, n in zip(xs, first)]).to(DEV).to(rt.act_dtype)
    x2 = torch.cat([x[n:] for x, n in zip(xs, first)]).to(DEV).to(rt.act_dtype)
    # step 1 writes the first tokens of every sequence into the pages step 2 will read
    b1.block_tables = {0: b2.block_tables[0]}
    part.forward(x1, b1, view)
    got = rt.settle(part.forward(x2, b2, view)).float().cpu().numpy()
    wd = {k: v.double().numpy() for k, v in w.items()}
    at = 0
    for x, n0, n1 in zip(xs, first, second):
        xr = x.to(rt.act_dtype).double().numpy()
        pos = np.arange(n0 + n1)
        q = plain.rope(plain.head_norm(plain.linear(xr, wd["q_proj.weight"]), n_q, d, wd["q_norm.weight"], 1e-5), n_q, d, pos, 1e4)
        k = plain.rope(plain.head_norm(plain.linear(xr, wd["k_proj.weight"]), n_kv, d, wd["k_norm.weight"], 1e-5), n_kv, d, pos, 1e4)
        v = plain.linear(xr, wd["v_proj.weight"])
        ref = plain.linear(plain.causal_gqa(q, k, v, n_q, n_kv, d, window=window), wd["o_proj.weight"])[n0:]
        assert plain.nmse(got[at:at + n1], ref) < tol
        at += n1


@pytest.mark.parametrize("dtype,tol", [("float32", 1e-11), ("bfloat16", 1e-4)])
@pytest.mark.parametrize("rows", [1, 9, 40, 130])
def test_gated_mlp_part(dtype, tol, rows):
    from kipp_amd.config.specs import GatedMLPSpec
    from kipp_amd.parts import part_class
    rt = _runtime(dtype)
    spec = GatedMLPSpec(hidden_size=80, intermediate_size=200, prefix="m.")
    cls = part_class("feed_forward", spec.kind)
    part = cls(spec, rt)
    wdt = torch.float32 if dtype == "float32" else torch.bfloat16
    w = _weights(cls, spec, 4, wdt)
    _load(part, cls, spec, w, rt)
    x = torch.randn(rows, 80).to(rt.act_dtype)
    got = rt.settle(part.forward(x.to(DEV)))        # few rows: the last product comes back not yet launched
    got = got.sum(dim=0) if got.dim() == 3 else got
    wd = {k: v.double().numpy() for k, v in w.items()}
    ref = plain.swiglu_mlp(x.double().numpy(), wd["gate_proj.weight"], wd["up_proj.weight"], wd["down_proj.weight"])
    assert plain.nmse(got.float().cpu().numpy(), ref) < tol


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_embedding_and_head_parts(dtype):
    from kipp_amd.config.specs import EmbeddingSpec, HeadSpec
    from kipp_amd.parts import part_class
    rt = _runtime(dtype)
    espec = EmbeddingSpec(vocab_size=301, hidden_size=40)
    ecls = part_class("embedding", espec.kind)
    emb = ecls(espec, rt)
    wdt = torch.float32 if dtype == "float32" else torch.bfloat16
    ew = _weights(ecls, espec, 5, wdt)
    _load(emb, ecls, espec, ew, rt)
    toks = torch.tensor([0, 300, 17, 17], dtype=torch.int32, device=DEV)
    assert torch.equal(emb.forward(toks).cpu(), ew["weight"].float()[[0, 300, 17, 17]])
    x = torch.randn(3, 40).to(rt.act_dtype)
    for tied in (True, False):
        hspec = HeadSpec(301, 40, tied)
        hcls = part_class("head", hspec.kind)
        head = hcls(hspec, rt)
        hw = _weights(hcls, hspec, 6, wdt)
        assert (len(hw) == 0) == tied
        head.load({n: rt.place(t) for n, t in hw.items()}, embedding=emb)
        ref = x.double().numpy() @ (ew["weight"] if tied else hw["weight"]).double().numpy().T
        assert plain.nmse(head.forward(x.to(DEV)).cpu().numpy(), ref) < (1e-11 if dtype == "float32" else 1e-10)


@pytest.mark.parametrize("dtype,tol", [("float32", H.NMSE_F32), ("bfloat16", H.NMSE_BF16["tiny"])])
def test_a_known_beginning_is_adopted_and_changes_nothing(model_folders, tiny_configs, dtype, tol):
    """Request b starts like the finished request a: its first pages are taken
    from the index, only the rest is run, and the logits are those of a cold run."""
    from kipp_amd.engine import Engine, StepEntry
    folder = model_folders[("b", dtype)]
    engine = Engine.from_folder(folder, dtype=dtype, page_size=8, num_pages=40, share_prefixes=True)
    a = H.random_tokens(1, 45, 509)
    b = a[:29] + H.random_tokens(2, 20, 509)
    engine.step([StepEntry("a", a, [])])
    engine.close("a")
    rb = engine.open("b", b)
    assert rb.length == 24 and rb.adopted == [3]            # three full pages of eight
    got = engine.step([StepEntry("b", b[24:], list(range(len(b) - 24)))]).float().cpu().numpy()
    H.assert_close(got, H.plain_logits(folder, b)[24:], tol, f"adopted prefix {dtype}")
    stats = engine.cache.groups[0].pool.stats()
    assert stats.reused_pages_total == 3
    engine.close("b")
    engine.cache.check()
    assert engine.cache.free_pages() == [40]


def test_step_refuses_bad_input_and_changes_nothing(model_folders):
    from kipp_amd.cache import OutOfPages
    from kipp_amd.engine import Engine, StepEntry
    engine = Engine.from_folder(model_folders[("a", "float32")], dtype="float32", page_size=16, num_pages=3)
    engine.step([StepEntry("x", [1, 2, 3], [2])])
    with pytest.raises(ValueError, match="vocabulary"):
        engine.step([StepEntry("x", [256], [0])])
    with pytest.raises(ValueError, match="twice"):
        engine.step([StepEntry("x", [1], [0]), StepEntry("x", [2], [0])])
    with pytest.raises(ValueError, match="wanted place"):
        engine.step([StepEntry("x", [1], [1])])
    with pytest.raises(OutOfPages):
        engine.step([StepEntry("x", [1], [0]), StepEntry("y", list(range(40)), [])])
    assert engine.length("x") == 3 and "y" not in engine.cache.requests and engine.cache.free_pages() == [2]
    with pytest.raises(ValueError, match="positions"):
        engine.step([StepEntry("x", [1] * 126, [])])
    engine.cache.check()
    ok = engine.step([StepEntry("x", [4], [0])])
    assert ok.shape == (1, 256)
