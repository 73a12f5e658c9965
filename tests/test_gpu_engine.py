"""The engine against the plain implementation: whole sequences, decoding one
by one, portions of changing size and mixed batches with few pages, in float32
and in bfloat16, for both tiny configurations."""
import numpy as np
import pytest

from tests import helpers as H

pytestmark = pytest.mark.gpu

PAGE = {"a": 16, "b": 8}
LENGTHS = {"a": [1, 17, 40, 64], "b": [7, 33, 61, 100]}


def _engine(model_folders, key, dtype, num_pages=None, max_tokens=512, **kw):
    from kipp_amd.engine import Engine
    return Engine.from_folder(model_folders[(key, dtype)], dtype=dtype, page_size=PAGE[key],
                              num_pages=num_pages, max_tokens=None if num_pages else max_tokens, **kw)


def _requests(key, cfg, seed=0):
    return {f"r{i}": H.random_tokens(seed * 100 + i, n, cfg["vocab_size"]) for i, n in enumerate(LENGTHS[key])}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("key", ["a", "b"])
@pytest.mark.parametrize("cut", ["whole", "tail", "portions", "mixed"])
def test_cuttings_match_plain(model_folders, tiny_configs, key, dtype, cut):
    cfg = tiny_configs[key]
    requests = _requests(key, cfg)
    tol = H.NMSE_F32 if dtype == "float32" else H.NMSE_BF16["tiny"]
    if cut == "mixed":
        more = {f"s{i}": H.random_tokens(900 + i, n, cfg["vocab_size"]) for i, n in enumerate(LENGTHS[key])}
        requests = {**requests, **more}
        steps = H.mixed(requests, seed=5)
        # exactly as many pages as the live requests hold at the peak: freed pages are used again
        pages = H.peak_pages(requests, steps, PAGE[key])
        assert pages < sum(-(-len(t) // PAGE[key]) for t in requests.values())
        engine = _engine(model_folders, key, dtype, num_pages=pages, share_prefixes=False)
    else:
        engine = _engine(model_folders, key, dtype, share_prefixes=False)
        steps = {"whole": H.whole, "tail": H.tail_one_by_one, "portions": H.changing_portions}[cut](requests)
    got = H.replay(engine, requests, steps)
    for rid, toks in requests.items():
        ref = H.plain_logits(model_folders[(key, dtype)], toks)
        H.assert_close(got[rid], ref, tol, f"{key}/{dtype}/{cut}/{rid}")
    assert engine.cache.free_pages() == [g.pool.num_pages for g in engine.cache.groups]


@pytest.mark.parametrize("key", ["a", "b"])
def test_float32_cuttings_are_bitwise_equal(model_folders, tiny_configs, key):
    """In float32 every reduction runs in an order fixed by the token's own
    position, so the logits do not depend on the cutting at all."""
    cfg = tiny_configs[key]
    requests = _requests(key, cfg, seed=3)
    base = H.replay(_engine(model_folders, key, "float32", share_prefixes=False), requests, H.whole(requests))
    for maker in (H.tail_one_by_one, H.changing_portions, lambda r: H.mixed(r, seed=11)):
        got = H.replay(_engine(model_folders, key, "float32", share_prefixes=False), requests, maker(requests))
        for rid in requests:
            assert np.array_equal(got[rid], base[rid]), f"{key}/{rid}: bits differ between cuttings"


@pytest.mark.parametrize("key", ["a", "b"])
def test_without_the_streaming_layout(model_folders, tiny_configs, key):
    """`Runtime(stream_layout=False)` keeps every weight once, as rows: the same kernels read the
    weights from there (decoding one by one and in a mixed batch), against the plain implementation."""
    from kipp_amd.engine import Engine
    from kipp_amd.engine.model import load_model
    from kipp_amd.runtime import Runtime
    cfg = tiny_configs[key]
    requests = _requests(key, cfg, seed=2)
    folder = model_folders[(key, "bfloat16")]
    for maker in (H.tail_one_by_one, lambda r: H.mixed(r, seed=9)):
        steps = maker(requests)
        engine = Engine(load_model(folder, Runtime("bfloat16", stream_layout=False)), page_size=PAGE[key], max_tokens=512,
                        share_prefixes=False)
        assert all(block.parts["ffn"].w_gate_up.tiles is None for block in engine.model.blocks)
        got = H.replay(engine, requests, steps)
        for rid, toks in requests.items():
            H.assert_close(got[rid], H.plain_logits(folder, toks), H.NMSE_BF16["tiny"], f"{key}/rows only/{rid}")


@pytest.mark.parametrize("key", ["a", "b"])
def test_norms_in_kernels_of_their_own(model_folders, tiny_configs, key):
    """With few rows the residual add and the norm ride on the products around them; `fuse_norms =
    False` gives every norm its own kernel again.  Both against the plain implementation, and the
    fused engine launches fewer kernels' worth of norms: it never calls the norm kernel with a delta."""
    from kipp_amd.engine import Engine
    from kipp_amd.engine.model import load_model
    from kipp_amd.runtime import Runtime
    cfg = tiny_configs[key]
    requests = _requests(key, cfg, seed=4)
    folder = model_folders[(key, "bfloat16")]
    steps = H.tail_one_by_one(requests)
    for fuse in (False, True):
        rt = Runtime("bfloat16")
        rt.fuse_norms = fuse
        calls = {"delta": 0, "plain": 0}
        inner = rt.ops.rmsnorm

        class Counting:
            def __getattr__(self, name, ops=rt.ops):
                return getattr(ops, name)

            @staticmethod
            def rmsnorm(x, weight, eps, out, delta=None):
                calls["delta" if delta is not None and x.shape[0] <= 8 else "plain"] += 1
                return inner(x, weight, eps, out, delta=delta)
        rt.ops = Counting()
        engine = Engine(load_model(folder, rt), page_size=PAGE[key], max_tokens=512, share_prefixes=False, use_graphs=False)
        got = H.replay(engine, requests, steps)
        for rid, toks in requests.items():
            H.assert_close(got[rid], H.plain_logits(folder, toks), H.NMSE_BF16["tiny"], f"{key}/fused norms {fuse}/{rid}")
        assert (calls["delta"] == 0) == fuse, calls


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_head_size_that_is_no_multiple_of_16(tmp_path, tiny_configs, dtype):
    """Head size 24 (q width 96 beside a hidden width of 80): the float32 path takes any head size up to 256, and
    under bfloat16 the mixer sends such a geometry to the generic attention kernel, which is counted, instead
    of the configuration refusing it.  Portions, single tokens and a mixed batch against the plain implementation."""
    from kipp_amd.engine import Engine
    from kipp_amd.weights import write_random_model
    cfg = dict(tiny_configs["b"], head_dim=24, num_attention_heads=4, num_key_value_heads=2)
    folder = write_random_model(str(tmp_path / "d24"), cfg, seed=77, dtype=dtype)
    requests = {f"r{i}": H.random_tokens(40 + i, n, cfg["vocab_size"]) for i, n in enumerate([9, 33, 50])}
    for maker in (H.tail_one_by_one, H.changing_portions, lambda r: H.mixed(r, seed=3)):
        engine = Engine.from_folder(folder, dtype=dtype, page_size=8, max_tokens=512, share_prefixes=False)
        got = H.replay(engine, requests, maker(requests))
        for rid, toks in requests.items():
            H.assert_close(got[rid], H.plain_logits(folder, toks), H.NMSE_F32 if dtype == "float32" else H.NMSE_BF16["tiny"],
                           f"head size 24/{dtype}/{rid}")
        assert (engine.rt.generic_attention_launches > 0) == (dtype == "bfloat16")
