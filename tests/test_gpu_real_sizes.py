"""The layer sizes of the benchmark shape (Qwen3-4B: hidden 2560, 32 query and 8
key/value heads of 128, SwiGLU 9728, vocabulary 151936, tied), with two layers
so that the plain implementation stays affordable: the kernels run at the
sizes they are measured at, against the same plain reference."""
import numpy as np
import pytest
import torch

from tests import helpers as H
from tests.plain import qwen3_plain as plain

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def real_folder(tmp_path_factory):
    from kipp_amd.config import shape_config
    from kipp_amd.weights import write_random_model
    cfg = shape_config("qwen3-4b")
    cfg["num_hidden_layers"] = 2
    folder = str(tmp_path_factory.mktemp("real") / "qwen3-4b-2layers")
    write_random_model(folder, cfg, seed=21, dtype="bfloat16")
    return folder


@pytest.fixture(scope="module")
def real_reference(real_folder):
    cfg, weights = plain.load_folder(real_folder)
    requests = {"p": H.random_tokens(1, 150, 151936), "q": H.random_tokens(2, 37, 151936), "r": H.random_tokens(3, 70, 151936)}
    refs = {}
    for rid, toks in requests.items():
        refs[rid] = plain.forward_whole(cfg, weights, toks)
    return requests, refs


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_benchmark_layer_sizes_match_plain(real_folder, real_reference, dtype):
    from kipp_amd.engine import Engine
    requests, refs = real_reference
    tol = H.NMSE_F32 if dtype == "float32" else H.NMSE_BF16["real"]
    _cuttings_against_plain(real_folder, requests, refs, dtype, tol, "4B sizes")


CUTTINGS = (("whole", H.whole), ("tail", lambda r: H.tail_one_by_one(r, 20)), ("portions", H.changing_portions),
            ("mixed", lambda r: H.mixed(r, seed=4)))


def _cuttings_against_plain(folder, requests, refs, dtype, tol, what):
    """Whole prompts, the last 20 tokens one by one, portions of changing size down to two tokens, and a mixed batch
    with as many pages as the live requests hold at their peak."""
    from kipp_amd.engine import Engine
    for cut, maker in CUTTINGS:
        steps = maker(requests)
        engine = Engine.from_folder(folder, dtype=dtype, page_size=16, num_pages=H.peak_pages(requests, steps, 16),
                                    max_requests=4, share_prefixes=False)
        got = H.replay(engine, requests, steps)
        for rid in requests:
            H.assert_close(got[rid], refs[rid], tol, f"{what}/{dtype}/{cut}/{rid}")
            if dtype == "float32":
                assert np.array_equal(got[rid].argmax(axis=1), refs[rid].argmax(axis=1))
        if dtype == "bfloat16":
            assert engine.rt.generic_attention_launches == 0 and engine.rt.library_products == 0
        del engine


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_benchmark_layer_sizes_through_the_c_host(real_folder, real_reference, dtype):
    """The same four cuttings through kipp_step of the C host at the 4B layer sizes, against the same plain rows."""
    from kipp_amd.chost import CModel
    requests, refs = real_reference
    tol = H.NMSE_F32 if dtype == "float32" else H.NMSE_BF16["real"]
    for cut, maker in CUTTINGS:
        steps = maker(requests)
        with CModel(real_folder, path={"float32": "gpu-fp32", "bfloat16": "gpu-bf16"}[dtype], page_tokens=16,
                    kv_pool_pages=H.peak_pages(requests, steps, 16), max_sessions=4, share_prefixes=False) as model:
            got = H.replay_c(model, requests, steps, scramble_every=5 if cut == "mixed" else 0)
            for rid in requests:
                H.assert_close(got[rid], refs[rid], tol, f"C host, 4B sizes/{dtype}/{cut}/{rid}")
    # the three prompts in one step: 257 rows, which go to the products built for hundreds of rows (the activation as their end)
    together = [([(rid, len(toks)) for rid, toks in requests.items()], list(requests))]
    with CModel(real_folder, path={"float32": "gpu-fp32", "bfloat16": "gpu-bf16"}[dtype], page_tokens=16,
                kv_pool_pages=H.peak_pages(requests, together, 16), max_sessions=4, share_prefixes=False) as model:
        got = H.replay_c(model, requests, together)
        for rid in requests:
            H.assert_close(got[rid], refs[rid], tol, f"C host, 4B sizes/{dtype}/together/{rid}")


# The layer sizes of the two larger shapes that the serving workloads run (Qwen3-8B: hidden 4096, SwiGLU 12288, 32 query
# heads; Qwen3-32B: hidden 5120, SwiGLU 25600, 64 query heads, eight to a key/value head; both with a head of its own),
# two layers each and a small vocabulary that is no power of two, so that the plain implementation stays affordable.
LARGER = {"qwen3-8b": {"p": 150, "q": 37, "r": 70}, "qwen3-32b": {"p": 100, "q": 37, "r": 50}}


@pytest.fixture(scope="module", params=sorted(LARGER))
def larger_shape(request, tmp_path_factory):
    from kipp_amd.config import shape_config
    from kipp_amd.weights import write_random_model
    shape = request.param
    cfg = shape_config(shape)
    cfg.update(num_hidden_layers=2, vocab_size=2053)
    folder = str(tmp_path_factory.mktemp("larger") / f"{shape}-2layers")
    write_random_model(folder, cfg, seed=23, dtype="bfloat16")
    plain_cfg, weights = plain.load_folder(folder)
    requests = {rid: H.random_tokens(40 + i, n, 2053) for i, (rid, n) in enumerate(LARGER[shape].items())}
    refs = {rid: plain.forward_whole(plain_cfg, weights, toks) for rid, toks in requests.items()}
    del weights
    return shape, folder, requests, refs


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_larger_shapes_layer_sizes_match_plain(larger_shape, dtype):
    """What the serving workloads run at: products of 4,096 and 5,120 columns against up to 51,200 rows, 64 query heads in
    groups of eight, the few-rows products that keep their norm's kernel because every workgroup would read too much of x
    (the 32B sizes), an untied head."""
    shape, folder, requests, refs = larger_shape
    tol = H.NMSE_F32 if dtype == "float32" else H.NMSE_BF16["real"]
    _cuttings_against_plain(folder, requests, refs, dtype, tol, f"{shape} sizes")


@pytest.mark.parametrize("fault", ["read-slot", "other-run"])
def test_the_tolerance_at_these_sizes_notices_a_cache_fault(real_folder, real_reference, fault):
    """The bound for bfloat16 at the benchmark's layer sizes is wider than at the tiny sizes; it still fails a run in which
    every read of the cache lands one slot further, or every layer but the first reads the first layer's cache."""
    from kipp_amd.engine import Engine
    from tests.test_gpu_adversarial import Faulty
    requests, refs = real_reference
    steps = H.tail_one_by_one(requests, 20)
    engine = Engine.from_folder(real_folder, dtype="bfloat16", page_size=16, num_pages=H.peak_pages(requests, steps, 16) + 2,
                                max_requests=4, share_prefixes=False, use_graphs=False)
    faulty = Faulty(engine.rt.ops, fault, engine)
    engine.rt.ops = faulty
    got = H.replay(engine, requests, steps)
    assert faulty.hits > 0
    worst = max(plain.nmse(got[rid][i], refs[rid][i]) for rid in requests for i in range(len(requests[rid])))
    assert worst > 10 * H.NMSE_BF16["real"], f"{fault}: worst NMSE {worst:.2e} is no further from the bound than rounding"
    with pytest.raises(AssertionError):
        for rid in requests:
            H.assert_close(got[rid], refs[rid], H.NMSE_BF16["real"], f"4B sizes/{fault}/{rid}")


def test_split_products_keep_their_norm_kernels(real_folder, real_reference):
    """The residual add rides on a product only where that product need not be split over workgroups or
    reads little of X; with the limit at zero the output and down projections of these sizes (which are
    split) are launched as they are and every norm has its kernel again.  Both ways against the plain
    implementation."""
    from kipp_amd.engine import Engine
    from kipp_amd.engine.model import load_model
    from kipp_amd.runtime import Runtime
    requests, refs = real_reference
    steps = H.tail_one_by_one(requests, 12)
    for limit in (0, None):
        rt = Runtime("bfloat16")
        if limit is not None:
            rt.fuse_norm_x_bytes = limit
        fused = {"yes": 0, "no": 0}
        inner = rt.product_add_norm

        def counting(delta, x, weight, eps):
            out = inner(delta, x, weight, eps)
            fused["no" if out is None else "yes"] += 1
            return out
        rt.product_add_norm = counting
        engine = Engine(load_model(real_folder, rt), page_size=16, max_tokens=512, share_prefixes=False, use_graphs=False)
        got = H.replay(engine, requests, steps)
        for rid in requests:
            H.assert_close(got[rid], refs[rid], H.NMSE_BF16["real"], f"4B sizes/limit {limit}/{rid}")
        assert (fused["yes"] == 0 and fused["no"] > 0) if limit == 0 else (fused["yes"] > 0 and fused["no"] == 0), fused


@pytest.fixture(scope="module")
def long_folder(tmp_path_factory):
    """Head size 128 and a long context on a narrow model: decoding runs through the
    fused attention kernel and the recorded graphs, over many splits of the keys."""
    from kipp_amd.config import shape_config
    from kipp_amd.weights import write_random_model
    cfg = shape_config("tiny-a")
    cfg.update(hidden_size=96, num_attention_heads=4, num_key_value_heads=1, head_dim=128, intermediate_size=160,
               vocab_size=311, num_hidden_layers=2, max_position_embeddings=2304, tie_word_embeddings=False)
    folder = str(tmp_path_factory.mktemp("long") / "narrow-long")
    write_random_model(folder, cfg, seed=5, dtype="bfloat16")
    return folder


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decoding_across_a_graph_bucket_and_many_splits(long_folder, dtype):
    """A prompt of 1,000 tokens in portions, then 60 tokens one by one: the context
    passes 1,024 (another recorded graph) and split edges; two more requests decode
    beside it, one of them ending early so that the batch shrinks; every row against
    the plain implementation."""
    from kipp_amd.engine import Engine, StepEntry
    cfg, weights = plain.load_folder(long_folder)
    seqs = {"long": H.random_tokens(31, 1060, 311), "mid": H.random_tokens(32, 300, 311), "short": H.random_tokens(33, 40, 311)}
    refs = {k: plain.forward_whole(cfg, weights, v) for k, v in seqs.items()}
    tol = H.NMSE_F32 if dtype == "float32" else H.NMSE_BF16["real"]
    engine = Engine.from_folder(long_folder, dtype=dtype, page_size=16, max_tokens=1088 + 320 + 64, max_requests=3,
                                share_prefixes=False)
    fed = {"long": 1000, "mid": 240, "short": 10}
    for rid, n in fed.items():                                  # prompts in portions of 300
        for at in range(0, n, 300):
            engine.step([StepEntry(rid, seqs[rid][at:min(at + 300, n)], [])])
    got = {rid: [] for rid in seqs}
    for _ in range(60):
        live = [rid for rid in seqs if fed[rid] < len(seqs[rid])]
        logits = engine.step([StepEntry(rid, [seqs[rid][fed[rid]]], [0]) for rid in live]).cpu().numpy()
        for row, rid in zip(logits, live):
            got[rid].append(row)
            fed[rid] += 1
    assert engine.graphs.replays > 40 and len(engine.graphs.graphs) >= 3     # 3 and 2 requests, contexts below and above 1,024
    for rid in seqs:
        first = {"long": 1000, "mid": 240, "short": 10}[rid]
        H.assert_close(np.stack(got[rid]), refs[rid][first:fed[rid]], tol, f"long context/{dtype}/{rid}")


def test_the_splits_merged_by_a_launch_of_its_own(long_folder):
    """`Runtime.merge_in_kernel = False` (KIPP_AMD_DECODE_MERGE=launch) drops the count of finished splits: decode
    attention then merges a head's splits in a launch of its own, which needs no ordering between workgroups.  The same
    sums in the same order: behind 700 and 300 tokens (several splits a head) the same bits as merged by the last
    workgroup, eager and as recorded graphs, and the plain implementation's values."""
    from kipp_amd.engine import Engine, StepEntry
    from kipp_amd.engine.model import load_model
    from kipp_amd.runtime import Runtime
    cfg, weights = plain.load_folder(long_folder)
    seqs = {"long": H.random_tokens(41, 720, 311), "mid": H.random_tokens(42, 320, 311)}
    got = {}
    for merge in (True, False):
        rt = Runtime("bfloat16")
        rt.merge_in_kernel = merge
        engine = Engine(load_model(long_folder, rt), page_size=16, max_tokens=1152, max_requests=2, share_prefixes=False)
        for rid, toks in seqs.items():
            engine.step([StepEntry(rid, toks[:-20], [])])
        rows = []
        for i in range(20, 0, -1):
            rows.append(engine.step([StepEntry(rid, [toks[-i]], [0]) for rid, toks in seqs.items()]).cpu().numpy())
        got[merge] = np.stack(rows)
        spaces = [space for graph in engine.graphs.graphs.values() for name, space in graph.batch.host.items()
                  if isinstance(name, tuple) and name[0] == "decode_workspace"]
        assert engine.graphs.replays >= 10 and spaces and all((len(space) == 3) == merge for space in spaces)
    assert np.array_equal(got[True], got[False])
    for at, (rid, toks) in enumerate(seqs.items()):
        H.assert_close(got[False][:, at], plain.forward_whole(cfg, weights, toks)[-20:], H.NMSE_BF16["real"], f"merge by a launch/{rid}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n_requests", [80, 128, 200])
def test_many_requests_decode_together(long_folder, dtype, n_requests):
    """More rows than one 64-row product takes: prompts of 3 to 40 tokens enter in one step, then all decode
    together for 6 steps (the products stage their rows in chunks of 128 columns, the steps are recorded
    graphs).  From 96 rows on (one key/value head each) decode attention is the kernel in which a
    workgroup walks a whole context, from the projection's output; with 80 the keys are split in the steps
    that run as they are, and the recorded steps, filled up to 96 rows, take the other kernel.  Every
    tenth request against the plain implementation."""
    from kipp_amd.engine import Engine, StepEntry
    cfg, weights = plain.load_folder(long_folder)
    rng = np.random.default_rng(7)
    seqs = {f"r{i}": H.random_tokens(100 + i, int(rng.integers(3, 41)) + 6, 311) for i in range(n_requests)}
    engine = Engine.from_folder(long_folder, dtype=dtype, page_size=16, max_tokens=n_requests * 64, max_requests=n_requests,
                                share_prefixes=False)
    fed = {rid: len(toks) - 6 for rid, toks in seqs.items()}
    engine.step([StepEntry(rid, seqs[rid][:fed[rid]], []) for rid in seqs])
    got = {rid: [] for rid in seqs}
    for _ in range(6):
        logits = engine.step([StepEntry(rid, [seqs[rid][fed[rid]]], [0]) for rid in seqs]).cpu().numpy()
        for row, rid in zip(logits, seqs):
            got[rid].append(row)
            fed[rid] += 1
    assert engine.graphs.replays >= 4
    from kipp_amd.csrc import ops
    assert ops.attention_decode_streams(n_requests, 1, 128, 4, 16, 64) == (n_requests >= 96)
    tol = H.NMSE_F32 if dtype == "float32" else H.NMSE_BF16["real"]
    for rid in list(seqs)[::10]:
        ref = plain.forward_whole(cfg, weights, seqs[rid])
        H.assert_close(np.stack(got[rid]), ref[len(seqs[rid]) - 6:], tol, f"{n_requests} together/{dtype}/{rid}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_batch_whose_size_changes_replays_one_graph(long_folder, dtype):
    """17 to 24 requests decode together, another number in every step (the others wait): all those steps
    are one recorded shape of 24 rows, the rows that fill up write to the cache's scratch page; a request
    that joined late and the ones that paused give the logits of the plain implementation."""
    from kipp_amd.engine import Engine, StepEntry
    from kipp_amd.engine.graphs import padded_size
    assert [padded_size(n) for n in (1, 8, 9, 12, 13, 16, 17, 100, 129, 256)] == [1, 8, 9, 12, 13, 16, 24, 128, 192, 256]
    cfg, weights = plain.load_folder(long_folder)
    seqs = {f"r{i}": H.random_tokens(300 + i, 20 + 3 * i + 14, 311) for i in range(24)}
    engine = Engine.from_folder(long_folder, dtype=dtype, page_size=16, max_tokens=24 * 128, max_requests=24, share_prefixes=False)
    fed = {rid: len(toks) - 14 for rid, toks in seqs.items()}
    engine.step([StepEntry(rid, seqs[rid][:fed[rid]], []) for rid in seqs])
    got = {rid: [] for rid in seqs}
    order = list(seqs)
    for step, n in enumerate([24, 19, 21, 17, 24, 20, 18, 23, 24, 17, 22, 24, 19, 24]):
        live = [rid for rid in (order[step % 24:] + order[:step % 24]) if fed[rid] < len(seqs[rid])][:n]
        logits = engine.step([StepEntry(rid, [seqs[rid][fed[rid]]], [0]) for rid in live]).cpu().numpy()
        assert logits.shape[0] == len(live)
        for row, rid in zip(logits, live):
            got[rid].append(row)
            fed[rid] += 1
    assert len(engine.graphs.graphs) == 1 and engine.graphs.replays >= 11
    tol = H.NMSE_F32 if dtype == "float32" else H.NMSE_BF16["real"]
    for rid, toks in seqs.items():
        ref = plain.forward_whole(cfg, weights, toks)
        first = len(toks) - 14
        H.assert_close(np.stack(got[rid]), ref[first:first + len(got[rid])], tol, f"changing batch/{dtype}/{rid}")
    engine.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_many_decoding_rows_beside_prompt_portions(long_folder, dtype):
    """Steps that hold 20 to 34 single tokens AND two or three prompt portions of changing size (2 to 290
    tokens; a few steps pass 192 rows and take the products for many rows), at head size 128: in bfloat16 one
    forward pass then runs the rotary kernel, the prefill attention and the split decode attention side
    by side.  The pool holds exactly what live requests need at the peak, so pages are used again while
    others are still read.  Every row of every request against the plain implementation."""
    from kipp_amd.engine import Engine
    cfg, weights = plain.load_folder(long_folder)
    rng = np.random.default_rng(3)
    requests, tail = {}, {}
    for i in range(70):
        tail[f"r{i}"] = 25 + (i * 7) % 26
        requests[f"r{i}"] = H.random_tokens(700 + i, int(rng.integers(4, 200)) + tail[f"r{i}"], 311)
    steps = H.busy(requests, 1, tail)
    singles = [sum(1 for _, n in entries if n == 1) for entries, _ in steps]
    portions = [sum(1 for _, n in entries if n > 1) for entries, _ in steps]
    assert sum(1 for s, p in zip(singles, portions) if s >= 20 and p >= 2) >= 50 and max(singles) > 32
    assert sum(1 for entries, _ in steps if sum(n for _, n in entries) > 256) >= 2
    pages = H.peak_pages(requests, steps, 16)
    assert pages < 0.6 * sum(-(-len(t) // 16) for t in requests.values())
    engine = Engine.from_folder(long_folder, dtype=dtype, page_size=16, num_pages=pages, max_requests=64, share_prefixes=False)
    got = H.replay(engine, requests, steps)
    tol = H.NMSE_F32 if dtype == "float32" else H.NMSE_BF16["real"]
    for rid, toks in requests.items():
        H.assert_close(got[rid], plain.forward_whole(cfg, weights, toks), tol, f"busy/{dtype}/{rid}")
    assert engine.cache.free_pages() == [pages]


def test_a_long_position_limit_keeps_the_matrix_core_kernels(real_folder, real_reference, tmp_path):
    """A model folder whose config.json allows 40,960 positions (the reference's Qwen3-4B,
    /root/reference/src/kipp_checkpoints.h:31): block tables are as wide as the contexts of a step, not
    as that limit, so short contexts decode on the matrix-core attention kernels under recorded graphs,
    nothing falls to the generic kernel, and the logits match the plain implementation."""
    import json
    import os
    from kipp_amd.engine import Engine
    folder = str(tmp_path / "long-limit")
    os.makedirs(folder)
    with open(os.path.join(real_folder, "config.json")) as f:
        config = json.load(f)
    config["max_position_embeddings"] = 40960
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config, f)
    os.symlink(os.path.join(real_folder, "model.safetensors"), os.path.join(folder, "model.safetensors"))
    requests, refs = real_reference
    requests = {rid: requests[rid] for rid in ("p", "q")}
    steps = H.tail_one_by_one(requests, 20)
    engine = Engine.from_folder(folder, dtype="bfloat16", page_size=16, max_tokens=512, max_requests=4, share_prefixes=False)
    assert engine.cache.max_position == 40960
    got = H.replay(engine, requests, steps)
    for rid in requests:
        H.assert_close(got[rid], refs[rid], H.NMSE_BF16["real"], f"long limit/{rid}")
    assert engine.rt.generic_attention_launches == 0
    assert engine.graphs.replays >= 30
    assert all(max(g.blocks) <= 1024 // 16 for g in engine.graphs.graphs.values())


@pytest.mark.parametrize("ours", [True, False, "auto"])
def test_prompt_portions_of_many_rows_by_either_product(real_folder, real_reference, ours):
    """Portions of 230 and 390 rows (more than the streaming products are best at) at the benchmark's layer
    sizes, with every product of theirs on our matrix-core kernel (SwiGLU in its end, K split into slabs that the norms add; the fastest of the cuts that
    give the planned cut's bits), then on the library's, then left to the clock among all of them (the
    default): against the plain implementation, every row.  Our kernel alone gives the same bits on a second
    engine, whatever its clock chose."""
    from kipp_amd.engine import Engine, StepEntry
    from kipp_amd.engine.model import load_model
    from kipp_amd.runtime import Runtime
    cfg, weights = plain.load_folder(real_folder)
    toks = H.random_tokens(9, 620, 151936)
    ref = plain.forward_whole(cfg, weights, toks)

    def run():
        Runtime._choices_of_process.clear()         # every engine times for itself here
        rt = Runtime("bfloat16")
        rt.own_prompt_products = ours
        engine = Engine(load_model(real_folder, rt), page_size=16, max_tokens=1024, max_requests=2, share_prefixes=False)
        got = [engine.step([StepEntry("a", toks[:230], list(range(230)))]),
               engine.step([StepEntry("a", toks[230:], list(range(390)))])]
        return rt, torch.cat(got).float().cpu().numpy()
    rt, got = run()
    H.assert_close(got, ref, H.NMSE_BF16["real"], f"many rows, ours {ours}")
    choices = set(rt.prompt_product_choices.values())
    assert len(rt.prompt_product_choices) >= 4                  # QKV, output, gate-up, down: each decided
    if ours is True:
        assert rt.tile_products > 0 and rt.library_products == 0 and "library" not in choices
        again = run()[1]
        assert np.array_equal(got, again)
    elif ours is False:
        assert rt.tile_products == 0 and rt.library_products > 0 and choices == {"library"}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_portions_behind_a_long_context_cut_their_keys(long_folder, dtype):
    """A portion of a few hundred rows behind a thousand keys and more is few, long work items for the prefill
    attention: under bfloat16 their keys are cut over more workgroups and merged (the first portion, from an
    empty context, is not cut).  Every row of every portion against the plain implementation."""
    from kipp_amd.engine import Engine, StepEntry
    cfg, weights = plain.load_folder(long_folder)
    toks = H.random_tokens(41, 1500, 311)
    ref = plain.forward_whole(cfg, weights, toks)
    engine = Engine.from_folder(long_folder, dtype=dtype, page_size=16, max_tokens=1536, max_requests=2, share_prefixes=False)
    seen = []
    mixer = engine.model.blocks[0].mixer
    inner = mixer._prefill_work

    def watching(batch):
        work = inner(batch)
        seen.append(work[2] is not None)
        return work
    mixer._prefill_work = watching
    got, at = [], 0
    for n in (700, 300, 130, 370):
        got.append(engine.step([StepEntry("long", toks[at:at + n], list(range(n)))]).float().cpu().numpy())
        at += n
    tol = H.NMSE_F32 if dtype == "float32" else H.NMSE_BF16["real"]
    H.assert_close(np.concatenate(got), ref, tol, f"portions behind a long context/{dtype}")
    if dtype == "bfloat16":
        assert seen == [True, True, True, True]      # 700 keys already exceed a cut of 512; every portion was cut


def test_the_c_host_cuts_the_keys_of_such_portions_too(long_folder):
    """The same portions through the C host: from the second on their keys are cut (700 keys already exceed a cut of
    512) and merged; every row against the plain implementation."""
    from kipp_amd.chost import CModel
    cfg, weights = plain.load_folder(long_folder)
    toks = H.random_tokens(41, 1500, 311)
    ref = plain.forward_whole(cfg, weights, toks)
    with CModel(long_folder, path="gpu-bf16", page_tokens=16, kv_pool_pages=96, max_sessions=2, max_step_tokens=1024,
                share_prefixes=False) as model:
        session = model.session()
        got, at = [], 0
        for n in (700, 300, 130, 370):
            got.append(model.step([(session, toks[at:at + n], list(range(n)))]))
            at += n
        assert model.cut_attention_steps == 4
    H.assert_close(np.concatenate(got), ref, H.NMSE_BF16["real"], "portions behind a long context/C host")


@pytest.mark.parametrize("host", ["python", "c"])
def test_portions_of_several_requests_behind_long_contexts(long_folder, host):
    """Three requests of 1,400, 900 and 620 tokens fed together in portions of 40 to 260 tokens, then one by one: once a
    context passes 512 keys the portions' keys are cut, with a different number of cuts for every request (and for the
    tiles of one portion), beside portions that are not cut and single tokens.  Every row of every request against
    the plain implementation, through either host."""
    cfg, weights = plain.load_folder(long_folder)
    requests = {"x": H.random_tokens(61, 1400, 311), "y": H.random_tokens(62, 900, 311), "z": H.random_tokens(63, 620, 311)}
    steps = H.mixed(requests, seed=9, max_live=3, prefill_portion=(40, 260), decode_tail=6)
    assert sum(1 for entries, _ in steps if sum(1 for _, n in entries if n > 1) >= 2) >= 5
    pages = H.peak_pages(requests, steps, 16) + 2
    if host == "python":
        from kipp_amd.engine import Engine
        engine = Engine.from_folder(long_folder, dtype="bfloat16", page_size=16, num_pages=pages, max_requests=4, share_prefixes=False)
        cut = []
        mixer = engine.model.blocks[0].mixer
        inner = mixer._prefill_work
        mixer._prefill_work = lambda batch: (lambda work: (cut.append(work[2] is not None), work)[1])(inner(batch))
        got = H.replay(engine, requests, steps)
        assert sum(cut) >= 5
    else:
        from kipp_amd.chost import CModel
        with CModel(long_folder, path="gpu-bf16", page_tokens=16, kv_pool_pages=pages, max_sessions=4, max_step_tokens=1024,
                    share_prefixes=False) as model:
            got = H.replay_c(model, requests, steps)
            assert model.cut_attention_steps >= 5
    for rid, toks in requests.items():
        H.assert_close(got[rid], plain.forward_whole(cfg, weights, toks), H.NMSE_BF16["real"], f"portions behind long contexts/{host}/{rid}")


def test_warm_up_decides_before_the_first_request(real_folder, real_reference):
    """`Engine.warm_up` runs portions of the given sizes on a request of its own: the products' cuts for those sizes are
    decided then (not in a request's first step), the pool is as empty as before, nothing was published, and a prompt
    afterwards has the bits it has on an engine that was never warmed up."""
    from kipp_amd.engine import Engine, StepEntry
    requests, _ = real_reference
    toks = requests["p"]
    warm = Engine.from_folder(real_folder, dtype="bfloat16", page_size=16, max_tokens=512, max_requests=2)
    assert not warm.rt.prompt_product_choices
    warm.warm_up((256, 100000))                                   # the second neither fits the pool nor the positions: left out
    assert warm.rt.prompt_product_choices and not warm.cache.requests
    for g in warm.cache.groups:
        assert g.pool.free_count == g.pool.num_pages and all(c is None for c in g.pool.content)
    decided = dict(warm.rt.prompt_product_choices)
    got = warm.step([StepEntry("p", toks, list(range(len(toks))))]).float().cpu()
    cold = Engine.from_folder(real_folder, dtype="bfloat16", page_size=16, max_tokens=512, max_requests=2)
    want = cold.step([StepEntry("p", toks, list(range(len(toks))))]).float().cpu()
    assert torch.equal(got, want)
    assert all(warm.rt.prompt_product_choices[k] == v for k, v in decided.items())
