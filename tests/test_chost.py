"""The C host (`kipp_amd/host`, through `kipp_amd.chost`) on its scalar float32 path, which needs no GPU: the step
function under every cutting against the plain implementation and bit for bit against itself, scrambled block
tables, pages that are used again, shared beginnings, truncation, what happens when pages run out; configuration
and weight errors; the sampler against the Python one."""
import json
import os
import random
import shutil

import numpy as np
import pytest

from kipp_amd.chost import CModel, KippError, Rng, sample
from tests import helpers as H

PAGE = {"a": 16, "b": 8}
LENGTHS = {"a": [1, 17, 40, 64], "b": [7, 33, 61, 100]}


def _requests(key, cfg, seed=0):
    return {f"r{i}": H.random_tokens(seed * 100 + i, n, cfg["vocab_size"]) for i, n in enumerate(LENGTHS[key])}


def _model(model_folders, key, pages=64, **kw):
    return CModel(model_folders[(key, "float32")], path="cpu-fp32", page_tokens=PAGE[key], kv_pool_pages=pages, **kw)


@pytest.mark.parametrize("key", ["a", "b"])
@pytest.mark.parametrize("cut", ["whole", "tail", "portions", "mixed"])
def test_host_path_cuttings_match_plain_and_each_other(model_folders, tiny_configs, key, cut):
    """Every cutting against the plain implementation, and bit for bit against the whole prompts: on the scalar path
    every sum runs in an order that its own row and position fix.  The mixed cutting runs with exactly as many pages as
    the live requests hold at their peak, so pages that were given back are used again, and with every session's block
    tables reversed every third step."""
    cfg = tiny_configs[key]
    requests = _requests(key, cfg)
    with _model(model_folders, key, share_prefixes=False) as model:
        base = H.replay_c(model, requests, H.whole(requests))
    if cut == "mixed":
        more = {f"s{i}": H.random_tokens(900 + i, n, cfg["vocab_size"]) for i, n in enumerate(LENGTHS[key])}
        with _model(model_folders, key, share_prefixes=False) as model:
            base.update(H.replay_c(model, more, H.whole(more)))
        requests = {**requests, **more}
        steps = H.mixed(requests, seed=5)
        pages = H.peak_pages(requests, steps, PAGE[key])
        assert pages < sum(-(-len(t) // PAGE[key]) for t in requests.values())
        model = _model(model_folders, key, pages=pages, share_prefixes=False)
        got = H.replay_c(model, requests, steps, scramble_every=3)
    else:
        steps = {"whole": H.whole, "tail": H.tail_one_by_one, "portions": H.changing_portions}[cut](requests)
        model = _model(model_folders, key, share_prefixes=False)
        got = H.replay_c(model, requests, steps, scramble_every=2 if cut != "whole" else 0)
    for rid, toks in requests.items():
        H.assert_close(got[rid], H.plain_logits(model_folders[(key, "float32")], toks), H.NMSE_F32, f"C host {key}/{cut}/{rid}")
        assert np.array_equal(got[rid], base[rid]), f"{key}/{cut}/{rid}: bits differ from the whole prompt's"
    stats = model.pool_stats()
    assert stats["free_blocks"] == stats["total_blocks"]
    model.close()


def test_a_scrambled_table_is_noticed_when_the_contents_stay(model_folders, tiny_configs):
    """The scramble hook moves the pages' contents along with the table.  If a step read through a table that does
    not match where the keys lie, the logits would change: shown by feeding a sequence, swapping two pages'
    *roles* by hand (evaluating the rest in a second model whose sessions got their pages in another order
    gives the same bits; evaluating behind pages of another sequence does not)."""
    cfg = tiny_configs["b"]
    toks = H.random_tokens(5, 60, cfg["vocab_size"])
    other = H.random_tokens(6, 60, cfg["vocab_size"])
    with _model(model_folders, "b", share_prefixes=False) as model:
        s = model.session()
        model.step([(s, toks[:40], [])])
        right = model.step([(s, toks[40:], list(range(20)))])
    order = list(range(64))
    random.Random(3).shuffle(order)
    with _model(model_folders, "b", share_prefixes=False, page_order=order) as model:
        s = model.session()
        model.step([(s, toks[:40], [])])
        assert s.pages() == order[:5]
        assert np.array_equal(model.step([(s, toks[40:], list(range(20)))]), right)       # where pages lie changes nothing
    with _model(model_folders, "b", share_prefixes=False) as model:
        s = model.session()
        model.step([(s, other[:40], [])])                                                  # another sequence's keys in the pages
        wrong = model.step([(s, toks[40:], list(range(20)))])
        assert not np.array_equal(wrong, right)


def test_steps_are_all_or_nothing(model_folders, tiny_configs):
    cfg = tiny_configs["a"]
    vocab = cfg["vocab_size"]
    with _model(model_folders, "a", pages=4, share_prefixes=False) as model:
        a, b = model.session(), model.session()
        model.step([(a, H.random_tokens(1, 40, vocab), [])])              # 3 of 4 pages
        before = model.pool_stats()["free_blocks"]
        with pytest.raises(KippError, match="range: KV pool exhausted"):
            model.step([(a, [1, 2], [1]), (b, H.random_tokens(2, 20, vocab), [19])])     # a fits, b needs 2 pages: 1 free
        assert model.pool_stats()["free_blocks"] == before and (a.length, b.length) == (40, 0)
        with pytest.raises(KippError, match="twice"):
            model.step([(a, [1], [0]), (a, [2], [0])])
        with pytest.raises(KippError, match="vocabulary"):
            model.step([(a, [vocab], [0])])
        with pytest.raises(KippError, match="wanted place"):
            model.step([(a, [1, 2], [2])])
        with pytest.raises(KippError, match="at least one token"):
            model.step([(a, [], [])])
        with pytest.raises(KippError, match="capacity"):
            model.step([(a, H.random_tokens(3, 100, vocab), [])])          # 140 tokens: beyond the model's 128 positions
        assert model.pool_stats()["free_blocks"] == before and a.length == 40
        row = model.step([(a, [7], [0])])                                  # and it still works afterwards
        assert row.shape == (1, vocab) and a.length == 41


def test_shared_beginnings_truncation_and_rows_one_by_one(model_folders, tiny_configs):
    """kipp.h's session calls: a finished session publishes its full pages, a fresh one adopts the longest known beginning
    (whole pages, at most (n - 1) / page), truncation never goes below it, eval_n and eval_scored give the rows of
    single-token evaluation (/root/reference/src/kipp.h:172-235, /root/reference/tests/kipp_test.c:3233-3238)."""
    cfg = tiny_configs["b"]
    vocab, folder = cfg["vocab_size"], model_folders[("b", "float32")]
    toks = H.random_tokens(8, 64, vocab)
    ref = H.plain_logits(folder, toks)
    with _model(model_folders, "b", pages=24) as model:
        first = model.session()
        H.assert_close(first.eval(toks[:50])[None], ref[49:50], H.NMSE_F32, "eval")
        first.destroy()                                                     # publishes 6 full pages of 8
        second = model.session()
        assert second.match_prefix(toks[:48]) == 40                         # an exact multiple adopts one page less: a token is left to run
        second.destroy()
        second = model.session()
        assert second.match_prefix(toks) == 48 and second.adopted_tokens == 48
        assert model.pool_stats()["reused_blocks_total"] == 5 + 6
        rows = second.eval_n(toks[48:], 10)
        H.assert_close(rows, ref[54:], H.NMSE_F32, "eval_n behind an adopted beginning")
        with pytest.raises(KippError, match="adopted"):
            second.truncate(40)
        second.truncate(56)
        again = second.eval_scored(toks[56:], 8)
        assert np.array_equal(again, rows[2:])
        third = model.session()
        with pytest.raises(KippError, match="fresh"):
            second.match_prefix(toks)
        batch = model.eval_batch([(third, toks[:30])])
        H.assert_close(batch, ref[29:30], H.NMSE_F32, "eval_batch")
        second.reset()
        assert second.length == 0
    with _model(model_folders, "b", share_prefixes=False) as model:
        s = model.session()
        with pytest.raises(KippError, match="unsupported"):
            s.match_prefix(toks)
        with pytest.raises(KippError, match="alive"):
            err_model = model
            lib = err_model.lib
            from kipp_amd.chost import _Error, _raise
            import ctypes
            e = _Error()
            if lib.kipp_model_close(err_model.handle, ctypes.byref(e)) != 0:
                _raise(lib, e)


def test_model_info_and_stop_tokens(model_folders, tiny_configs, tmp_path):
    with _model(model_folders, "b") as model:
        info = model.info
        cfg = tiny_configs["b"]
        assert info.architecture == b"Qwen3ForCausalLM" and info.path == 2
        assert (info.block_count, info.embedding_length, info.feed_forward_length, info.attention_head_count, info.attention_head_count_kv,
                info.attention_head_dim, info.vocab_size, info.context_length, info.tied_embeddings) == (
            cfg["num_hidden_layers"], cfg["hidden_size"], cfg["intermediate_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"],
            cfg["head_dim"], cfg["vocab_size"], cfg["max_position_embeddings"], 0)
        assert abs(info.rope_theta - cfg["rope_theta"]) < 1 and abs(info.rms_norm_eps - cfg["rms_norm_eps"]) < 1e-12
        assert info.cache_groups == 1 and info.page_tokens == 8 and info.weight_bytes > 0 and info.cache_bytes > 0
    folder = str(tmp_path / "stops")
    shutil.copytree(model_folders[("a", "float32")], folder)
    cfg = json.load(open(os.path.join(folder, "config.json")))
    cfg["eos_token_id"] = [7, 200]
    json.dump(cfg, open(os.path.join(folder, "config.json"), "w"))
    with CModel(folder, path="cpu-fp32") as model:
        assert model.is_stop_token(7) and model.is_stop_token(200) and not model.is_stop_token(8)


def _edit_config(model_folders, tmp_path, **changes):
    folder = str(tmp_path / "edited")
    if os.path.exists(folder):
        shutil.rmtree(folder)
    shutil.copytree(model_folders[("a", "float32")], folder)
    path = os.path.join(folder, "config.json")
    cfg = json.load(open(path))
    for key, value in changes.items():
        if value is ...:
            cfg.pop(key, None)
        else:
            cfg[key] = value
    json.dump(cfg, open(path, "w"))
    return folder


@pytest.mark.parametrize("changes,code,match", [
    ({"rope_scaling": {"type": "yarn", "factor": 4}}, "unsupported", "rope_scaling"),
    ({"attention_bias": True}, "unsupported", "attention_bias"),
    ({"hidden_act": "gelu"}, "unsupported", "hidden_act"),
    ({"use_sliding_window": True}, "unsupported", "use_sliding_window"),
    ({"model_type": "llama"}, "unsupported", "model_type"),
    ({"architectures": ["LlamaForCausalLM"]}, "unsupported", "not in the registry; known: Qwen3ForCausalLM"),
    ({"num_key_value_heads": 3}, "format", "multiple"),
    ({"vocab_size": "256"}, "format", "vocab_size"),
    ({"num_hidden_layers": 0}, "format", "num_hidden_layers"),
    ({"rms_norm_eps": -1.0}, "format", "rms_norm_eps"),
    ({"tie_word_embeddings": "yes"}, "format", "tie_word_embeddings"),
    ({"eos_token_id": 99999}, "format", "eos_token_id"),
    ({"rope_theta": ..., "rms_norm_eps": ...}, "format", "rms_norm_eps, rope_theta"),
])
def test_configurations_the_host_refuses(model_folders, tmp_path, changes, code, match):
    folder = _edit_config(model_folders, tmp_path, **changes)
    with pytest.raises(KippError, match=match) as e:
        CModel(folder, path="cpu-fp32")
    assert e.value.code == code


def test_config_json_is_read_strictly(model_folders, tmp_path):
    folder = _edit_config(model_folders, tmp_path)
    path = os.path.join(folder, "config.json")
    good = open(path).read()
    for bad, match in ((good + " x", "something follows"), (good.replace('"vocab_size"', '"hidden_size": 1, "vocab_size"', 1), "duplicate key"),
                       (good.replace("256", "0256", 1), "leading zero"), ("[" * 70 + "]" * 70, "nested too deeply"),
                       (good.replace('"qwen3"', '"qw\x01en3"'), "control character"), (good[:-1], "unterminated|expected")):
        open(path, "w").write(bad)
        with pytest.raises(KippError, match=match):
            CModel(folder, path="cpu-fp32")


def test_one_error_lists_every_wrong_tensor(model_folders, tmp_path):
    """Missing, unexpected and wrongly shaped tensors and wrong types together, in one error
    (the reference stops at the first: /root/reference/src/kipp.c:859-906, 997-1002)."""
    import torch
    from kipp_amd.weights.safetensors_io import read_file, write_file
    folder = str(tmp_path / "broken")
    shutil.copytree(model_folders[("a", "float32")], folder)
    tensors = dict(read_file(os.path.join(folder, "model.safetensors")))
    del tensors["model.layers.1.mlp.up_proj.weight"], tensors["model.norm.weight"]
    tensors["lm_head.weight"] = torch.zeros(256, 64)                            # tied: the head has no tensor of its own
    tensors["model.layers.0.self_attn.q_norm.weight"] = torch.zeros(8)
    tensors["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(32, 64, dtype=torch.int32)
    write_file(os.path.join(folder, "model.safetensors"), tensors)
    with pytest.raises(KippError) as e:
        CModel(folder, path="cpu-fp32")
    text = e.value.message
    assert e.value.code == "format" and "do not match the configuration" in text
    assert "missing tensors (2): model.layers.1.mlp.up_proj.weight, model.norm.weight" in text
    assert "unexpected tensors (1): lm_head.weight" in text
    assert "model.layers.0.self_attn.q_norm.weight: shape (8), expected (16)" in text
    assert "model.layers.0.self_attn.k_proj.weight: type I32" in text


def test_safetensors_format_errors(model_folders, tmp_path):
    """Errors of the file itself: truncation, a header that does not fit, spans that overlap or leave the file, a span
    that is not product(shape) x element size (/root/reference/src/kipp.c:1032-1061, /root/reference/tools/convert_to_gguf.py:337-340)."""
    import struct
    folder = str(tmp_path / "files")
    shutil.copytree(model_folders[("a", "float32")], folder)
    path = os.path.join(folder, "model.safetensors")
    raw = open(path, "rb").read()
    (n,) = struct.unpack("<Q", raw[:8])
    header = json.loads(raw[8:8 + n])

    def rewrite(new_header, payload=raw[8 + n:]):
        text = json.dumps(new_header).encode()
        open(path, "wb").write(struct.pack("<Q", len(text)) + text + payload)

    def expect(match):
        with pytest.raises(KippError, match=match) as e:
            CModel(folder, path="cpu-fp32")
        assert e.value.code == "format"
    open(path, "wb").write(raw[:5])
    expect("truncated before the header length")
    open(path, "wb").write(struct.pack("<Q", 10**9) + raw[8:])
    expect("does not fit the file")
    open(path, "wb").write(raw[:8] + b"[" + raw[9:])
    expect("not valid JSON")
    names = sorted(k for k in header if k != "__metadata__")
    a, b = names[0], names[1]
    broken = json.loads(json.dumps(header))
    broken[b]["data_offsets"] = [header[a]["data_offsets"][0], header[a]["data_offsets"][0] + header[b]["data_offsets"][1] - header[b]["data_offsets"][0]]
    rewrite(broken)
    expect("overlap")
    broken = json.loads(json.dumps(header))
    broken[a]["data_offsets"][1] += 4
    rewrite(broken)
    expect("spans .* bytes but its shape")
    rewrite(header, raw[8 + n:-16])
    expect("lies outside the file")
    broken = json.loads(json.dumps(header))
    broken[a]["dtype"] = "F8_E4M3"
    rewrite(broken)
    expect("unsupported dtype")
    broken = json.loads(json.dumps(header))
    del broken[a]["shape"]
    rewrite(broken)
    expect("malformed")


def test_sharded_folders(model_folders, tiny_configs, tmp_path):
    """model.safetensors.index.json: every tensor from the shard that the weight_map names
    (/root/reference/tools/convert_to_gguf.py:297-314)."""
    from kipp_amd.weights.safetensors_io import read_file, write_file
    src = model_folders[("b", "float32")]
    folder = str(tmp_path / "sharded")
    os.makedirs(folder)
    shutil.copy(os.path.join(src, "config.json"), folder)
    tensors = dict(read_file(os.path.join(src, "model.safetensors")))
    names = sorted(tensors)
    halves = {"model-00001-of-00002.safetensors": names[::2], "model-00002-of-00002.safetensors": names[1::2]}
    for shard, members in halves.items():
        write_file(os.path.join(folder, shard), {n: tensors[n] for n in members})
    json.dump({"weight_map": {n: shard for shard, members in halves.items() for n in members}},
              open(os.path.join(folder, "model.safetensors.index.json"), "w"))
    toks = H.random_tokens(4, 21, tiny_configs["b"]["vocab_size"])
    with CModel(folder, path="cpu-fp32", page_tokens=8) as model:
        got = model.step([(model.session(), toks, list(range(21)))])
    H.assert_close(got, H.plain_logits(src, toks), H.NMSE_F32, "sharded")
    index = json.load(open(os.path.join(folder, "model.safetensors.index.json")))
    index["weight_map"]["model.ghost.weight"] = "model-00001-of-00002.safetensors"
    json.dump(index, open(os.path.join(folder, "model.safetensors.index.json"), "w"))
    with pytest.raises(KippError, match="listed but absent from their shard: model.ghost.weight"):
        CModel(folder, path="cpu-fp32")


def test_bfloat16_weights_are_widened_exactly(model_folders, tiny_configs):
    """A folder stored in bfloat16 on the float32 path: the same values, widened, as the plain implementation reads them."""
    toks = H.random_tokens(12, 30, tiny_configs["a"]["vocab_size"])
    folder = model_folders[("a", "bfloat16")]
    with CModel(folder, path="cpu-fp32") as model:
        got = model.step([(model.session(), toks, list(range(30)))])
    H.assert_close(got, H.plain_logits(folder, toks), H.NMSE_F32, "bfloat16 file, float32 path")


def test_the_c_sampler_is_the_python_sampler(tiny_configs):
    """Same order, same float widths, same generator: the same token and the same generator state for random
    parameters (vectors of the reference's own tests pin the Python one: tests/test_sampler.py)."""
    from kipp_amd.sampling import SampleParams, XorShift64Star
    from kipp_amd.sampling import sample as py_sample
    rng = np.random.default_rng(5)
    for case in range(300):
        vocab = int(rng.integers(2, 400))
        logits = (rng.normal(size=vocab) * rng.choice([0.5, 3.0, 12.0])).astype(np.float32)
        if case % 7 == 0:
            logits[rng.integers(0, vocab, size=3)] = logits.max()               # ties
        recent = [int(t) for t in rng.integers(0, vocab + 3, size=int(rng.integers(0, 12)))]
        bias = {int(t): float(rng.normal() * 4) for t in rng.integers(0, vocab + 2, size=int(rng.integers(0, 4)))}
        p = SampleParams(temperature=float(rng.choice([0.0, 0.3, 1.0, 2.5])), top_p=float(rng.choice([1.0, 0.9, 0.3, 1e-6])),
                         top_k=int(rng.choice([0, 1, 5, 1000])), min_p=float(rng.choice([0.0, 0.05, 0.5])),
                         repetition_penalty=float(rng.choice([1.0, 1.3, 0.8])), presence_penalty=float(rng.choice([0.0, 0.7])),
                         frequency_penalty=float(rng.choice([0.0, 0.2])), logit_bias=bias)
        seed = int(rng.integers(1, 2**62))
        py_rng, c_rng = XorShift64Star(seed), Rng(seed)
        want = py_sample(logits, p, py_rng, recent)
        got = sample(logits, p.temperature, p.top_p, p.top_k, p.min_p, p.frequency_penalty, p.presence_penalty, p.repetition_penalty,
                     recent, bias, c_rng)
        assert got == want, (case, p)
        assert c_rng.state.value == py_rng.state
    with pytest.raises(KippError, match="top_p"):
        sample(np.zeros(4, np.float32), temperature=1.0, top_p=0.0, rng=Rng(1))
    with pytest.raises(KippError, match="nonzero RNG"):
        sample(np.zeros(4, np.float32), temperature=1.0, rng=Rng(0))
    assert sample(np.array([1.0, 3.0, 3.0, 2.0], np.float32)) == 1               # greedy: the lowest index among equals, no generator


def _toy_mean_folder(folder):
    """A model folder of the architecture that tests/chost/host_test.c defines and registers itself: attention in the even
    layers, a mixer that keeps a running mean as per-session state in the odd ones.  Tensors by the names its parts declare."""
    import json
    import torch
    from kipp_amd.weights.safetensors_io import write_file
    hidden, inner, layers, vocab = 24, 40, 4, 61
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as f:
        json.dump({"architectures": ["ToyMeanForCausalLM"], "vocab_size": vocab, "hidden_size": hidden, "intermediate_size": inner,
                   "num_hidden_layers": layers, "max_position_embeddings": 64}, f)
    gen = torch.Generator().manual_seed(5)
    normal = lambda *shape: torch.randn(*shape, generator=gen) * 0.3
    tensors = {"model.embed_tokens.weight": normal(vocab, hidden), "model.norm.weight": 1 + 0.1 * normal(hidden)}
    for l in range(layers):
        p = f"model.layers.{l}."
        tensors[p + "input_layernorm.weight"] = 1 + 0.1 * normal(hidden)
        tensors[p + "post_attention_layernorm.weight"] = 1 + 0.1 * normal(hidden)
        for name, shape in (("gate_proj", (inner, hidden)), ("up_proj", (inner, hidden)), ("down_proj", (hidden, inner))):
            tensors[p + f"mlp.{name}.weight"] = normal(*shape)
        if l % 2 == 1:
            tensors[p + "mixer.w.weight"] = normal(hidden, hidden)
        else:
            for name, rows in (("q_proj", hidden), ("k_proj", hidden // 2), ("v_proj", hidden // 2)):
                tensors[p + f"self_attn.{name}.weight"] = normal(rows, hidden)
            tensors[p + "self_attn.o_proj.weight"] = normal(hidden, hidden)
    write_file(os.path.join(folder, "model.safetensors"), tensors)
    return folder


def test_host_logic_under_the_sanitizers(model_folders, tmp_path):
    """tests/chost/host_test.c, linked with the host's sources (without the GPU's table) under AddressSanitizer and
    UndefinedBehaviorSanitizer: JSON, checked sizes, pool and cache manager under random orders, both tiny models
    opened and stepped on the scalar path under several cuttings with scrambled tables, error paths, the sampler; and an
    architecture that the test program defines itself (a mixer with per-session state of fixed size), registered, built,
    loaded and stepped by the library as it is."""
    import subprocess
    from kipp_amd.host import build
    here = os.path.dirname(os.path.abspath(__file__))
    exe = build.test_program(os.path.join(here, "chost", "host_test.c"), str(tmp_path / "host_test"))
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1:halt_on_error=1")
    toy = _toy_mean_folder(str(tmp_path / "toy"))
    proc = subprocess.run([exe, model_folders[("a", "float32")], model_folders[("b", "float32")], model_folders[("b", "bfloat16")], "--toy", toy],
                          capture_output=True, text=True, timeout=300, env=env)
    assert proc.returncode == 0, proc.stdout[-2000:] + proc.stderr[-6000:]
    assert proc.stdout.strip().splitlines()[-1].startswith("ok ")
    assert "runtime error" not in proc.stderr and "AddressSanitizer" not in proc.stderr and "LeakSanitizer" not in proc.stderr


def test_the_host_compiles_without_warnings():
    import subprocess
    from kipp_amd.host import build
    for gpu in (False, True):
        flags, _ = build._flags(gpu, False)
        for src in build._sources(gpu):
            proc = subprocess.run([build._compiler()] + flags + ["-fsyntax-only", src], capture_output=True, text=True)
            assert proc.returncode == 0 and "warning" not in proc.stderr, proc.stderr


def test_command_line_on_the_scalar_path(model_folders, tiny_configs, capsys):
    """`--path cpu-fp32`: the command line through the C host, no GPU: the greedy tokens are the plain argmax, the top-N
    table is that of the last token that counts, one KIPP_METRIC line; --max-context and --kv-mib are checked before
    anything runs (/root/reference/src/kipp_cli.c:1057-1067, 1213-1217)."""
    from kipp_amd.cli import main
    from tests.plain import qwen3_plain as plain
    folder = model_folders[("b", "float32")]
    prompt = H.random_tokens(17, 11, tiny_configs["b"]["vocab_size"])
    common = ["--model", folder, "--path", "cpu-fp32", "--tokens", ",".join(map(str, prompt)), "--page", "8"]
    assert main(common + ["--decode", "7", "--top", "4", "--prefill-chunk", "4"]) == 0
    out, err = capsys.readouterr()
    lines = out.strip().splitlines()
    assert lines[0].startswith("generated\t")
    generated = [int(t) for t in lines[0].split("\t")[1].split()]
    cfg, weights = plain.load_folder(folder)
    logits = plain.forward_whole(cfg, weights, prompt + generated)
    for i, token in enumerate(generated):
        assert token == int(np.argmax(logits[len(prompt) - 1 + i]))
    table = [line.split("\t") for line in lines[1:]]
    last = logits[len(prompt) + len(generated) - 2]                # the row the last generated token was chosen from
    assert [int(r[1]) for r in table] == [int(i) for i in np.argsort(-last)[:4]] and [int(r[0]) for r in table] == [1, 2, 3, 4]
    assert abs(float(table[0][2]) - last.max()) < 1e-4
    assert f"KIPP_METRIC backend=cpu-fp32 prefill_tokens={len(prompt)}" in err and "decode_tokens=6" in err
    with pytest.raises(SystemExit, match="exceed the context of 12 tokens"):
        main(common + ["--decode", "7", "--max-context", "12"])
    with pytest.raises(SystemExit, match="holds no page"):
        main(common + ["--decode", "2", "--kv-mib", "0.001"])
    assert main(common + ["--decode", "5", "--kv-mib", "0.02", "--temperature", "0.8", "--seed", "9"]) == 0    # 3 pages of 6,144 bytes
    first = capsys.readouterr().out.splitlines()[0]
    assert main(common + ["--decode", "5", "--kv-mib", "0.02", "--temperature", "0.8", "--seed", "9"]) == 0
    assert capsys.readouterr().out.splitlines()[0] == first       # seeded
    with pytest.raises(KippError, match="KV pool exhausted"):
        main(common + ["--decode", "20", "--kv-mib", "0.02"])      # 31 tokens need 4 pages
    assert main(["--random", "tiny-a", "--seed-weights", "4", "--path", "cpu-fp32", "--tokens", "1,2,3", "--decode", "2"]) == 0


def test_the_c_command_line_matches_the_python_one(model_folders, tiny_configs, capsys, tmp_path):
    """kipp_cli.c over the C scheduler: the same stdout as `python -m kipp_amd.cli --path cpu-fp32` (tokens and top-N table),
    one KIPP_METRIC line, a token file, and refusals with exit code 2 or 1 before or after the model is opened."""
    import subprocess
    from kipp_amd.cli import main
    from kipp_amd.host import build
    exe = build.cli_path()
    folder = model_folders[("a", "float32")]
    prompt = H.random_tokens(23, 13, tiny_configs["a"]["vocab_size"])
    common = ["--model", folder, "--path", "cpu-fp32", "--page", "8", "--decode", "9", "--top", "5", "--prefill-chunk", "5"]
    for sampling in ([], ["--temperature", "0.9", "--top-k", "12", "--top-p", "0.9", "--seed", "5"]):
        assert main(common + ["--tokens", ",".join(map(str, prompt))] + sampling) == 0
        python_out = capsys.readouterr().out
        proc = subprocess.run([exe] + common + ["--tokens", ",".join(map(str, prompt))] + sampling, capture_output=True, text=True, timeout=60)
        assert proc.returncode == 0, proc.stderr
        assert proc.stdout == python_out
        assert f"KIPP_METRIC backend=cpu-fp32 prefill_tokens={len(prompt)}" in proc.stderr and "decode_tokens=8" in proc.stderr
    token_file = tmp_path / "prompt.u32"
    token_file.write_bytes(np.asarray(prompt, "<u4").tobytes())
    from_file = subprocess.run([exe] + common + ["--tokens-file", str(token_file)], capture_output=True, text=True, timeout=60)
    greedy = subprocess.run([exe] + common + ["--tokens", ",".join(map(str, prompt))], capture_output=True, text=True, timeout=60)
    assert from_file.returncode == 0 and greedy.returncode == 0 and from_file.stdout == greedy.stdout
    for extra, code, words in ((["--tokens", "1,2", "--max-context", "8"], 1, "exceed the context of 8 tokens"),
                               (["--tokens", "1,x"], 2, "token ids"),
                               (["--tokens", "1,2", "--path", "metal"], 2, "not built into this engine"),
                               (["--tokens", "1,2", "--kv-mib", "0.0001"], 1, "holds no page"),
                               (["--tokens", str(10 ** 6)], 1, "vocabulary"),
                               (["--tokens", "1,2", "--kv-pages", "1"], 1, "pool")):
        proc = subprocess.run([exe] + common + extra, capture_output=True, text=True, timeout=60)
        assert proc.returncode == code and words in proc.stderr, (extra, proc.returncode, proc.stderr)
    assert subprocess.run([exe, "--help"], capture_output=True, text=True).stdout.startswith("usage: kipp")


def test_perplexity_through_the_c_command_lines(model_folders, tiny_configs, capsys, tmp_path):
    """--ppl on the scalar path, by kipp_cli.c and by `python -m kipp_amd.cli --host c`: windows that do not overlap, each
    from an empty session, a window of W tokens scores W - 1 targets (/root/reference/src/kipp_cli.c:722-790); against
    the plain implementation, and the refusals."""
    import subprocess
    from kipp_amd.cli import main
    from kipp_amd.host import build
    from tests.plain import qwen3_plain as plain
    exe = build.cli_path()
    folder = model_folders[("b", "float32")]
    vocab = tiny_configs["b"]["vocab_size"]
    stream = H.random_tokens(55, 75, vocab)
    path = tmp_path / "tokens.u32"
    path.write_bytes(np.asarray(stream, "<u4").tobytes())
    cfg, weights = plain.load_folder(folder)
    nll, scored = 0.0, 0
    for at in range(0, 75, 32):
        tokens = stream[at:at + 32]
        logits = plain.forward_whole(cfg, weights, tokens)
        for r in range(len(tokens) - 1):
            row = logits[r]
            nll += row.max() + np.log(np.exp(row - row.max()).sum()) - row[tokens[r + 1]]
            scored += 1
    common = ["--model", folder, "--path", "cpu-fp32", "--page", "8", "--ppl", str(path), "--ppl-window", "32", "--prefill-chunk", "10"]
    proc = subprocess.run([exe] + common, capture_output=True, text=True, timeout=120)
    assert proc.returncode == 0, proc.stderr
    assert main(common + ["--host", "c"]) == 0
    for stderr in (proc.stderr, capsys.readouterr().err):
        line = [l for l in stderr.splitlines() if l.startswith("KIPP_PPL")][0]
        fields = dict(f.split("=") for f in line.split()[1:])
        assert fields["backend"] == "cpu-fp32" and int(fields["tokens"]) == 75 and int(fields["scored"]) == scored == 72
        assert int(fields["window"]) == 32 and abs(float(fields["nll"]) - nll) < 1e-3 and abs(float(fields["ppl"]) - np.exp(nll / scored)) < 1e-3
        assert "ppl: window 3/3" in stderr
    limited = subprocess.run([exe] + common + ["--ppl-limit", "33"], capture_output=True, text=True, timeout=120)
    assert limited.returncode == 0 and "tokens=33 scored=31" in limited.stderr          # the second window's one token scores nothing
    (tmp_path / "odd.u32").write_bytes(b"12345")
    (tmp_path / "far.u32").write_bytes(np.asarray([1, vocab], "<u4").tobytes())
    for extra, code, words in ((["--decode", "3"], 2, "cannot be combined"),
                               (["--ppl-window", "1"], 2, "at least 2"),
                               (["--ppl-window", "100000"], 1, "--ppl-window must be between 2 and"),
                               (["--ppl", str(tmp_path / "odd.u32")], 2, "not a uint32 token file"),
                               (["--ppl", str(tmp_path / "far.u32")], 1, "token 1 is out of range"),
                               (["--ppl-limit", "1"], 2, "at least two tokens")):
        bad = subprocess.run([exe] + common + extra, capture_output=True, text=True, timeout=120)
        assert bad.returncode == code and words in bad.stderr, (extra, bad.returncode, bad.stderr)


def test_step_nll_is_the_row_s_log_softmax_at_its_target(model_folders, tiny_configs):
    """kipp_step_nll: a mixed step answered with one float64 a wanted place, -log softmax(row)[target], from the logits
    that kipp_step gives for the same step; targets outside the vocabulary and too little room are refused before anything runs."""
    cfg = tiny_configs["a"]
    vocab = cfg["vocab_size"]
    with CModel(model_folders[("a", "float32")], path="cpu-fp32", page_tokens=4, kv_pool_pages=32, share_prefixes=False) as model:
        a, b, c, d = (model.session() for _ in range(4))
        pa, pb = H.random_tokens(1, 13, vocab), H.random_tokens(2, 7, vocab)
        rows = model.step([(a, pa, [0, 3, 12]), (b, pb, [6])]).astype(np.float64)
        targets = [5, vocab - 1, 0, 9]
        got = model.step_nll([(c, pa, [0, 3, 12]), (d, pb, [6])], targets)
        top = rows.max(axis=1)
        want = top + np.log(np.exp(rows - top[:, None]).sum(axis=1)) - rows[np.arange(4), targets]
        assert np.allclose(got, want, rtol=1e-12, atol=1e-12)
        assert len(model.step_nll([(c, [5], [])], [])) == 0 and c.length == 14
        with pytest.raises(KippError, match="outside the vocabulary"):
            model.step_nll([(c, [1], [0])], [vocab])
        assert c.length == 14


def test_step_argmax_is_the_argmax_of_step(model_folders, tiny_configs):
    """kipp_step_argmax: the same step answered with one index a wanted place, the lowest among equal logits; room is checked."""
    cfg = tiny_configs["a"]
    with CModel(model_folders[("a", "float32")], path="cpu-fp32", page_tokens=4, kv_pool_pages=32, share_prefixes=False) as model:
        a, b, c, d = (model.session() for _ in range(4))
        pa, pb = H.random_tokens(1, 13, cfg["vocab_size"]), H.random_tokens(2, 7, cfg["vocab_size"])
        rows = model.step([(a, pa, [3, 12]), (b, pb, [6])])
        assert model.step_argmax([(c, pa, [3, 12]), (d, pb, [6])]) == [int(np.argmax(r)) for r in rows]
        assert model.step_argmax([(c, [5], [])]) == []
        with pytest.raises(KippError, match="do not fit"):
            import ctypes
            from kipp_amd import chost
            items = (chost._StepItem * 1)()
            t, tp = chost._u32([7, 8])
            w, wp = chost._u32([0, 1])
            items[0] = chost._StepItem(d.handle, tp, 2, wp, 2)
            one = np.zeros(1, np.uint32)
            error = chost._Error()
            if model.lib.kipp_step_argmax(model.handle, items, 1, one.ctypes.data_as(chost._u32p), 1, ctypes.byref(error)) != 0:
                chost._raise(model.lib, error)
        assert d.length == 7                                          # the refused step left the session as it was


def test_single_tokens_made_ready_once_decode_like_step_argmax(model_folders, tiny_configs):
    """`CModel.singles`: the items of kipp_step_argmax built once and fed from one buffer; six greedy steps of three sessions
    give the tokens that step_argmax gives entry by entry."""
    cfg = tiny_configs["b"]
    prompts = [H.random_tokens(10 + i, 5 + 3 * i, cfg["vocab_size"]) for i in range(3)]
    with CModel(model_folders[("b", "float32")], path="cpu-fp32", page_tokens=8, kv_pool_pages=24, share_prefixes=False) as model:
        one, two = [model.session() for _ in prompts], [model.session() for _ in prompts]
        first = model.step_argmax([(s, p, [len(p) - 1]) for s, p in zip(one, prompts)])
        assert model.step_argmax([(s, p, [len(p) - 1]) for s, p in zip(two, prompts)]) == first
        batch = model.singles(two)
        batch.tokens[:] = first
        tokens, seen, want = list(first), [], []
        for _ in range(6):
            tokens = model.step_argmax([(s, [t], [0]) for s, t in zip(one, tokens)])
            want.append(tokens)
            seen.append([int(t) for t in batch.step(feed_back=True)[:3]])
        assert seen == want and [s.length for s in two] == [s.length for s in one]


# ---------------------------------------------------------------------------------------------- the C scheduler

def _greedy(folder, prompt, n, stop=()):
    """What greedy generation gives by the plain implementation: the argmax at every step (recomputing the whole sequence)."""
    from tests.plain import qwen3_plain as plain
    cfg, weights = plain.load_folder(folder)
    toks, out = list(prompt), []
    for _ in range(n):
        t = int(np.argmax(plain.forward_whole(cfg, weights, toks)[-1]))
        if t in stop:
            break
        out.append(t)
        toks.append(t)
    return out


def test_c_scheduler_portions_decode_first_and_the_budget(model_folders, tiny_configs):
    """A prompt goes in in portions, its last portion asks for logits, then one token a step; a decoding request's token
    comes first in a step and portions get what the budget leaves; every generated token is the plain argmax."""
    from kipp_amd.chost import CScheduler
    folder, vocab = model_folders[("a", "float32")], tiny_configs["a"]["vocab_size"]
    a, b = H.random_tokens(1, 11, vocab), H.random_tokens(2, 9, vocab)
    with _model(model_folders, "a", pages=16) as model:
        sched = CScheduler(model, max_step_tokens=6, prefill_chunk=4)
        sched.add(1, a, 5)
        steps = 0
        while not sched.idle:
            produced = sched.step()
            steps += 1
            if steps == 3:
                assert produced and sched.stats["prompt_tokens"] == 11          # portions of 4, 4, 3: the third brings the first token
                sched.add(2, b, 3)                                               # arrives while request 1 decodes
            if steps == 4:
                assert sched.stats["prompt_tokens"] == 11 + 4                    # its first portion, beside request 1's token ...
                assert [rid for rid, _ in produced] == [1]
            if steps == 5:
                assert sched.stats["prompt_tokens"] == 11 + 4 + 4                # ... and so on, 1 + 4 <= 6 a step
        assert sched.result(1)["output"] == _greedy(folder, a, 5) and sched.result(1)["finish_reason"] == "length"
        assert sched.result(2)["output"] == _greedy(folder, b, 3)
        st = sched.stats
        assert (st["requests"], st["finished"], st["failed"], st["generated_tokens"], st["prompt_tokens"]) == (2, 2, 0, 8, 20)
        assert st["queue_wait_count"] == 2 and st["ttft_count"] == 2 and st["decode_seconds_sum"] >= 0
        assert model.pool_stats()["free_blocks"] == 16
        with pytest.raises(KippError, match="already"):
            sched.add(1, a, 2)                                                   # finished, its result not collected yet
        sched.collect(1)
        sched.add(1, a, 2)
        sched.run()
        assert sched.result(1)["output"] == _greedy(folder, a, 2)
        sched.destroy()


def test_c_scheduler_refusals_stop_tokens_and_cancel(model_folders, tiny_configs):
    from kipp_amd.chost import CScheduler
    folder, vocab = model_folders[("a", "float32")], tiny_configs["a"]["vocab_size"]
    prompt = H.random_tokens(3, 7, vocab)
    free = _greedy(folder, prompt, 6)
    with _model(model_folders, "a", pages=4) as model:                           # 64 tokens of pages
        sched = CScheduler(model, max_step_tokens=16, prefill_chunk=8)
        for bad, match in (((9, [], 2), "empty prompt"), ((9, [vocab], 2), "vocabulary"), ((9, [1] * 100, 40), "positions"),
                           ((9, [1] * 60, 10), "more than its pool")):
            with pytest.raises(KippError, match=match):
                sched.add(*bad)
        assert sched.stats["refused"] == 4
        sched.add(1, prompt, 6, stop_tokens=[free[3]])
        sched.add(2, prompt[:5], 0)                                              # nothing to generate: its prompt runs, then it ends
        sched.add(3, H.random_tokens(4, 12, vocab), 30)
        sched.step()
        sched.cancel(3)
        sched.run()
        first = free.index(free[3])
        assert sched.result(1) == {"id": 1, "finish_reason": "stop", "output": free[:first], "error": ""}   # the stop token is neither kept nor fed back
        assert sched.result(2)["finish_reason"] == "length" and sched.result(2)["output"] == []
        assert sched.result(3)["finish_reason"] == "cancelled"
        with pytest.raises(KippError, match="neither waiting nor running"):
            sched.cancel(3)
        assert model.pool_stats()["free_blocks"] == 4
        sched.destroy()


def test_c_scheduler_waits_in_order_when_pages_are_short(model_folders, tiny_configs):
    """Pressure delays, never corrupts (/root/reference/tests/test_server.py:899): three requests of which two fit the pool at a
    time; the third waits although a fourth, smaller one behind it would fit (strict arrival order), and every output is what
    it would be alone."""
    from kipp_amd.chost import CScheduler
    folder, vocab = model_folders[("b", "float32")], tiny_configs["b"]["vocab_size"]
    prompts = {i: H.random_tokens(20 + i, n, vocab) for i, n in ((1, 20), (2, 18), (3, 21), (4, 3))}
    with _model(model_folders, "b", pages=8, share_prefixes=False) as model:      # pages of 8: a request of 20 + 5 tokens needs 3
        sched = CScheduler(model, max_step_tokens=32, prefill_chunk=16)
        for i, p in prompts.items():
            sched.add(i, p, 5 if i < 4 else 2)
        sched.step()
        assert sched.result(3)["finish_reason"] is None and sched.stats["waits_for_pages"] >= 1
        assert sched.stats["queue_wait_count"] == 2                               # 1 and 2 run; 3 waits, and 4 behind it
        sched.run()
        for i, p in prompts.items():
            assert sched.result(i)["output"] == _greedy(folder, p, 5 if i < 4 else 2)
        assert model.pool_stats()["free_blocks"] == 8 and sched.stats["finished"] == 4
        sched.destroy()


def test_c_scheduler_requests_that_begin_alike_adopt_pages(model_folders, tiny_configs):
    """Four requests with a common beginning of five pages arrive together: the later ones wait until the first has
    published those pages (as soon as each is full) and adopt them; the outputs are still the plain argmax."""
    from kipp_amd.chost import CScheduler
    folder, vocab = model_folders[("b", "float32")], tiny_configs["b"]["vocab_size"]
    common = H.random_tokens(61, 43, vocab)
    prompts = [common + H.random_tokens(62 + i, n, vocab) for i, n in enumerate([5, 1, 17, 9])]
    with _model(model_folders, "b", pages=64) as model:
        sched = CScheduler(model, max_step_tokens=24, prefill_chunk=10)
        for i, p in enumerate(prompts):
            sched.add(i, p, 6)
        sched.run()
        st = sched.stats
        assert st["prefix_tokens_reused"] == 3 * 40 and st["prompt_tokens"] == sum(map(len, prompts)) - 120 and st["waits_for_prefix"] > 0
        for i, p in enumerate(prompts):
            assert sched.result(i)["output"] == _greedy(folder, p, 6)
        assert model.pool_stats()["free_blocks"] == 64
        sched.destroy()


def test_c_scheduler_a_failed_step_fails_its_requests_and_the_queue_moves_on(model_folders, tiny_configs):
    """/root/reference/src/kipp_server.c:2081-2088: the batch fails as a unit.  The third forward pass is told to fail: the two
    requests that had tokens in it end as failed with the error's text and give everything back; the one that waited is
    admitted and runs to its end."""
    from kipp_amd.chost import CScheduler
    folder, vocab = model_folders[("a", "float32")], tiny_configs["a"]["vocab_size"]
    prompts = {1: H.random_tokens(31, 30, vocab), 2: H.random_tokens(32, 20, vocab), 3: H.random_tokens(33, 40, vocab)}
    with _model(model_folders, "a", pages=6, share_prefixes=False) as model:      # 3 + 2 pages run; the third request needs 3
        sched = CScheduler(model, max_step_tokens=32, prefill_chunk=16)
        for i, p in prompts.items():
            sched.add(i, p, 4)
        model.lib.kipp_test_fail_forward_after(model.handle, 2)
        sched.run()
        assert sched.result(1)["finish_reason"] == "failed" and sched.result(2)["finish_reason"] == "failed"
        assert "told to fail" in sched.result(1)["error"] and sched.result(1)["error"].startswith("internal:")
        assert sched.result(3) == {"id": 3, "finish_reason": "length", "output": _greedy(folder, prompts[3], 4), "error": ""}
        st = sched.stats
        assert (st["failed"], st["failed_steps"], st["finished"]) == (2, 1, 3)
        assert model.pool_stats()["free_blocks"] == 6
        sched.destroy()


def test_c_scheduler_seeded_sampling_and_penalties(model_folders, tiny_configs):
    """A temperature request has a generator of its own, seeded by the request; the penalties look back over the tokens it
    generated: the same tokens as the Python sampler chooses from the plain logits with the same seed."""
    from kipp_amd.chost import CScheduler
    from kipp_amd.sampling import SampleParams, XorShift64Star
    from kipp_amd.sampling import sample as py_sample
    from tests.plain import qwen3_plain as plain
    folder, vocab = model_folders[("b", "float32")], tiny_configs["b"]["vocab_size"]
    prompt = H.random_tokens(9, 12, vocab)
    with _model(model_folders, "b", pages=16) as model:
        sched = CScheduler(model, keep_last_logits=True)
        sched.add(7, prompt, 10, temperature=0.9, top_k=40, top_p=0.95, repetition_penalty=1.3, frequency_penalty=0.2, seed=11)
        sched.add(8, prompt, 4)                                                  # greedy, beside it
        sched.run()
        got = sched.result(7)["output"]
        assert len(got) == 10 and sched.result(8)["output"] == _greedy(folder, prompt, 4)
        cfg, weights = plain.load_folder(folder)
        rng, toks, out = XorShift64Star(11), list(prompt), []
        params = SampleParams(temperature=0.9, top_k=40, top_p=0.95, repetition_penalty=1.3, frequency_penalty=0.2)
        for _ in range(10):
            row = plain.forward_whole(cfg, weights, toks)[-1].astype(np.float32)
            t = py_sample(row, params, rng, out[-64:])
            out.append(t)
            toks.append(t)
        assert got == out
        last = sched.last_logits(7)
        H.assert_close(last[None], plain.forward_whole(cfg, weights, prompt + out[:-1])[-1:], 1e-9, "the logits the last token was chosen from")
        sched.destroy()
