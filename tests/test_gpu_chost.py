"""The C host on the GPU (`kipp_amd.chost.CModel`, paths gpu-fp32 and gpu-bf16): the same schedules as the Python
engine's tests through kipp_step, against the plain implementation, against the library's own scalar path, and in
float32 bit for bit against the Python engine, which launches the same kernels."""
import numpy as np
import pytest

from tests import helpers as H

pytestmark = pytest.mark.gpu

PAGE = {"a": 16, "b": 8}
LENGTHS = {"a": [1, 17, 40, 64], "b": [7, 33, 61, 100]}
PATH = {"float32": "gpu-fp32", "bfloat16": "gpu-bf16"}


def _requests(key, cfg, seed=0):
    return {f"r{i}": H.random_tokens(seed * 100 + i, n, cfg["vocab_size"]) for i, n in enumerate(LENGTHS[key])}


def _model(model_folders, key, dtype, pages=64, **kw):
    from kipp_amd.chost import CModel
    return CModel(model_folders[(key, dtype)], path=PATH[dtype], page_tokens=PAGE[key], kv_pool_pages=pages, share_prefixes=False, **kw)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("key", ["a", "b"])
@pytest.mark.parametrize("cut", ["whole", "tail", "portions", "mixed"])
def test_c_host_cuttings_match_plain(model_folders, tiny_configs, key, dtype, cut):
    cfg = tiny_configs[key]
    requests = _requests(key, cfg)
    tol = H.NMSE_F32 if dtype == "float32" else H.NMSE_BF16["tiny"]
    if cut == "mixed":
        more = {f"s{i}": H.random_tokens(900 + i, n, cfg["vocab_size"]) for i, n in enumerate(LENGTHS[key])}
        requests = {**requests, **more}
        steps = H.mixed(requests, seed=5)
        pages = H.peak_pages(requests, steps, PAGE[key])          # pages that were given back are used again
        model = _model(model_folders, key, dtype, pages=pages)
        got = H.replay_c(model, requests, steps, scramble_every=3)
    else:
        steps = {"whole": H.whole, "tail": H.tail_one_by_one, "portions": H.changing_portions}[cut](requests)
        model = _model(model_folders, key, dtype)
        got = H.replay_c(model, requests, steps, scramble_every=4 if cut == "portions" else 0)
    for rid, toks in requests.items():
        H.assert_close(got[rid], H.plain_logits(model_folders[(key, dtype)], toks), tol, f"C host {key}/{dtype}/{cut}/{rid}")
    stats = model.pool_stats()
    assert stats["free_blocks"] == stats["total_blocks"]
    model.close()


@pytest.mark.parametrize("key", ["a", "b"])
def test_c_host_float32_is_the_python_engine_bit_for_bit(model_folders, tiny_configs, key):
    """Both hosts launch the same float32 kernels, whose sums run in an order that a row's own position fixes: the
    same bits from either host, under different cuttings."""
    from kipp_amd.engine import Engine
    cfg = tiny_configs[key]
    requests = _requests(key, cfg, seed=3)
    engine = Engine.from_folder(model_folders[(key, "float32")], dtype="float32", page_size=PAGE[key], max_tokens=512, share_prefixes=False)
    base = H.replay(engine, requests, H.whole(requests))
    for maker in (H.whole, H.tail_one_by_one, lambda r: H.mixed(r, seed=11)):
        with _model(model_folders, key, "float32") as model:
            got = H.replay_c(model, requests, maker(requests))
        for rid in requests:
            assert np.array_equal(got[rid], base[rid]), f"{key}/{rid}: the C host's bits differ from the Python engine's"


@pytest.mark.parametrize("key", ["a", "b"])
def test_c_host_gpu_float32_against_its_scalar_path(model_folders, tiny_configs, key):
    """The GPU's float32 kernels against the scalar C references, through the whole model: same formulas, sums in another
    order."""
    from kipp_amd.chost import CModel
    cfg = tiny_configs[key]
    requests = _requests(key, cfg, seed=6)
    steps = H.changing_portions(requests)
    with _model(model_folders, key, "float32") as gpu, CModel(model_folders[(key, "float32")], path="cpu-fp32", page_tokens=PAGE[key],
                                                                kv_pool_pages=64, share_prefixes=False) as cpu:
        got, ref = H.replay_c(gpu, requests, steps), H.replay_c(cpu, requests, steps)
    for rid in requests:
        H.assert_close(got[rid], ref[rid].astype(np.float64), 1e-9, f"GPU float32 against the scalar path {key}/{rid}")


def test_c_host_sessions_on_the_gpu(model_folders, tiny_configs):
    """kipp.h's session calls on the bfloat16 path: shared beginnings, eval_n (the wanted tokens one by one) beside
    eval_scored (one step), truncation, a step that is refused leaves everything as it was."""
    from kipp_amd.chost import CModel, KippError
    cfg = tiny_configs["b"]
    vocab, folder = cfg["vocab_size"], model_folders[("b", "bfloat16")]
    toks = H.random_tokens(8, 64, vocab)
    ref = H.plain_logits(folder, toks)
    with CModel(folder, path="gpu-bf16", page_tokens=8, kv_pool_pages=12) as model:
        first = model.session()
        H.assert_close(first.eval(toks[:50])[None], ref[49:50], H.NMSE_BF16["tiny"], "eval")
        first.destroy()
        second = model.session()
        assert second.match_prefix(toks) == 48
        one_by_one = second.eval_n(toks[48:], 10)
        H.assert_close(one_by_one, ref[54:], H.NMSE_BF16["tiny"], "eval_n")
        second.truncate(54)
        at_once = second.eval_scored(toks[54:], 10)
        H.assert_close(at_once, ref[54:], H.NMSE_BF16["tiny"], "eval_scored")
        third = model.session()
        before = model.pool_stats()["free_blocks"]
        with pytest.raises(KippError, match="KV pool exhausted"):
            model.step([(second, [1], [0]), (third, H.random_tokens(1, 40, vocab), [39])])
        assert model.pool_stats()["free_blocks"] == before and (second.length, third.length) == (64, 0)
        row = model.step([(third, toks[:20], [19])])
        H.assert_close(row, ref[19:20], H.NMSE_BF16["tiny"], "a step after a refused one")
        second.destroy()
        third.destroy()
        # evaluation without a session (a session of its own, gone afterwards; a published beginning is not adopted)
        H.assert_close(model.eval(toks[:30])[None], ref[29:30], H.NMSE_BF16["tiny"], "model eval")
        assert model.pool_stats()["free_blocks"] == model.pool_stats()["total_blocks"]
        with pytest.raises(KippError, match="between 1 and 256"):
            model.eval(list(toks) * 5)


def test_c_host_products_of_every_row_class(model_folders, tiny_configs):
    """A prompt of 230 tokens in one step, portions of 9 to 200 rows and single tokens: the bfloat16 products of the C
    host go to the few-rows kernel, the staged one and the tiled matrix-core kernel by their rows."""
    cfg = tiny_configs["b"]
    toks = H.random_tokens(31, 250, cfg["vocab_size"])
    ref = H.plain_logits(model_folders[("b", "bfloat16")], toks)
    for cuts in ([230, 1, 1, 18], [9, 200, 40, 1], [3, 5, 130, 110, 2]):
        with _model(model_folders, "b", "bfloat16") as model:
            s = model.session()
            rows = []
            for n in cuts:
                at = s.length
                rows.append(model.step([(s, toks[at:at + n], list(range(n)))]))
            H.assert_close(np.concatenate(rows), ref, H.NMSE_BF16["tiny"], f"C host, cuts {cuts}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("key", ["a", "b"])
def test_c_scheduler_on_the_gpu(model_folders, tiny_configs, key, dtype):
    """Seven requests through the C scheduler over so few pages that some wait, portions of six tokens beside decoded
    tokens, two sharing a beginning: every chosen token is the plain implementation's best (within the precision's margin
    of its row), pages all come back, and the counters add up."""
    from kipp_amd.chost import CModel, CScheduler
    cfg = tiny_configs[key]
    vocab = cfg["vocab_size"]
    prompts = {i: H.random_tokens(40 + i, n, vocab) for i, n in enumerate([5, 23, 41, 12, 33, 9, 28])}
    prompts[6] = prompts[2][:2 * PAGE[key] + 3] + prompts[6][:5]
    budget = {i: 4 + 3 * (i % 4) for i in prompts}
    margin = 1e-4 if dtype == "float32" else 0.05
    with CModel(model_folders[(key, dtype)], path=PATH[dtype], page_tokens=PAGE[key], kv_pool_pages=(110 + PAGE[key] - 1) // PAGE[key] + 2,
                max_sessions=4, share_prefixes=True) as model:
        sched = CScheduler(model, max_step_tokens=13, prefill_chunk=6)
        for i, prompt in prompts.items():
            sched.add(i, prompt, budget[i])
        sched.run()
        assert sched.idle
        for i, prompt in prompts.items():
            result = sched.result(i)
            assert result["finish_reason"] == "length" and len(result["output"]) == budget[i]
            ref = H.plain_logits(model_folders[(key, dtype)], prompt + result["output"])
            for j, token in enumerate(result["output"]):
                row = ref[len(prompt) - 1 + j]
                assert row[token] >= row.max() - margin, (key, dtype, i, j, token, int(row.argmax()))
        stats = sched.stats
        assert stats["finished"] == 7 and stats["failed"] == 0 and stats["generated_tokens"] == sum(budget.values())
        assert stats["prompt_tokens"] + stats["prefix_tokens_reused"] == sum(len(p) for p in prompts.values())
        assert stats["waits_for_pages"] > 0
        sched.destroy()
        pool = model.pool_stats()
        assert pool["free_blocks"] == pool["total_blocks"]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_c_host_tokens_chosen_beside_the_logits(model_folders, tiny_configs, dtype):
    """kipp_step_sample: a mixed step (a portion beside single tokens) whose wanted rows are chosen by the device sampler,
    greedy rows and sampled ones with top-k, min-p and top-p, each with the draw that the host sampler takes from a
    generator of the same seed: the same tokens as kipp_sample_ex on the same step's logits.  The scalar path refuses."""
    from kipp_amd.chost import CModel, KippError, Rng, sample
    cfg = tiny_configs["b"]
    vocab, folder = cfg["vocab_size"], model_folders[("b", dtype)]
    with CModel(folder, path=PATH[dtype], page_tokens=8, kv_pool_pages=40, share_prefixes=False) as model:
        twins = []
        for pick in (0, 1):
            sessions = [model.session() for _ in range(4)]
            for i, s in enumerate(sessions[:3]):
                model.step([(s, H.random_tokens(60 + i, 9 + 5 * i, vocab), [])])
            twins.append(sessions)
        portion = H.random_tokens(70, 11, vocab)
        entries = lambda ss: [(ss[0], [3], [0]), (ss[3], portion, [2, 10]), (ss[1], [7], [0]), (ss[2], [11], [0])]
        recent = [5, 9, 5, 5, 77, vocab + 4, 9]
        settings = [dict(), dict(temperature=0.8, top_p=0.9), dict(temperature=1.3, top_k=5, repetition_penalty=1.4, recent=recent),
                    dict(temperature=0.7, top_p=0.95, top_k=40, min_p=0.05, logit_bias={3: 4.0, 100: -2.0, 3 + vocab: 1.0}),
                    dict(presence_penalty=0.5, frequency_penalty=0.2, recent=recent, logit_bias={9: 6.0})]
        for round_ in range(6):                                  # every round other draws; the sessions grow by their tokens
            logits = model.step(entries(twins[0]))
            seeds = [1000 * round_ + 17 * r + 1 for r in range(5)]
            choices = [dict(kw, uniform=Rng(seed).uniform()) for kw, seed in zip(settings, seeds)]
            chosen = model.step_sample(entries(twins[1]), choices)
            expect = [sample(logits[r], rng=Rng(seed), **kw) for r, (kw, seed) in enumerate(zip(settings, seeds))]
            assert chosen == expect, (round_, chosen, expect)    # (the twins' steps are the same launches: the same bits of logits)
            assert chosen[0] == int(np.argmax(logits[0]))
        with pytest.raises(ValueError):
            model.step_sample(entries(twins[1]), choices[:2])
        before = [s.length for s in twins[1]]
        with pytest.raises(KippError, match="top_p in"):
            model.step_sample(entries(twins[1]), [dict(c, top_p=1.5) for c in choices])
        assert [s.length for s in twins[1]] == before            # refused as a whole: nothing was appended
    with CModel(model_folders[("b", "float32")], path="cpu-fp32", page_tokens=8, kv_pool_pages=8) as scalar:
        with pytest.raises(KippError, match="no sampler of its own"):
            scalar.step_sample([(scalar.session(), [1], [0])], [dict()])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_c_host_rows_scored_beside_the_logits(model_folders, tiny_configs, dtype):
    """kipp_step_nll on the GPU paths: -log softmax at a target for every wanted row of a mixed step, against float64 over
    the logits that the same step gives a twin session (the same launches, so the same bits of logits)."""
    from kipp_amd.chost import CModel
    cfg = tiny_configs["b"]
    vocab, folder = cfg["vocab_size"], model_folders[("b", dtype)]
    with CModel(folder, path=PATH[dtype], page_tokens=8, kv_pool_pages=24, share_prefixes=False) as model:
        a, b, c, d = (model.session() for _ in range(4))
        pa, pb = H.random_tokens(31, 29, vocab), H.random_tokens(32, 3, vocab)
        want_a = list(range(0, 29, 3))
        rows = model.step([(a, pa, want_a), (b, pb, [2])]).astype(np.float64)
        targets = H.random_tokens(33, len(want_a) + 1, vocab)
        got = model.step_nll([(c, pa, want_a), (d, pb, [2])], targets)
        top = rows.max(axis=1)
        want = top + np.log(np.exp(rows - top[:, None]).sum(axis=1)) - rows[np.arange(len(targets)), targets]
        assert np.allclose(got, want, rtol=1e-12, atol=1e-12), np.abs(got - want).max()
        one = model.step_nll([(c, [4], [0]), (d, [9], [0])], [1, 2])          # single tokens: the recorded kind of step
        again = model.step([(a, [4], [0]), (b, [9], [0])]).astype(np.float64)
        top = again.max(axis=1)
        assert np.allclose(one, top + np.log(np.exp(again - top[:, None]).sum(axis=1)) - again[[0, 1], [1, 2]], rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_c_scheduler_samples_on_the_device_as_on_the_host(model_folders, tiny_configs, dtype, monkeypatch):
    """Requests with temperature, top-k, top-p and min-p beside greedy ones through the C scheduler: chosen by the device
    sampler, with the draws of each request's generator, they are the tokens that KIPP_AMD_SAMPLER=host (every row's
    logits read back and given to kipp_sample_ex) chooses, also where requests have penalties and a bias."""
    from kipp_amd.chost import CModel, CScheduler
    cfg = tiny_configs["a"]
    vocab = cfg["vocab_size"]
    prompts = {i: H.random_tokens(90 + i, n, vocab) for i, n in enumerate([7, 19, 4, 26, 13])}
    how = {0: dict(temperature=0.9, top_p=0.9, seed=11), 1: dict(temperature=1.2, top_k=8, seed=12), 2: dict(),
           3: dict(temperature=0.7, min_p=0.1, top_p=0.95, seed=14), 4: dict(temperature=1.0, seed=15)}
    outputs = {}
    for sampler in ("device", "host", "penalty", "penalty on the host"):
        monkeypatch.setenv("KIPP_AMD_SAMPLER", "host" if sampler.endswith("host") else "device")
        with CModel(model_folders[("a", dtype)], path=PATH[dtype], page_tokens=PAGE["a"], kv_pool_pages=64, max_sessions=5,
                    share_prefixes=False) as model:
            sched = CScheduler(model, max_step_tokens=24, prefill_chunk=8)
            for i, prompt in prompts.items():
                extra = {}
                if sampler.startswith("penalty"):
                    extra = {4: dict(repetition_penalty=1.3), 2: dict(frequency_penalty=0.4, logit_bias={5: 1.5, 11: -3.0}),
                             0: dict(presence_penalty=0.6)}.get(i, {})
                sched.add(i, prompt, 12, **how[i], **extra)
            sched.run()
            outputs[sampler] = {i: sched.result(i)["output"] for i in prompts}
            assert all(len(o) == 12 for o in outputs[sampler].values())
            sched.destroy()
    assert outputs["device"] == outputs["host"]
    assert outputs["penalty"] == outputs["penalty on the host"]
    assert outputs["penalty"][4] != outputs["device"][4] and all(outputs["penalty"][i] == outputs["device"][i] for i in (1, 3))
    ref = H.plain_logits(model_folders[("a", dtype)], prompts[2] + outputs["device"][2])
    margin = 1e-4 if dtype == "float32" else 0.05
    for j, token in enumerate(outputs["device"][2]):             # the greedy request among them
        row = ref[len(prompts[2]) - 1 + j]
        assert row[token] >= row.max() - margin


@pytest.mark.parametrize("key", ["a", "b"])
def test_both_schedulers_choose_the_same_sampled_tokens(model_folders, tiny_configs, key):
    """On the float32 path the two hosts' logits are the same bits, their generators are the same and both choose on the
    device: requests with every sampling option (temperature, top-k, top-p, min-p, the three penalties, a bias, greedy ones
    among them) get the same tokens from the Python scheduler and from the C one."""
    from kipp_amd.chost import CModel, CScheduler
    from kipp_amd.engine import Engine
    from kipp_amd.engine.scheduler import Request, Scheduler
    from kipp_amd.sampling import SampleParams
    cfg = tiny_configs[key]
    vocab, folder = cfg["vocab_size"], model_folders[(key, "float32")]
    rng = np.random.default_rng(5)
    prompts = [H.random_tokens(300 + i, int(rng.integers(2, 30)), vocab) for i in range(7)]
    how = [dict(), dict(temperature=0.9), dict(temperature=1.3, top_k=12, top_p=0.9), dict(temperature=0.7, min_p=0.05, repetition_penalty=1.4),
           dict(presence_penalty=0.6, frequency_penalty=0.3), dict(temperature=1.0, top_p=0.8, logit_bias={3: 2.0, 17: -5.0}, frequency_penalty=0.2),
           dict(temperature=0.5, top_k=3, presence_penalty=-0.3)]
    new = 20
    engine = Engine.from_folder(folder, dtype="float32", page_size=PAGE[key], max_tokens=7 * 64, share_prefixes=False)
    sched = Scheduler(engine, max_step_tokens=24, prefill_chunk=8)
    for i, prompt in enumerate(prompts):
        sched.add(Request(i, prompt, new, params=SampleParams(**how[i]), seed=40 + i))
    while not sched.idle:
        sched.step()
    by_python = {rid: list(r.output) for rid, r in sched.finished.items()}
    with CModel(folder, path="gpu-fp32", page_tokens=PAGE[key], kv_pool_pages=7 * 64 // PAGE[key] + 8, max_sessions=7, share_prefixes=False) as model:
        csched = CScheduler(model, max_step_tokens=24, prefill_chunk=8)
        for i, prompt in enumerate(prompts):
            csched.add(i, prompt, new, seed=40 + i, **how[i])
        csched.run()
        by_c = {i: csched.result(i)["output"] for i in range(7)}
        csched.destroy()
    assert by_python == by_c and all(len(o) == new for o in by_c.values())


def test_c_command_line_on_the_gpu(model_folders, tiny_configs):
    """The C program on gpu-bf16 and gpu-fp32, given the folder of the built kernels: greedy tokens that the plain
    implementation agrees with, and the KIPP_METRIC line naming the path."""
    import os
    import subprocess
    from kipp_amd.csrc import build as kernels
    from kipp_amd.host import build
    exe = build.cli_path()
    prompt = H.random_tokens(77, 19, tiny_configs["b"]["vocab_size"])
    for dtype, margin in (("float32", 1e-4), ("bfloat16", 0.05)):
        folder = model_folders[("b", dtype)]
        proc = subprocess.run([exe, "--model", folder, "--path", PATH[dtype], "--tokens", ",".join(map(str, prompt)), "--decode", "6", "--page", "8",
                               "--kernels", os.path.join(os.path.dirname(kernels.__file__), "_lib")], capture_output=True, text=True, timeout=120)
        assert proc.returncode == 0, proc.stderr
        generated = [int(t) for t in proc.stdout.splitlines()[0].split("\t")[1].split()]
        assert len(generated) == 6 and f"KIPP_METRIC backend={PATH[dtype]}" in proc.stderr
        ref = H.plain_logits(folder, prompt + generated)
        for j, token in enumerate(generated):
            row = ref[len(prompt) - 1 + j]
            assert row[token] >= row.max() - margin
        # sampled: the tokens are chosen on the device and the last row of logits still comes back for the table: the
        # same output as with every row read back and chosen by kipp_sample_ex, from kipp_cli.c and from `bin/kipp --host c`
        import sys
        sampled = ["--model", folder, "--path", PATH[dtype], "--tokens", ",".join(map(str, prompt)), "--decode", "9", "--page", "8",
                   "--temperature", "0.9", "--top-k", "30", "--top-p", "0.9", "--seed", "21", "--top", "5"]
        outs = []
        for command in ([exe, "--kernels", os.path.join(os.path.dirname(kernels.__file__), "_lib")],
                        [sys.executable, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "bin", "kipp"), "--host", "c"]):
            for sampler in ("device", "host"):
                if sampler == "host" and command[0] != exe:
                    continue                                     # the Python command line has no switch: it is held to kipp_cli.c's output
                run = subprocess.run(command + sampled, capture_output=True, text=True, timeout=300, env=dict(os.environ, KIPP_AMD_SAMPLER=sampler))
                assert run.returncode == 0, run.stderr
                outs.append(run.stdout)
        assert outs[0] == outs[1] == outs[2] and len(outs[0].splitlines()) == 6 and len(outs[0].splitlines()[0].split("\t")[1].split()) == 9


@pytest.mark.parametrize("key", ["a", "b"])
def test_c_host_recorded_steps_give_the_bits_of_steps_run_as_they_are(model_folders, tiny_configs, key):
    """Steps of single tokens are recorded once their shape has come twice and run again from the recording.  Two models
    walk the same schedule, one with recording switched off: three requests decode one token a step, prompts of a fourth and
    fifth come in between (steps that are never recorded, and that use the same workspace), tables are scrambled on the
    way, one request leaves.  Every row of every step has the same bits from both, many steps did run from recordings, and
    the rows are the plain implementation's."""
    from kipp_amd.chost import CModel
    cfg = tiny_configs[key]
    vocab = cfg["vocab_size"]
    prompts = [H.random_tokens(60 + i, n, vocab) for i, n in enumerate([45, 21, 33])]
    late = [H.random_tokens(70 + i, n, vocab) for i, n in enumerate([27, 40])]
    models = [CModel(model_folders[(key, "bfloat16")], path="gpu-bf16", page_tokens=PAGE[key], kv_pool_pages=80, max_sessions=8,
                     share_prefixes=False, eager_steps=eager) for eager in (True, False)]
    got = [[], []]
    for which, model in enumerate(models):
        rows = got[which]
        sessions = [model.session() for _ in prompts]
        for s, p in zip(sessions, prompts):
            rows.append(model.step([(s, p[:-12], [len(p) - 13])]))
        extra = []
        for step in range(12):
            live = [(s, [p[len(p) - 12 + step]], [0]) for s, p in zip(sessions, prompts)]
            if step >= 9:
                live = live[:2]                                     # a shape of two rows from here on
            rows.append(model.step(live))
            if step in (3, 6):                                      # a prompt in between: a step that is not recorded
                extra.append(model.session())
                rows.append(model.step([(extra[-1], late[len(extra) - 1], [0, 5])]))
            if step == 5:
                for s in sessions:
                    s.scramble()
            if step == 7:
                rows.append(model.step_argmax(live))                # the other kind of answer has a recording of its own
                for s, _, _ in live:
                    s.truncate(s.length - 1)
    assert models[0].graph_replays == 0 and models[1].graph_replays >= 8
    for a, b in zip(*got):
        assert np.array_equal(np.asarray(a), np.asarray(b))
    ref = [H.plain_logits(model_folders[(key, "bfloat16")], p) for p in prompts]
    for step in range(9):
        at = len(prompts) + step + (1 if step > 3 else 0) + (1 if step > 6 else 0) + (1 if step > 7 else 0)
        for i, p in enumerate(prompts):
            H.assert_close(got[1][at][i:i + 1], ref[i][len(p) - 12 + step:len(p) - 11 + step], H.NMSE_BF16["tiny"], f"recorded step {step}, request {i}")
    for model in models:
        model.close()


def test_c_host_keeps_a_bounded_number_of_recordings(model_folders, tiny_configs, monkeypatch):
    """With room for two recordings, runs of steps of one, two and three rows push each other out (the one used longest
    ago goes) and are recorded again: every step still has the bits of the model that records nothing."""
    from kipp_amd.chost import CModel
    monkeypatch.setenv("KIPP_AMD_GRAPH_SHAPES", "2")
    vocab = tiny_configs["a"]["vocab_size"]
    prompts = [H.random_tokens(80 + i, 30, vocab) for i in range(3)]
    got = []
    for eager in (True, False):
        rows = []
        with CModel(model_folders[("a", "bfloat16")], path="gpu-bf16", page_tokens=16, kv_pool_pages=12, max_sessions=3,
                    share_prefixes=False, eager_steps=eager) as model:
            sessions = [model.session() for _ in prompts]
            for s, p in zip(sessions, prompts):
                model.step([(s, p[:6], [])])
            for step in range(18):
                live = 1 + (step // 3) % 3                           # three steps of one row, of two, of three, and again
                rows.append(model.step([(s, [p[6 + step]], [0]) for s, p in list(zip(sessions, prompts))[:live]]))
                for s in sessions[live:]:                            # the others keep pace without being asked for logits
                    model.step([(s, [prompts[sessions.index(s)][6 + step]], [])])
            replays = model.graph_replays
        got.append(rows)
        assert replays == 0 if eager else replays > 0
    for a, b in zip(*got):
        assert np.array_equal(a, b)
