"""Through the entry points: greedy generation, temperature sampling, the
command line, and trace replay as a user runs it."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

from tests import helpers as H
from tests.plain import qwen3_plain as plain

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _follows_plain_argmax(folder, prompt, output, margin):
    """Teacher-forced: every generated token is the plain implementation's
    argmax at its step (or within `margin` of it, for reduced precision)."""
    cfg, weights = plain.load_folder(folder)
    logits = plain.forward_whole(cfg, weights, list(prompt) + list(output))
    for i, tok in enumerate(output):
        row = logits[len(prompt) - 1 + i]
        assert row[tok] >= row.max() - margin, f"token {i}: chose {tok} ({row[tok]:.5f}), plain argmax {row.argmax()} ({row.max():.5f})"


@pytest.mark.parametrize("key,dtype,margin", [("a", "float32", 1e-5), ("b", "float32", 1e-5), ("a", "bfloat16", 0.03), ("b", "bfloat16", 0.03)])
def test_greedy_generation_through_the_entry_point(model_folders, tiny_configs, key, dtype, margin):
    from kipp_amd import generate
    vocab = tiny_configs[key]["vocab_size"]
    prompts = [H.random_tokens(40 + i, n, vocab) for i, n in enumerate([1, 9, 40, 23])]
    outputs = generate(model_folders[(key, dtype)], prompts, max_new_tokens=16, dtype=dtype,
                       page_size=16 if key == "a" else 8, prefill_chunk=16, max_step_tokens=24)
    assert [len(o) for o in outputs] == [16] * 4
    for prompt, out in zip(prompts, outputs):
        _follows_plain_argmax(model_folders[(key, dtype)], prompt, out, margin)


@pytest.mark.parametrize("dtype,margin", [("float32", 1e-5), ("bfloat16", 0.03)])
def test_requests_that_begin_alike_share_pages_and_still_follow_plain(model_folders, dtype, margin):
    """Four requests with a common beginning of five pages arrive together: the
    later ones adopt the pages the first one publishes while it is still
    running, and every generated token is still the plain argmax."""
    from kipp_amd.engine import Engine
    from kipp_amd.engine.scheduler import Request, Scheduler
    folder = model_folders[("b", dtype)]
    common = H.random_tokens(61, 43, 509)
    prompts = [common + H.random_tokens(62 + i, n, 509) for i, n in enumerate([5, 1, 17, 9])]
    engine = Engine.from_folder(folder, dtype=dtype, page_size=8, max_tokens=4 * 128)
    sched = Scheduler(engine, max_step_tokens=24, prefill_chunk=10)
    for i, prompt in enumerate(prompts):
        sched.add(Request(i, prompt, 12))
    done = sched.run()
    assert sched.stats.prefix_tokens_reused == 3 * 40 and sched.stats.prompt_tokens == sum(map(len, prompts)) - 120
    for i, prompt in enumerate(prompts):
        assert len(done[i].output) == 12
        _follows_plain_argmax(folder, prompt, done[i].output, margin)
    engine.cache.check()
    assert engine.cache.free_pages() == [64]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_running_one_step_ahead_changes_nothing(model_folders, dtype):
    """The scheduler launches a decode step before it has read the tokens of the
    step before.  Same tokens as when it waits for every step: greedy and seeded
    temperature requests, different lengths, a stop token that ends a request one
    step late, a request that arrives in the middle; every page comes back."""
    from kipp_amd.engine import Engine
    from kipp_amd.engine.scheduler import Request, Scheduler
    from kipp_amd.sampling import SampleParams
    folder = model_folders[("a", dtype)]
    prompts = [H.random_tokens(90 + i, n, 256) for i, n in enumerate([5, 17, 33, 2, 9])]

    def run(lookahead, stop_of_first=()):
        engine = Engine.from_folder(folder, dtype=dtype, page_size=16, max_tokens=5 * 128, share_prefixes=False)
        sched = Scheduler(engine, max_step_tokens=64, prefill_chunk=16, lookahead=lookahead)
        for i, prompt in enumerate(prompts[:4]):
            params = SampleParams(temperature=0.9, top_k=40, top_p=0.95) if i % 2 else SampleParams()
            sched.add(Request(i, prompt, [40, 7, 23, 31][i], params=params, seed=11 + i,
                              stop_tokens=tuple(stop_of_first) if i == 0 else ()))
        steps = 0
        while not sched.idle:
            sched.step()
            steps += 1
            if steps == 12:
                sched.add(Request(4, prompts[4], 15))          # arrives while the others decode
        engine.cache.check()
        assert engine.cache.free_pages() == [40] and not engine._uncommitted
        return {rid: (r.output, r.finish_reason) for rid, r in sched.finished.items()}, sched.stats

    plainly, _ = run(False)
    ahead, stats = run(True)
    assert ahead == plainly and [len(ahead[i][0]) for i in range(5)] == [40, 7, 23, 31, 15]
    # not only the same as when it waits: the greedy requests follow the plain implementation's argmax
    for i in (0, 2, 4):
        _follows_plain_argmax(folder, prompts[i], ahead[i][0], 1e-5 if dtype == "float32" else 0.03)
    # end request 0 early by a stop token it is known to produce: one step late, nothing else changes
    stop = plainly[0][0][20]
    first = plainly[0][0].index(stop)
    stopped, _ = run(True, stop_of_first=[stop])
    assert stopped[0] == (plainly[0][0][:first], "stop")
    assert all(stopped[i] == plainly[i] for i in range(1, 5))
    assert run(False, stop_of_first=[stop])[0] == stopped


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_bias_and_penalties_are_applied_where_the_logits_lie(model_folders, dtype):
    """Requests with penalties over their recent tokens and a bias, greedy and sampled, beside plain ones: the scheduler
    changes their rows on the device and chooses there; every token is what the host sampler chooses from the step's
    logits (read through `on_logits` before they are changed) with the request's parameters, recent tokens and draw."""
    from kipp_amd.engine import Engine
    from kipp_amd.engine.scheduler import Request, Scheduler
    from kipp_amd.sampling import SampleParams, XorShift64Star, sample
    folder = model_folders[("a", dtype)]
    prompts = [H.random_tokens(190 + i, n, 256) for i, n in enumerate([6, 21, 3, 14])]
    how = [SampleParams(repetition_penalty=1.5, frequency_penalty=0.3),
           SampleParams(temperature=0.9, top_p=0.9, presence_penalty=0.8, logit_bias={5: 2.0, 40: -4.0}),
           SampleParams(temperature=1.1, top_k=20),
           SampleParams(logit_bias={17: 0.7}, repetition_penalty=0.7)]
    engine = Engine.from_folder(folder, dtype=dtype, page_size=16, max_tokens=4 * 128, share_prefixes=False)
    seen = []

    def keep(requests, logits):
        seen.append(([r.id for r in requests], logits.cpu().numpy().copy(), [list(r.recent) for r in requests]))

    sched = Scheduler(engine, max_step_tokens=32, prefill_chunk=8, on_logits=keep)
    for i, prompt in enumerate(prompts):
        sched.add(Request(i, prompt, 14, params=how[i], seed=70 + i))
    while not sched.idle:
        sched.step()
    outputs = {rid: r.output for rid, r in sched.finished.items()}
    assert all(len(o) == 14 for o in outputs.values())
    twins = {i: XorShift64Star(70 + i) for i in range(4)}
    at = {i: 0 for i in range(4)}
    for ids, logits, recents in seen:
        for row, (rid, recent) in enumerate(zip(ids, recents)):
            want = sample(logits[row], how[rid], twins[rid], recent)
            assert outputs[rid][at[rid]] == want, (rid, at[rid])
            at[rid] += 1
    assert at == {i: 14 for i in range(4)}
    assert len(set(outputs[0])) > 3                              # the penalties keep a greedy request from repeating itself


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_one_step_ahead_with_shared_beginnings_and_a_stop_token(model_folders, dtype):
    """Sharing on: two requests with a common beginning of four pages (the second adopts what the first published early)
    and a third of its own decode together one step ahead of what the scheduler knows; a stop token ends the first one
    step late, and its step in vain leaves nothing behind: the same tokens as waiting for every step gives, the plain
    argmax for the greedy ones, every page back, and a later request still adopts the pages of the one that was stopped."""
    from kipp_amd.engine import Engine
    from kipp_amd.engine.scheduler import Request, Scheduler
    folder = model_folders[("b", dtype)]
    margin = 1e-5 if dtype == "float32" else 0.03
    common = H.random_tokens(71, 32, 509)
    prompts = [common + H.random_tokens(72, 6, 509), common + H.random_tokens(73, 11, 509), H.random_tokens(74, 21, 509)]

    def run(lookahead, stop=()):
        engine = Engine.from_folder(folder, dtype=dtype, page_size=8, max_tokens=4 * 128, share_prefixes=True)
        sched = Scheduler(engine, max_step_tokens=32, prefill_chunk=16, lookahead=lookahead)
        for i, prompt in enumerate(prompts):
            sched.add(Request(i, prompt, [30, 12, 18][i], stop_tokens=tuple(stop) if i == 0 else ()))
        done = sched.run()
        assert sched.stats.prefix_tokens_reused == 32
        # the one that was stopped published its pages as it went: a request that begins like it adopts them
        sched.add(Request("late", prompts[0] + done[0].output[:9], 3))
        late = sched.run()["late"]
        assert sched.stats.prefix_tokens_reused == 32 + (len(prompts[0]) + min(9, len(done[0].output)) - 1) // 8 * 8
        engine.cache.check()
        assert engine.cache.free_pages() == [64] and not engine._uncommitted
        return {rid: (r.output, r.finish_reason) for rid, r in done.items() if rid != "late"}, late.output, sched.stats.steps

    plainly, late_plainly, _ = run(False)
    ahead, late_ahead, _ = run(True)
    assert ahead == plainly and late_ahead == late_plainly
    for i in range(3):
        _follows_plain_argmax(folder, prompts[i], ahead[i][0], margin)
    stop = plainly[0][0][14]
    first = plainly[0][0].index(stop)
    stopped, late_stopped, _ = run(True, stop=[stop])
    assert stopped[0] == (plainly[0][0][:first], "stop") and stopped[1] == plainly[1] and stopped[2] == plainly[2]
    assert run(False, stop=[stop])[:2] == (stopped, late_stopped)
    _follows_plain_argmax(folder, prompts[0] + stopped[0][0][:9], late_stopped, margin)


def test_the_scheduler_with_many_requests(model_folders):
    """150 requests at once (more than one 128-row product and more than the default of running requests):
    greedy and seeded sampling, lengths of 3 to 20; one step ahead gives what waiting for every step gives,
    and every page comes back."""
    from kipp_amd.engine import Engine
    from kipp_amd.engine.scheduler import Request, Scheduler
    from kipp_amd.sampling import SampleParams
    folder = model_folders[("b", "bfloat16")]
    rng = np.random.default_rng(5)
    prompts = [H.random_tokens(500 + i, int(rng.integers(2, 30)), 509) for i in range(150)]
    lengths = [int(rng.integers(3, 21)) for _ in range(150)]

    def run(lookahead):
        engine = Engine.from_folder(folder, dtype="bfloat16", page_size=8, max_tokens=150 * 64, max_requests=150,
                                    share_prefixes=False)
        sched = Scheduler(engine, max_step_tokens=1024, prefill_chunk=64, max_running=150, lookahead=lookahead)
        for i, prompt in enumerate(prompts):
            params = SampleParams(temperature=0.8, top_k=50, top_p=0.9, min_p=0.01) if i % 3 == 0 else SampleParams()
            sched.add(Request(i, prompt, lengths[i], params=params, seed=1000 + i))
        while not sched.idle:
            sched.step()
        engine.cache.check()
        assert engine.cache.free_pages() == [g.pool.num_pages for g in engine.cache.groups] and not engine._uncommitted
        return {rid: r.output for rid, r in sched.finished.items()}

    plainly = run(False)
    ahead = run(True)
    assert ahead == plainly and [len(ahead[i]) for i in range(150)] == lengths


def test_long_decoding_matches_plain(model_folders, tiny_configs):
    """100 tokens decoded one by one after a short prompt, every logits row compared."""
    from kipp_amd.engine import Engine, StepEntry
    folder = model_folders[("b", "float32")]
    engine = Engine.from_folder(folder, dtype="float32", page_size=8, max_tokens=256)
    toks = H.random_tokens(77, 3, 509)
    rows = [engine.step([StepEntry("d", toks, [2])])]
    for _ in range(100):
        nxt = int(engine.choose(rows[-1], [type("R", (), {"params": __import__("kipp_amd.sampling", fromlist=["x"]).SampleParams(), "rng": None, "recent": []})()])[0])
        toks.append(nxt)
        rows.append(engine.step([StepEntry("d", [nxt], [0])]))
    got = np.concatenate([r.cpu().numpy() for r in rows])
    ref = H.plain_logits(folder, toks)[2:]
    H.assert_close(got, ref, H.NMSE_F32, "long decode")


def test_first_tokens_of_a_sequence(model_folders):
    """Positions 0, 1, 2 each as a step of their own: the empty-cache edge."""
    from kipp_amd.engine import Engine, StepEntry
    for dtype, tol in (("float32", H.NMSE_F32), ("bfloat16", H.NMSE_BF16["tiny"])):
        folder = model_folders[("a", dtype)]
        engine = Engine.from_folder(folder, dtype=dtype, page_size=16, max_tokens=64)
        toks = [200, 3, 77]
        got = np.concatenate([engine.step([StepEntry("f", [t], [0])]).float().cpu().numpy() for t in toks])
        H.assert_close(got, H.plain_logits(folder, toks), tol, f"first tokens {dtype}")


def test_temperature_sampling_is_seeded(model_folders, tiny_configs):
    from kipp_amd import generate
    folder = model_folders[("b", "bfloat16")]
    prompts = [H.random_tokens(5, 7, 509), H.random_tokens(6, 33, 509), H.random_tokens(7, 61, 509)]
    kw = dict(max_new_tokens=12, temperature=0.8, seed=11, dtype="bfloat16", page_size=8, prefill_chunk=16)
    a, b = generate(folder, prompts, **kw), generate(folder, prompts, **kw)
    c = generate(folder, prompts, **dict(kw, seed=12))
    assert a == b and a != c and all(len(o) == 12 for o in a)
    top1 = generate(folder, prompts, **dict(kw, top_k=1))
    assert top1 == generate(folder, prompts, **dict(kw, temperature=0.0))


def test_command_line(model_folders):
    folder = model_folders[("a", "float32")]
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "kipp"), "--model", folder, "--dtype", "float32",
                          "--tokens", "5,17,3,99", "--decode", "6", "--top", "3"], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr
    lines = run.stdout.strip().splitlines()
    assert lines[0].startswith("generated\t") and len(lines[0].split("\t")[1].split()) == 6
    generated = [int(t) for t in lines[0].split("\t")[1].split()]
    _follows_plain_argmax(folder, [5, 17, 3, 99], generated, 1e-5)
    table = [l.split("\t") for l in lines[1:4]]
    assert [r[0] for r in table] == ["1", "2", "3"] and float(table[0][2]) >= float(table[1][2]) >= float(table[2][2])
    # the table is of the last evaluated position: the prompt plus all but the last generated token
    ref = H.plain_logits(folder, [5, 17, 3, 99] + generated[:-1])[-1]
    assert int(table[0][1]) == int(ref.argmax()) and abs(float(table[0][2]) - ref.max()) < 1e-4
    assert "KIPP_METRIC backend=hip-float32 prefill_tokens=4" in run.stderr and "decode_tokens=5" in run.stderr


def test_command_line_perplexity(model_folders, tmp_path):
    """--ppl: windows that do not overlap, each from an empty context, a window of W
    tokens scores W - 1 targets; against the plain implementation."""
    import struct
    folder = model_folders[("b", "float32")]
    stream = H.random_tokens(55, 75, 509)
    path = tmp_path / "tokens.u32"
    path.write_bytes(struct.pack("<75I", *stream))
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "kipp"), "--model", folder, "--dtype", "float32", "--page", "8",
                          "--ppl", str(path), "--ppl-window", "32", "--prefill-chunk", "10"], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr
    nll, scored = 0.0, 0
    for at in range(0, 75, 32):
        tokens = stream[at:at + 32]
        logits = H.plain_logits(folder, tokens)
        for r in range(len(tokens) - 1):
            row = logits[r]
            nll += row.max() + np.log(np.exp(row - row.max()).sum()) - row[tokens[r + 1]]
            scored += 1
    line = [l for l in run.stderr.splitlines() if l.startswith("KIPP_PPL")][0]
    fields = dict(f.split("=") for f in line.split()[1:])
    assert fields["backend"] == "hip-float32" and int(fields["tokens"]) == 75 and int(fields["scored"]) == scored == 72
    assert abs(float(fields["nll"]) - nll) < 1e-3 and abs(float(fields["ppl"]) - np.exp(nll / scored)) < 1e-3
    assert "ppl: window 3/3" in run.stderr
    through_c = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "kipp"), "--model", folder, "--host", "c", "--path", "gpu-fp32",
                                "--page", "8", "--ppl", str(path), "--ppl-window", "32", "--prefill-chunk", "10"],
                               capture_output=True, text=True, timeout=300)
    assert through_c.returncode == 0, through_c.stderr
    line = [l for l in through_c.stderr.splitlines() if l.startswith("KIPP_PPL")][0]
    fields = dict(f.split("=") for f in line.split()[1:])
    assert fields["backend"] == "gpu-fp32" and int(fields["scored"]) == 72 and abs(float(fields["nll"]) - nll) < 1e-3
    bad = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "kipp"), "--model", folder, "--backend", "metal", "--tokens", "1"],
                         capture_output=True, text=True, timeout=300)
    assert bad.returncode != 0 and "only hip" in bad.stderr


def _trace(requests, steps):
    fed = {r: 0 for r in requests}
    lines = []
    for i, (entries, ends) in enumerate(steps):
        es = []
        for rid, n in entries:
            es.append({"id": rid, "tokens": list(requests[rid][fed[rid]:fed[rid] + n]), "want": list(range(n))})
            fed[rid] += n
        lines.append(json.dumps({"step": i, "entries": es, "end": ends}))
    return lines


def test_trace_run_says_why_it_refuses_a_step(model_folders, tmp_path):
    """More tokens than --max-tokens gives pages for: one line on standard error, exit code 1, no `done`."""
    folder = model_folders[("a", "float32")]
    proc = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out", str(tmp_path / "o"),
                           "--max-tokens", "64"], input=json.dumps({"step": 0, "entries": [{"id": "x", "tokens": list(range(1, 131)), "want": [129]}],
                                                                    "end": []}) + "\n",
                          capture_output=True, text=True, timeout=120)
    assert proc.returncode == 1 and "done" not in proc.stdout
    assert "step 0 refused" in proc.stderr and "Traceback" not in proc.stderr



@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("key,page,cut,host", [("b", 16, "mixed", "python"), ("a", 16, "portions", "python"), ("b", 8, "portions", "python"),
                                               ("a", 32, "tail", "python"), ("b", 16, "mixed", "c"), ("a", 16, "tail", "c")])
def test_trace_run(model_folders, tiny_configs, tmp_path, dtype, key, page, cut, host):
    folder = model_folders[(key, dtype)]
    vocab = tiny_configs[key]["vocab_size"]
    requests = {f"r{i}": H.random_tokens(300 + i, n, vocab) for i, n in enumerate([70, 33, 100, 7, 61, 90])}
    steps = {"mixed": lambda r: H.mixed(r, seed=9), "portions": H.changing_portions, "tail": H.tail_one_by_one}[cut](requests)
    # --max-tokens: live requests' counts, each rounded up to 64
    fed, peak = {}, 0
    for entries, ends in steps:
        for rid, n in entries:
            fed[rid] = fed.get(rid, 0) + n
        peak = max(peak, sum(-(-n // 64) * 64 for n in fed.values()))
        for rid in ends:
            del fed[rid]
    out = tmp_path / "out"
    proc = subprocess.Popen([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", str(out),
                             "--max-tokens", str(peak), "--page", str(page), "--host", host], stdin=subprocess.PIPE, stdout=subprocess.PIPE,
                            text=True)
    for i, line in enumerate(_trace(requests, steps)):
        proc.stdin.write(line + "\n")
        proc.stdin.flush()
        assert proc.stdout.readline().strip() == f"done {i}"
    proc.stdin.close()
    assert proc.wait(timeout=60) == 0
    rows = {r: [] for r in requests}
    for i, (entries, _) in enumerate(steps):
        data = np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, vocab)
        at = 0
        for rid, n in entries:
            rows[rid].append(data[at:at + n])
            at += n
        assert at == data.shape[0]
    tol = H.NMSE_F32 if dtype == "float32" else H.NMSE_BF16["tiny"]
    for rid, toks in requests.items():
        H.assert_close(np.concatenate(rows[rid]), H.plain_logits(folder, toks), tol, f"trace {key} page {page} {cut} {dtype} {host} {rid}")


def _run_trace(folder, dtype, out, lines, *options):
    proc = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", str(out), *options],
                          input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout.split() == [w for i in range(len(lines)) for w in ("done", str(i))]


@pytest.mark.parametrize("host", ["python", "c"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_with_requests_that_share_a_beginning(model_folders, tiny_configs, tmp_path, dtype, host):
    """--share: a request whose first tokens an earlier request left in the cache adopts those pages (whole pages,
    none that holds a wanted place) and runs the rest only; the logits at the wanted places are the plain ones.
    Pages of 24 tokens, which do not divide 64."""
    folder, vocab = model_folders[("b", dtype)], tiny_configs["b"]["vocab_size"]
    first = H.random_tokens(1, 70, vocab)
    second = first[:50] + H.random_tokens(2, 30, vocab)
    third = first[:50] + H.random_tokens(3, 11, vocab)
    lines = [json.dumps(rec) for rec in (
        {"step": 0, "entries": [{"id": "a", "tokens": first[:40], "want": []}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": first[40:], "want": [25, 29]}], "end": ["a"]},
        # b adopts two pages (48 of the 50 tokens it has in common with a); c wants a place inside them and adopts one
        {"step": 2, "entries": [{"id": "b", "tokens": second, "want": list(range(60, 80))},
                                {"id": "c", "tokens": third[:45], "want": [30, 44]}], "end": []},
        {"step": 3, "entries": [{"id": "c", "tokens": third[45:], "want": list(range(16))}], "end": ["b", "c"]},
        # the pages a, b and c left are used again by a request that shares nothing
        {"step": 4, "entries": [{"id": "d", "tokens": H.random_tokens(4, 128, vocab), "want": [127]}], "end": ["d"]},
    )]
    out = tmp_path / "out"
    _run_trace(folder, dtype, out, lines, "--max-tokens", "192", "--page", "24", "--share", "--host", host)
    tol = H.NMSE_F32 if dtype == "float32" else H.NMSE_BF16["tiny"]

    def rows(step):
        return np.fromfile(out / f"{step}.f32", dtype="<f4").reshape(-1, vocab)
    assert not (out / "0.f32").exists()
    ref_a, ref_b, ref_c = (H.plain_logits(folder, t) for t in (first, second, third))
    H.assert_close(rows(1), ref_a[[65, 69]], tol, f"shared trace {dtype} a")
    got = rows(2)
    H.assert_close(got[:20], ref_b[60:80], tol, f"shared trace {dtype} b")
    H.assert_close(got[20:], ref_c[[30, 44]], tol, f"shared trace {dtype} c")
    H.assert_close(rows(3), ref_c[45:], tol, f"shared trace {dtype} c, second step")
    H.assert_close(rows(4), H.plain_logits(folder, H.random_tokens(4, 128, vocab))[[127]], tol, f"shared trace {dtype} d")


def test_two_bfloat16_replays_write_the_same_bytes(model_folders, tiny_configs, tmp_path):
    """The products of a portion of some hundred rows run on the engine's own kernel in the cut that gives the planned
    bits, whichever cut a process finds fastest: two processes write the same bytes."""
    folder, vocab = model_folders[("b", "bfloat16")], tiny_configs["b"]["vocab_size"]
    toks = H.random_tokens(9, 240, vocab)
    lines = [json.dumps({"step": 0, "entries": [{"id": "x", "tokens": toks[:230], "want": [0, 100, 229]}], "end": []}),
             json.dumps({"step": 1, "entries": [{"id": "x", "tokens": toks[230:], "want": [9]}], "end": ["x"]})]
    for name in ("one", "two"):
        _run_trace(folder, "bfloat16", tmp_path / name, lines, "--max-tokens", "256")
    for step in (0, 1):
        assert (tmp_path / "one" / f"{step}.f32").read_bytes() == (tmp_path / "two" / f"{step}.f32").read_bytes()
    H.assert_close(np.fromfile(tmp_path / "one" / "0.f32", dtype="<f4").reshape(-1, vocab), H.plain_logits(folder, toks)[[0, 100, 229]],
                   H.NMSE_BF16["tiny"], "replayed twice")
