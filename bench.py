"""Decode and prefill throughput of the Qwen3-4B-shaped model with random
bfloat16 weights on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One JSON line: `value` is decoded tokens a second at batch 8 (a step is one
decode step of the whole batch, tokens chosen greedily on the device and fed
back; by default 256 steps behind prompts of 2,048 tokens, the run from 2,048
to 2,304 tokens that the workload names), with the prefill of one 2,048-token prompt, the decode step's HBM
roofline and the batch-1 / batch-64 / batch-128 points beside it, then points at
longer contexts (decode at batch 8 behind 8,192 and 30,720 tokens, a prompt
portion of 512 tokens behind 4,096 and 16,384).  Peaks are MI355X's published
ones: HBM 8 TB/s, dense bf16 MFMA 2.5 PFLOP/s.

Protocol (after /root/reference/tools/bench.py:203-221 and
/root/reference/bench/README.md:62-68): warm-up steps are discarded; the K timed
steps are run `--repeats` times and the median repeat is the one reported, with
the median absolute deviation beside it; and the run FAILS, printing no line,
unless the timed decode steps were replays of recorded graphs made of the
engine's own kernels (no product went to the library, no attention fell to the
generic kernel): a number from a slower kernel class would otherwise look like
any other.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp16": 2.5e15, "fp8": 5.0e15, "fp32": 157.3e12}
PREFILL_TOKENS = 2048


def log(msg):
    print(f"bench: {msg}", file=sys.stderr, flush=True)


def model_numbers(spec, cache_groups, element_size):
    """What a step costs, from what the model's parts declare (no architecture's field names): the bytes of weights a
    decode step reads (every tensor once; the embedding table only where it is also the head, since a step gathers a
    few rows of it), the elements of the layers' matrices (2 flops a token each), the elements of the head's matrix,
    the cache bytes a token holds (from the cache groups) and the attention flops per (query, key) pair."""
    from kipp_amd.engine.model import model_params
    params = model_params(spec)
    embedding = spec.embedding.prefix + "weight"
    head = embedding if spec.head.tied else spec.head.prefix + "weight"

    def numel(p):
        n = 1
        for d in p.shape:
            n *= d
        return n
    weight_bytes = element_size * sum(numel(p) for name, p in params.items() if name != embedding or spec.head.tied)
    matrix_elems = 0
    per_layer = {}
    for index, layer in enumerate(spec.layers):
        names = [spec_.prefix for _, spec_ in layer.parts if hasattr(spec_, "prefix")]
        per_layer[index] = sum(numel(p) for name, p in params.items()
                               if len(p.shape) == 2 and any(name.startswith(pre) for pre in names) and name not in (embedding, head))
    pair_flops = 0.0
    for run in spec.order:
        matrix_elems += per_layer[run.layer]
        mixer = dict(spec.layers[run.layer].parts).get("mixer")
        pair_flops += 4.0 * getattr(mixer, "q_dim", 0)
    kv_bytes_per_token = sum(g.bytes_per_token(element_size) for g in cache_groups)
    return {"weight_bytes": float(weight_bytes), "matrix_elems": matrix_elems, "head_elems": numel(params[head]),
            "kv_bytes_per_token": kv_bytes_per_token, "pair_flops": pair_flops}


def prefill_flops(numbers, n, behind=0, wanted=1):
    """Flops of a prompt portion of `n` tokens behind `behind` tokens already in the cache, with `wanted` rows of logits."""
    gemm = 2.0 * n * numbers["matrix_elems"] + 2.0 * wanted * numbers["head_elems"]
    attn = numbers["pair_flops"] * (n * behind + n * (n + 1) / 2.0)      # QK^T and PV over the keys each row sees
    return gemm + attn


def fill(engine, ids, prompt_len, vocab, seed, chunk=2048):
    """Put a random prompt of `prompt_len` tokens into the cache for every id;
    returns the first decode token of each (greedy)."""
    import torch
    from kipp_amd.engine import StepEntry
    gen = torch.Generator().manual_seed(seed)
    first = {}
    for rid in ids:
        toks = torch.randint(0, vocab, (prompt_len,), generator=gen).tolist()
        for at in range(0, prompt_len, chunk):
            part = toks[at:at + chunk]
            last = at + chunk >= prompt_len
            logits = engine.step([StepEntry(rid, part, [len(part) - 1] if last else [])])
        first[rid] = int(logits.argmax(dim=-1)[0])
    return first


SAMPLED = dict(temperature=0.8, top_k=50, top_p=0.9)         # the sampled points: every request draws with these, seeded


def decode_run(engine, ids, tokens, steps, warmup, sampled=False):
    """`warmup` untimed and `steps` timed decode steps of all `ids` together, as the
    scheduler runs them: tokens are chosen on the device (greedily, or with `sampled`
    by the device sampler from each request's own generator) and feed the next step
    from there; the host reads them one step behind, while that step runs."""
    import torch
    from kipp_amd.engine import StepEntry
    from kipp_amd.sampling import SampleParams, XorShift64Star

    class Greedy:
        params, rng, recent = SampleParams(), None, ()

    class Sampled:
        recent = ()

        def __init__(self, seed):
            self.params, self.rng = SampleParams(**SAMPLED), XorShift64Star(seed)
    rows = [Sampled(100 + i) for i in range(len(ids))] if sampled else [Greedy()] * len(ids)
    logits = engine.step([StepEntry(r, [tokens[r]], [0]) for r in ids])
    picks = engine.choose(logits, rows, wait=False)
    entries = [StepEntry(r, [0], [0]) for r in ids]

    def one():
        nonlocal picks
        logits = engine.step(entries, device_tokens=picks.device)
        ahead = engine.choose(logits, rows, wait=False)
        for r, t in zip(ids, picks.result()):
            engine.commit(r, [t])                    # what the step just launched was fed
        picks = ahead
    for _ in range(warmup):
        one()
    torch.cuda.synchronize()
    start = time.perf_counter()
    for _ in range(steps):
        one()
    torch.cuda.synchronize()
    return time.perf_counter() - start


class WrongKernelClass(RuntimeError):
    """The timed steps did not run on the kernels the measurement is about."""


def measure_decode(engine, rt, ids, first, steps, warmup, repeats, weight_bytes, kv_per_token, sampled=False):
    """`repeats` timings of `steps` decode steps, each from the same contexts (what a repeat, and the warm-up before the
    first, decoded is cut off again: with 256 steps behind prompts of 2,048 tokens every repeat is the run 2,048 -> 2,304
    tokens); the median one is reported.
    Raises WrongKernelClass unless every timed step was a replay of a recorded graph of our own kernels."""
    timings = []
    lengths = [engine.length(r) for r in ids]

    def cut_back():
        for r, n in zip(ids, lengths):                   # every repeat, and every batch size, decodes behind the prompts alone
            engine.cache.truncate(engine.cache.requests[r], n)
    if warmup > 0:
        decode_run(engine, ids, first, warmup, 0, sampled)
        cut_back()
    again = 0
    rep = 0
    while rep < repeats:
        library, generic, replays = rt.library_products, rt.generic_attention_launches, engine.graphs.replays
        seconds = decode_run(engine, ids, first, steps, 0, sampled)
        cut_back()
        if rt.library_products != library or rt.generic_attention_launches != generic:
            raise WrongKernelClass(f"decode batch {len(ids)}: {rt.library_products - library} products went to the library and "
                                   f"{rt.generic_attention_launches - generic} attention launches to the generic kernel")
        if engine.graphs.replays - replays < steps and again < 3:
            again += 1         # the contexts passed into a bucket whose graph is recorded now: time these steps again
            continue
        if engine.graphs.replays - replays < steps:
            raise WrongKernelClass(f"decode batch {len(ids)}: only {engine.graphs.replays - replays} of {steps + 1} steps "
                                   f"were replays of a recorded graph")
        # bytes a step has to read: every weight once and the cache of the live requests (their lengths mid-way)
        kv_tokens = sum(n + 1 + (steps + 1) / 2.0 for n in lengths)
        timings.append((seconds / steps, weight_bytes + kv_tokens * kv_per_token))
        rep += 1
    per_step = sorted(t for t, _ in timings)
    median = per_step[len(per_step) // 2]
    mad = sorted(abs(t - median) for t in per_step)[len(per_step) // 2]
    nbytes = [b for t, b in timings if t == median][0]
    return {"tok_s": len(ids) / median, "ms": median * 1e3, "mad_ms": mad * 1e3, "steps": steps, "warmup": warmup,
            "bytes": nbytes, "repeats": repeats, "context": [lengths[0] + 1, lengths[0] + 1 + steps]}


def long_context_points(model, rt, cfg, numbers, args, weight_bytes, kv_per_token):
    """Decode at batch 8 behind 8,192 and 30,720 tokens and a prompt portion of 512 tokens behind 4,096 and
    16,384: tokens a second, and the fraction of the roofline (HBM for decode, bf16 MFMA for the portion)."""
    import torch
    from kipp_amd.engine import Engine, StepEntry
    batch, page, top = 8, 16, 30720
    steps, warmup = max(8, min(64, args.steps // 2)), max(2, args.warmup // 2)
    room = top + steps + warmup + 32
    engine = Engine(model, page_size=page, num_pages=batch * (-(-room // page)) + 4, max_requests=batch,
                    share_prefixes=False, max_position=room)
    ids = [f"long{i}" for i in range(batch)]
    gen = torch.Generator().manual_seed(3)
    points, fracs = {}, {}
    portion_ms = {4096: [], 16384: []}
    last = {}

    def feed(rid, n, want_last=False):
        toks = torch.randint(0, cfg.vocab_size, (n,), generator=gen).tolist()
        return engine.step([StepEntry(rid, toks, [n - 1] if want_last else [])])

    def fill_to(target):
        for rid in ids:
            while engine.cache.requests.get(rid) is None or engine.length(rid) < target:
                have = engine.length(rid) if rid in engine.cache.requests else 0
                if have in portion_ms and target - have >= 512:
                    torch.cuda.synchronize()
                    start = time.perf_counter()
                    feed(rid, 512)
                    torch.cuda.synchronize()
                    portion_ms[have].append((time.perf_counter() - start) * 1e3)
                    continue
                n = min(2048, target - have)
                for mark in portion_ms:              # stop at the places where a portion is timed
                    if have < mark < have + n:
                        n = mark - have
                logits = feed(rid, n, want_last=have + n == target)
                if have + n == target:
                    last[rid] = int(logits.argmax(dim=-1)[0])

    for ctx in (8192, top):
        t0 = time.perf_counter()
        fill_to(ctx)
        log(f"{batch} requests filled to {ctx} tokens in {time.perf_counter() - t0:.1f} s")
        r = measure_decode(engine, rt, ids, last, steps, warmup, 3, weight_bytes, kv_per_token)
        points[f"decode_b{batch}_ctx{ctx}"] = round(r["tok_s"], 1)
        fracs[f"decode_b{batch}_ctx{ctx}"] = round(r["bytes"] / (r["ms"] / 1e3) / 1e9 / HBM_PEAK_GBS, 4)
        log(f"decode batch {batch} behind {ctx} tokens: {r['ms']:.3f} ms/step, {r['tok_s']:.0f} tok/s, "
            f"{r['bytes'] / (r['ms'] / 1e3) / 1e9:.0f} GB/s")
        for rid in ids:                              # the tokens of the timed steps are in the cache; go on from a known one
            last[rid] = 0
    for behind, times in portion_ms.items():
        if not times:
            continue
        ms = sorted(times)[len(times) // 2]
        flops = prefill_flops(numbers, 512, behind, wanted=0)
        points[f"prefill512_ctx{behind}"] = round(512 / (ms / 1e3), 1)
        fracs[f"prefill512_ctx{behind}"] = round(flops / (ms / 1e3) / PEAK_FLOPS["bf16"], 4)
        log(f"a portion of 512 tokens behind {behind}: {ms:.2f} ms (median of {len(times)}), {512 / (ms / 1e3):.0f} tok/s")
    return points, fracs


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256,
                    help="timed decode steps; 256 behind prompts of 2,048 tokens is the workload's run from 2,048 to 2,304 tokens")
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--shape", default="qwen3-4b")
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than the shape has (named in config)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt", type=int, default=2048)
    ap.add_argument("--context", type=int, default=None, help="context length (default: the shape's)")
    ap.add_argument("--points", default="1,64,128", help="further decode batch sizes")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--repeats", type=int, default=5, help="times the K timed steps are run; the median is reported")
    ap.add_argument("--no-long", action="store_true", help="leave out the points at longer contexts")
    ap.add_argument("--no-sampled", action="store_true", help="leave out the points with sampling requests")
    ap.add_argument("--no-c-host", action="store_true", help="leave out the points measured through the C host")
    ap.add_argument("--products", choices=["default", "own", "auto", "library"], default="default",
                    help="products of many rows (prompt portions): the runtime's default, our kernel only, the fastest of ours and the library's, the library's")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import torch
    from kipp_amd.config import parse_config, shape_config
    from kipp_amd.engine import Engine, StepEntry, random_model
    from kipp_amd.runtime import Runtime

    config = shape_config(args.shape)
    full_layers = config["num_hidden_layers"]
    layers = args.layers or full_layers
    config["num_hidden_layers"] = layers
    if args.context:
        config["max_position_embeddings"] = args.context
    _, cfg = parse_config(config)
    context = cfg.max_position_embeddings
    points = [int(b) for b in args.points.split(",") if b]
    batches = sorted(set([args.batch] + points))
    max_batch = max(batches)
    page = 16
    log(f"building {args.shape} ({layers} of {full_layers} layers) with random bfloat16 weights on the device ...")
    t0 = time.perf_counter()
    rt = Runtime("bfloat16")
    if args.products != "default":
        rt.own_prompt_products = {"own": True, "auto": "auto", "library": False}[args.products]
    model = random_model(config, seed=0, runtime=rt)
    # every repeat and every batch size starts from the prompts again: room for one run of steps behind a prompt
    repeats = max(1, args.repeats)
    tokens_per_request = args.prompt + max(args.steps, args.warmup) + 16
    if tokens_per_request > context:
        print(f"bench: a prompt of {args.prompt} tokens and {args.steps} steps exceed the context of {context}", file=sys.stderr)
        return 1
    engine = Engine(model, page_size=page, num_pages=max_batch * (-(-tokens_per_request // page)) + 4,
                    max_requests=max_batch, share_prefixes=False)
    torch.cuda.synchronize()
    log(f"model and cache ready in {time.perf_counter() - t0:.1f} s")

    numbers = model_numbers(model.spec, engine.cache.groups, 2)
    weight_bytes, kv_per_token = numbers["weight_bytes"], numbers["kv_bytes_per_token"]

    # ---- prefill of one 2,048-token prompt (logits of the last place)
    prefill = None
    if not args.no_prefill:
        gen = torch.Generator().manual_seed(1)
        times = []
        for i in range(5):
            toks = torch.randint(0, cfg.vocab_size, (PREFILL_TOKENS,), generator=gen).tolist()
            torch.cuda.synchronize()
            start = time.perf_counter()
            engine.step([StepEntry("prefill", toks, [PREFILL_TOKENS - 1])])
            torch.cuda.synchronize()
            times.append(time.perf_counter() - start)
            engine.close("prefill")
        best = sorted(times[1:])[len(times[1:]) // 2]
        flops = prefill_flops(numbers, PREFILL_TOKENS)
        prefill = {"value": round(PREFILL_TOKENS / best, 1), "tokens": PREFILL_TOKENS, "ms": round(best * 1e3, 3),
                   "frac": round(flops / best / PEAK_FLOPS["bf16"], 4)}
        log(f"prefill {PREFILL_TOKENS} tokens: {best * 1e3:.2f} ms, {PREFILL_TOKENS / best:.0f} tok/s")

    # ---- decode at every batch size; the requests of the largest batch are filled once
    ids = [f"d{i}" for i in range(max_batch)]
    log(f"filling {max_batch} requests with {args.prompt}-token prompts ...")
    t0 = time.perf_counter()
    first = fill(engine, ids, args.prompt, cfg.vocab_size, seed=2)
    log(f"filled in {time.perf_counter() - t0:.1f} s")
    results = {}
    for b in batches:
        steps, warmup = args.steps, args.warmup
        try:
            results[b] = measure_decode(engine, rt, ids[:b], first, steps, warmup, repeats, weight_bytes, kv_per_token)
        except Exception as exc:          # a further point must not cost the headline: say so and go on
            if b == args.batch or isinstance(exc, WrongKernelClass):
                raise
            log(f"decode batch {b} failed and is left out: {type(exc).__name__}: {exc}")
            continue
        r = results[b]
        log(f"decode batch {b}: {r['ms']:.3f} ms/step (median of {repeats}, MAD {r['mad_ms']:.3f}), {r['tok_s']:.0f} tok/s, "
            f"{r['bytes'] / (r['ms'] / 1e3) / 1e9:.0f} GB/s")
        # the requests beyond this batch keep their caches; the first ones simply go on
    # ---- the same steps with every request sampling (temperature, top-k, top-p): the step plus the device sampler
    sampled_points = {}
    for b in (b for b in batches if b in (args.batch, 64) and not args.no_sampled):
        try:
            r = measure_decode(engine, rt, ids[:b], first, args.steps, args.warmup, min(repeats, 3), weight_bytes, kv_per_token, sampled=True)
        except Exception as exc:          # noqa: BLE001
            log(f"sampled decode at batch {b} failed and is left out: {type(exc).__name__}: {exc}")
            continue
        sampled_points[f"decode_b{b}_sampled"] = round(r["tok_s"], 1)
        log(f"decode batch {b}, sampled (T {SAMPLED['temperature']}, top-k {SAMPLED['top_k']}, top-p {SAMPLED['top_p']}): "
            f"{r['ms']:.3f} ms/step, {r['tok_s']:.0f} tok/s")

    # ---- longer contexts, on a cache of their own behind the same weights
    long_points, long_fracs = {}, {}
    if not args.no_long:
        del engine
        torch.cuda.empty_cache()
        try:
            long_points, long_fracs = long_context_points(model, rt, cfg, numbers, args, weight_bytes, kv_per_token)
        except WrongKernelClass:
            raise
        except Exception as exc:
            log(f"the points at longer contexts failed and are left out: {type(exc).__name__}: {exc}")

    # ---- the same decode through the C host
    c_points = {}
    if not args.no_c_host:
        try:
            from kipp_amd.workloads import c_host_decode
            c_points = c_host_decode(config, sorted(set([1, args.batch, 64]) & set(batches)) or [args.batch], args.prompt, args.steps, args.warmup)
        except Exception as exc:
            log(f"the points through the C host failed and are left out: {type(exc).__name__}: {exc}")

    main_r = results[args.batch]
    achieved = main_r["bytes"] / (main_r["ms"] / 1e3) / 1e9
    line = {
        "metric": f"decode tok/s at batch {args.batch} ({args.shape.replace('qwen3-', 'Qwen3-').upper().replace('QWEN3', 'Qwen3')}-shaped, bf16, random weights)",
        "value": round(main_r["tok_s"], 1), "unit": "tok/s", "n_gpus": 1, "steps": main_r["steps"],
        "warmup": main_r["warmup"], "ms_per_step": round(main_r["ms"], 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"model": args.shape, "layers": layers, "layers_of_shape": full_layers, "hidden": cfg.hidden_size,
                   "q_heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                   "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size, "tied": cfg.tie_word_embeddings,
                   "global_batch": args.batch, "seq_len": context, "prompt_tokens": args.prompt,
                   "decoded_tokens": main_r["steps"], "kv_page": page,
                   "parallelism": "none", "weights": "random N(0,0.02) seed 0"},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
        "points": {f"decode_b{b}": round(results[b]["tok_s"], 1) for b in batches if b != args.batch and b in results},
        "protocol": {"repeats": main_r["repeats"], "reported": "median", "mad_ms_per_step": round(main_r["mad_ms"], 4),
                     "timed_steps_are_graph_replays_of_own_kernels": True},
    }
    line["points"].update(sampled_points)
    line["points"].update(long_points)
    line["points"].update(c_points)
    line["points_roofline_frac"] = {f"decode_b{b}": round(results[b]["bytes"] / (results[b]["ms"] / 1e3) / 1e9 / HBM_PEAK_GBS, 4)
                                    for b in batches if b != args.batch and b in results}
    line["points_roofline_frac"].update(long_fracs)
    if prefill is not None:
        line["prefill"] = prefill
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
