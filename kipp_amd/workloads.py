"""Serving workloads through the scheduler, with random weights made on the
device: requests of many lengths under continuous batching with prompts cut into
portions, and requests that share a long beginning (paged prefix reuse).

    python -m kipp_amd.workloads continuous    [--shape qwen3-8b]  [--requests 32] ...
    python -m kipp_amd.workloads shared-prefix [--shape qwen3-32b] [--requests 8]  ...
    python -m kipp_amd.workloads hbm           [--gib 4]
    python -m kipp_amd.workloads mfma
    python -m kipp_amd.workloads products      [--shape qwen3-4b] [--rows 2048,512]
    python -m kipp_amd.workloads portion       [--shape qwen3-4b] [--rows 512] [--behind 4096]
    python -m kipp_amd.workloads c-host        [--shape qwen3-4b] [--batches 8] [--steps 256]

One JSON line: generated tokens a second over the whole run, prompt tokens a
second, time to the first token, and what the cache reused.  `hbm` is no
workload but the yardstick for the decode kernels: how fast a kernel that only
reads gets a large buffer out of memory (best of several grids and ring depths).
`mfma` is the yardstick for the prompt products: what the matrix cores sustain on
operands that never leave the registers.
`products` times the four matrix products of a layer for prompt portions, our
kernel beside the library's; `portion` times a prompt portion behind a context
that is already in the cache (what a step of chunked prefill costs).
`c-host` decodes through the C host (`kipp_amd/host`), host work included.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time


def log(msg: str) -> None:
    print(f"workload: {msg}", file=sys.stderr, flush=True)


def build_engine(shape: str, layers, context: int, pool_tokens: int, max_requests: int, seed: int = 1):
    import torch
    from .config import shape_config
    from .engine import Engine, random_model
    from .runtime import Runtime
    config = shape_config(shape)
    full = config["num_hidden_layers"]
    if layers:
        config["num_hidden_layers"] = min(layers, full)
    config["max_position_embeddings"] = max(context, 64)
    rt = Runtime("bfloat16", "cuda:0")
    start = time.perf_counter()
    model = random_model(config, seed, rt)
    torch.cuda.synchronize()
    log(f"{shape}: {config['num_hidden_layers']} of {full} layers made in {time.perf_counter() - start:.1f} s, "
        f"{torch.cuda.memory_allocated() / 2**30:.1f} GiB")
    engine = Engine(model, page_size=16, max_tokens=pool_tokens, max_requests=max_requests)
    return engine, config, full


def continuous_prompts(n: int, low: int, high: int, vocab: int, seed: int):
    import torch
    gen = torch.Generator().manual_seed(seed)
    lengths = torch.randint(low, high + 1, (n,), generator=gen).tolist()
    return [torch.randint(0, vocab, (length,), generator=gen).tolist() for length in lengths]


def shared_prefix_prompts(n: int, prefix: int, suffix: int, vocab: int, seed: int):
    import torch
    gen = torch.Generator().manual_seed(seed)
    head = torch.randint(0, vocab, (prefix,), generator=gen).tolist()
    return [head + torch.randint(0, vocab, (suffix,), generator=gen).tolist() for _ in range(n)]


def serve(engine, prompts, new_tokens: int, chunk: int, max_step_tokens: int, sampling: dict = None):
    """All requests arrive at once; runs until every one has finished.  `sampling`: the sampler's parameters by name for
    every request (none: greedy); request i draws from seed 100 + i."""
    import torch
    from .engine.scheduler import Request, Scheduler
    from .sampling import SampleParams
    sched = Scheduler(engine, max_step_tokens=max_step_tokens, prefill_chunk=chunk, max_running=len(prompts))
    for i, prompt in enumerate(prompts):
        sched.add(Request(i, prompt, new_tokens, params=SampleParams(**sampling), seed=100 + i) if sampling else Request(i, prompt, new_tokens))
    torch.cuda.synchronize()
    start = time.perf_counter()
    last = start
    while not sched.idle:
        sched.step()
        now = time.perf_counter()
        if now - last > 20:
            log(f"step {sched.stats.steps}: {sched.stats.prompt_tokens} prompt tokens run, "
                f"{sched.stats.generated_tokens} generated, {len(sched.running)} running, {len(sched.waiting)} waiting")
            last = now
    torch.cuda.synchronize()
    seconds = time.perf_counter() - start
    done = sched.finished
    first = [r.first_token_at - r.arrived for r in done.values() if r.first_token_at is not None]
    return sched, seconds, first


def serve_c(config, prompts, new_tokens: int, chunk: int, max_step_tokens: int, share: bool, sampling: dict = None):
    """The same through the C host (`kipp_amd/host`: its scheduler over kipp_step, no Python inside a step): the shape is
    written to a folder with random weights first.  Returns (the scheduler's counters, seconds)."""
    import shutil
    import tempfile

    from .chost import CModel, CScheduler
    from .weights import write_random_model
    tmp = tempfile.mkdtemp(prefix="kipp_workload_")
    try:
        start = time.perf_counter()
        folder = write_random_model(os.path.join(tmp, "model"), config, seed=0, dtype="bfloat16")
        log(f"C host: wrote the model folder in {time.perf_counter() - start:.1f} s")
        pages = sum(-(-(len(p) + new_tokens + 16) // 16) for p in prompts) + 8
        with CModel(folder, path="gpu-bf16", page_tokens=16, kv_pool_pages=pages, max_sessions=len(prompts) + 2,
                    max_step_tokens=max_step_tokens, share_prefixes=share) as model:
            vocab = config["vocab_size"]
            warm = CScheduler(model, max_step_tokens=max_step_tokens, prefill_chunk=chunk, max_running=2)
            for i, p in enumerate(prompts[:2]):          # other tokens: nothing of it is adopted later
                warm.add(i, [(t + 1) % vocab for t in p[:chunk + 3]], 4)
            warm.run()
            warm.destroy()
            sched = CScheduler(model, max_step_tokens=max_step_tokens, prefill_chunk=chunk, max_running=len(prompts))
            for i, p in enumerate(prompts):
                sched.add(i, p, new_tokens, seed=100 + i, **(sampling or {}))
            start = time.perf_counter()
            sched.run()
            seconds = time.perf_counter() - start
            stats = sched.stats
            sched.destroy()
        return stats, seconds
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


def hbm_read(gib: float) -> dict:
    """Read bandwidth of a buffer far larger than every cache, one pass a launch, over
    grids of 1 to 8 workgroups a compute unit and rings of 4 to 16 loads a lane."""
    import torch
    from .csrc import ops
    buf = torch.empty(int(gib * 2**30) // 4, dtype=torch.int32, device="cuda:0")
    buf.fill_(7)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    best, table = None, []
    for per_cu in (1, 2, 4, 8):
        for depth in (4, 8, 16):
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            fastest = 0.0
            for _ in range(4):
                start.record()
                got = ops.stream_read(buf, cus * per_cu, depth)
                end.record()
                torch.cuda.synchronize()
                fastest = max(fastest, got / (start.elapsed_time(end) * 1e-3) / 1e9)
            table.append({"workgroups_per_cu": per_cu, "depth": depth, "GB_s": round(fastest, 1)})
            log(f"{per_cu} workgroups a compute unit, {depth} loads a lane in flight: {fastest:7.1f} GB/s")
            if best is None or fastest > best["GB_s"]:
                best = table[-1]
    return {"workload": "hbm read", "GiB": gib, "compute_units": cus, "best": best, "all": table}


def mfma_rate() -> dict:
    """What the matrix cores sustain on operands that stay in registers: by the operands' bits (zeros, values
    of a normal distribution), the compute units at work, waves a SIMD and the kernel's length."""
    import torch
    from .csrc import ops
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    gen = torch.Generator().manual_seed(0)
    operands = {"zeros": torch.zeros(8192, dtype=torch.bfloat16),
                "normal": torch.randn(8192, generator=gen).to(torch.bfloat16)}
    table = []
    for name, host in operands.items():
        data = host.to("cuda:0")
        for groups, acc, what in ((cus, 16, "1 wave a SIMD"), (2 * cus, 8, "2 waves a SIMD"), (80, 16, "80 compute units")):
            for iters in (400, 4000, 40000):
                start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                ops.mfma_rate(data, groups, acc, iters)
                best = 0.0
                for _ in range(3):
                    start.record()
                    flops = ops.mfma_rate(data, groups, acc, iters)
                    end.record()
                    torch.cuda.synchronize()
                    ms = start.elapsed_time(end)
                    best = max(best, flops / (ms * 1e-3) / 1e15)
                table.append({"operands": name, "grid": what, "ms": round(ms, 3), "PFLOP_s": round(best, 3)})
                log(f"{name:6s} {what:17s} kernel of {ms:8.3f} ms: {best:5.3f} PFLOP/s")
    return {"workload": "mfma rate", "compute_units": cus, "all": table}


def _time(fn, runs: int = 20) -> float:
    """Microseconds a call, over `runs` calls after three that are not timed."""
    import torch
    for _ in range(3):
        fn()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(runs):
        fn()
    end.record()
    end.synchronize()
    return start.elapsed_time(end) / runs * 1e3


def products(shape: str, rows_list) -> dict:
    """The matrix products of one layer at `rows` rows: our kernel for prompt portions (SwiGLU in its end for
    gate/up, K in slabs for the others), cut as planned and in the best of the cuts the runtime times, beside the
    library's product (float32 result, SwiGLU a kernel of its own)."""
    import torch
    from .config import parse_config, shape_config
    from .csrc import ops
    from .runtime import Runtime
    _, cfg = parse_config(shape_config(shape))
    h, q, kv, inner = cfg.hidden_size, cfg.q_dim, cfg.kv_dim, cfg.intermediate_size
    sizes = {"qkv": (q + 2 * kv, h, "slabs"), "o": (h, q, "slabs"), "gate_up": (2 * inner, h, "swiglu"), "down": (h, inner, "slabs")}
    out = {"workload": "products", "shape": shape, "rows": {}}
    for rows in rows_list:
        table = {}
        for name, (n, k, end) in sizes.items():
            x = torch.randn(rows, k, device="cuda:0", dtype=torch.bfloat16)
            w = torch.randn(n, k, device="cuda:0", dtype=torch.bfloat16) * 0.02
            act = torch.empty(rows, n // 2, device="cuda:0", dtype=torch.bfloat16)
            ours = _time(lambda: ops.gemm_tiles(x, w, end, max_parts=4))
            best_cut, best = "plan", ours
            for cut in (Runtime.TILE_CUTS_SLABS if end == "slabs" else Runtime.TILE_CUTS_BF16):
                try:
                    took = _time(lambda: ops.gemm_tiles(x, w, end, max_parts=4, force=cut))
                except ops.KernelError:
                    continue
                if took < best:
                    best_cut, best = str(cut), took
            if end == "swiglu":
                library = _time(lambda: ops.swiglu(torch.mm(x, w.t(), out_dtype=torch.float32), act))
            else:
                library = _time(lambda: torch.mm(x, w.t(), out_dtype=torch.float32))
            flops = 2.0 * rows * n * k
            table[name] = {"ours_us": round(ours, 1), "ours_best_cut": best_cut, "ours_best_us": round(best, 1),
                           "library_us": round(library, 1), "ours_PFLOPs": round(flops / best / 1e9, 3),
                           "library_PFLOPs": round(flops / library / 1e9, 3)}
            log(f"{rows} rows {name:8s} ours as planned {ours:7.1f} us, best cut {best_cut} {best:7.1f} us ({flops / best / 1e9:.2f} PFLOP/s)   "
                f"library {library:7.1f} us ({flops / library / 1e9:.2f} PFLOP/s)")
        out["rows"][str(rows)] = table
    return out


def portion(shape: str, layers, rows: int, behind: int, runs: int = 6) -> dict:
    """A prompt portion of `rows` tokens behind `behind` tokens that are in the cache already: milliseconds a step."""
    import torch
    from .engine import StepEntry
    engine, config, full = build_engine(shape, layers, behind + (runs + 3) * rows + 64, behind + (runs + 3) * rows + 64, 2)
    gen = torch.Generator().manual_seed(1)

    def feed(n):
        engine.step([StepEntry("a", torch.randint(0, config["vocab_size"], (n,), generator=gen).tolist(), [])])
    at = 0
    while at < behind:
        n = min(2048, behind - at)
        feed(n)
        at += n
    for _ in range(2):
        feed(rows)
    torch.cuda.synchronize()
    start = time.perf_counter()
    for _ in range(runs):
        feed(rows)
    host_ms = (time.perf_counter() - start) / runs * 1e3          # the host's own time to launch a step (nothing is waited for)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - start) / runs * 1e3
    log(f"{rows} tokens behind {behind} to {behind + (runs + 2) * rows}: {ms:.2f} ms a step ({host_ms:.2f} ms of it the host's launching), "
        f"{rows / ms * 1e3:.0f} tok/s")
    return {"workload": "portion", "shape": shape, "layers": config["num_hidden_layers"], "rows": rows, "behind": behind,
            "ms_per_step": round(ms, 3), "host_ms_per_step": round(host_ms, 3), "tokens_per_s": round(rows / ms * 1e3, 1),
            "product_choices": {str(k): str(v) for k, v in engine.rt.prompt_product_choices.items()}}


def c_host_decode(config, batches, prompt, steps, warmup):
    """Decode through the C host (`kipp_amd/host`, no Python between the launches of a step): the same shape written to a
    folder with random weights, prompts filled through kipp_step, then `steps` greedy steps timed on the host's clock
    around kipp_step_argmax, everything a serving loop pays included (the batch's integers up, the tokens back); the
    call's arguments are made once (`CModel.singles`), so a step is one call into the library."""
    import shutil
    import tempfile

    import numpy as np
    from kipp_amd.chost import CModel
    from kipp_amd.weights import write_random_model
    tmp = tempfile.mkdtemp(prefix="kipp_bench_")
    points = {}
    try:
        t0 = time.perf_counter()
        folder = write_random_model(os.path.join(tmp, "model"), config, seed=0, dtype="bfloat16")
        log(f"C host: wrote the model folder in {time.perf_counter() - t0:.1f} s")
        most = max(batches)
        per_request = -(-(prompt + steps + warmup + 16) // 16)
        rng = np.random.default_rng(3)
        with CModel(folder, path="gpu-bf16", page_tokens=16, kv_pool_pages=most * per_request, max_sessions=most,
                    max_step_tokens=max(4096, prompt), share_prefixes=False) as model:
            sessions = [model.session() for _ in range(most)]
            for s in sessions:
                model.step([(s, rng.integers(0, config["vocab_size"], prompt).tolist(), [])])
            for b in batches:
                batch = model.singles(sessions[:b])
                batch.tokens[:] = [1 + i for i in range(b)]
                for _ in range(warmup):
                    batch.step(feed_back=True)
                start = time.perf_counter()
                for _ in range(steps):
                    batch.step(feed_back=True)
                took = time.perf_counter() - start
                points[f"decode_b{b}_c_host"] = round(b * steps / took, 1)
                log(f"C host: decode batch {b}: {took / steps * 1e3:.3f} ms/step, {b * steps / took:.0f} tok/s ({model.graph_replays} steps so far ran from recordings)")
                for s in sessions[:b]:
                    s.truncate(prompt)
    finally:
        shutil.rmtree(tmp, ignore_errors=True)
    return points


def main(argv=None) -> int:
    if argv is None:
        argv = sys.argv[1:]
    if argv and argv[0] in ("products", "portion"):
        ap = argparse.ArgumentParser(prog=f"python -m kipp_amd.workloads {argv[0]}")
        ap.add_argument("--shape", default="qwen3-4b")
        ap.add_argument("--layers", type=int, default=0)
        ap.add_argument("--rows", default="2048,512" if argv[0] == "products" else "512")
        ap.add_argument("--behind", type=int, default=4096)
        args = ap.parse_args(argv[1:])
        import torch
        if not torch.cuda.is_available():
            print("workload: no GPU", file=sys.stderr)
            return 1
        rows = [int(r) for r in args.rows.split(",") if r]
        result = products(args.shape, rows) if argv[0] == "products" else portion(args.shape, args.layers, rows[0], args.behind)
        print(json.dumps(result), flush=True)
        return 0
    if argv and argv[0] == "c-host":
        ap = argparse.ArgumentParser(prog="python -m kipp_amd.workloads c-host")
        ap.add_argument("--shape", default="qwen3-4b")
        ap.add_argument("--layers", type=int, default=0)
        ap.add_argument("--batches", default="8")
        ap.add_argument("--prompt", type=int, default=2048)
        ap.add_argument("--steps", type=int, default=256)
        ap.add_argument("--warmup", type=int, default=8)
        args = ap.parse_args(argv[1:])
        from .config import shape_config
        config = shape_config(args.shape)
        if args.layers:
            config["num_hidden_layers"] = args.layers
        points = c_host_decode(config, [int(b) for b in args.batches.split(",") if b], args.prompt, args.steps, args.warmup)
        print(json.dumps({"workload": "c-host", "shape": args.shape, "layers": config["num_hidden_layers"], "prompt": args.prompt,
                          "steps": args.steps, "tokens_per_s": points}), flush=True)
        return 0
    if argv and argv[0] == "mfma":
        import torch
        if not torch.cuda.is_available():
            print("workload: no GPU", file=sys.stderr)
            return 1
        print(json.dumps(mfma_rate()), flush=True)
        return 0
    if argv and argv[0] == "hbm":
        ap = argparse.ArgumentParser(prog="python -m kipp_amd.workloads hbm")
        ap.add_argument("--gib", type=float, default=4.0, help="size of the buffer that is read")
        args = ap.parse_args(argv[1:])
        import torch
        if not torch.cuda.is_available():
            print("workload: no GPU", file=sys.stderr)
            return 1
        print(json.dumps(hbm_read(args.gib)), flush=True)
        return 0
    ap = argparse.ArgumentParser(prog="python -m kipp_amd.workloads", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("workload", choices=["continuous", "shared-prefix"])
    ap.add_argument("--shape", default=None, help="a name under kipp_amd/config/shapes (default: qwen3-8b / qwen3-32b)")
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the shape has (0: all)")
    ap.add_argument("--requests", type=int, default=None)
    ap.add_argument("--new", type=int, default=None, help="tokens generated for each request")
    ap.add_argument("--min-prompt", type=int, default=512)
    ap.add_argument("--max-prompt", type=int, default=4096)
    ap.add_argument("--prefix", type=int, default=6000)
    ap.add_argument("--suffix", type=int, default=500)
    ap.add_argument("--prefill-chunk", type=int, default=512)
    ap.add_argument("--max-step-tokens", type=int, default=2048)
    ap.add_argument("--context", type=int, default=None)
    ap.add_argument("--seed", type=int, default=1)
    ap.add_argument("--no-sharing", action="store_true", help="shared-prefix: compute every prompt in full, for comparison")
    ap.add_argument("--host", choices=["python", "c"], default="python", help="which host serves: the Python engine or the C library")
    ap.add_argument("--temperature", type=float, default=0.0, help="above 0: every request samples (seeded), with the options below")
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--top-k", type=int, default=0)
    ap.add_argument("--repetition-penalty", type=float, default=1.0)
    args = ap.parse_args(argv)

    import torch
    if not torch.cuda.is_available():
        print("workload: no GPU", file=sys.stderr)
        return 1
    cont = args.workload == "continuous"
    shape = args.shape or ("qwen3-8b" if cont else "qwen3-32b")
    n = args.requests or (32 if cont else 8)
    new = args.new or (128 if cont else 256)
    context = args.context or (8192 if cont else 16384)
    longest = args.max_prompt if cont else args.prefix + args.suffix
    if longest + new > context:
        print(f"workload: prompt {longest} + {new} new tokens exceed the context {context}", file=sys.stderr)
        return 1
    per_request = -(-(longest + new) // 64) * 64
    sampling = None
    if args.temperature > 0.0 or args.repetition_penalty != 1.0:
        sampling = dict(temperature=args.temperature, top_p=args.top_p, top_k=args.top_k, repetition_penalty=args.repetition_penalty)
    if args.host == "c":
        from .config import shape_config
        config = shape_config(shape)
        full_layers = config["num_hidden_layers"]
        if args.layers:
            config["num_hidden_layers"] = min(args.layers, full_layers)
        config["max_position_embeddings"] = max(context, 64)
        vocab = config["vocab_size"]
        prompts = (continuous_prompts(n, args.min_prompt, args.max_prompt, vocab, args.seed) if cont
                   else shared_prefix_prompts(n, args.prefix, args.suffix, vocab, args.seed))
        st, seconds = serve_c(config, prompts, new, args.prefill_chunk, args.max_step_tokens, not args.no_sharing, sampling)
        prompt_tokens = sum(len(p) for p in prompts)
        print(json.dumps({
            "workload": args.workload, "host": "c", "value": st["generated_tokens"] / seconds, "unit": "generated tokens/s",
            "seconds": seconds, "requests": n, "generated_tokens": st["generated_tokens"], "prompt_tokens": prompt_tokens,
            "prompt_tokens_run": st["prompt_tokens"], "prefix_tokens_reused": st["prefix_tokens_reused"],
            "total_tokens_per_s": (prompt_tokens + st["generated_tokens"]) / seconds, "steps": st["steps"],
            "first_token_s_mean": st["ttft_seconds_sum"] / max(1, st["ttft_count"]), "dtype": "bf16",
            "data": "synthetic uniform-random tokens, random weights",
            "config": {"model": shape, "layers": config["num_hidden_layers"], "layers_full": full_layers, "context": context,
                       "prefill_chunk": args.prefill_chunk, "max_step_tokens": args.max_step_tokens, "new_tokens": new,
                       "kv_page": 16, "sharing": not args.no_sharing, "sampling": json.dumps(sampling) if sampling else "greedy"}}), flush=True)
        return 0
    engine, config, full_layers = build_engine(shape, args.layers, context, n * per_request, n, args.seed)
    if args.no_sharing:
        engine.cache.share = False
    vocab = config["vocab_size"]
    if cont:
        prompts = continuous_prompts(n, args.min_prompt, args.max_prompt, vocab, args.seed)
    else:
        prompts = shared_prefix_prompts(n, args.prefix, args.suffix, vocab, args.seed)

    warm = [p[:args.prefill_chunk + 3] for p in prompts[:2]]            # other tokens: nothing of it is adopted later
    serve(engine, [[(t + 1) % vocab for t in p] for p in warm], 4, args.prefill_chunk, args.max_step_tokens)
    sched, seconds, first = serve(engine, prompts, new, args.prefill_chunk, args.max_step_tokens, sampling)
    st = sched.stats
    prompt_tokens = sum(len(p) for p in prompts)
    out = {
        "workload": args.workload, "value": st.generated_tokens / seconds, "unit": "generated tokens/s",
        "seconds": seconds, "requests": n, "generated_tokens": st.generated_tokens,
        "prompt_tokens": prompt_tokens, "prompt_tokens_run": st.prompt_tokens,
        "prefix_tokens_reused": st.prefix_tokens_reused,
        "total_tokens_per_s": (prompt_tokens + st.generated_tokens) / seconds,
        "steps": st.steps, "first_token_s_mean": sum(first) / max(1, len(first)), "first_token_s_max": max(first or [0.0]),
        "dtype": "bf16", "data": "synthetic uniform-random tokens, random weights",
        "config": {"model": shape, "layers": config["num_hidden_layers"], "layers_full": full_layers,
                   "hidden": config["hidden_size"], "intermediate": config["intermediate_size"],
                   "heads": config["num_attention_heads"], "kv_heads": config["num_key_value_heads"],
                   "head_dim": config["head_dim"], "vocab": vocab, "context": context,
                   "prefill_chunk": args.prefill_chunk, "max_step_tokens": args.max_step_tokens,
                   "new_tokens": new, "kv_page": 16, "sharing": not args.no_sharing,
                   "sampling": json.dumps(sampling) if sampling else "greedy"},
    }
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
