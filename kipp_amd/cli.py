"""Command line in the manner of the reference's `kipp`
(/root/reference/src/kipp_cli.c:571-610 options, :1145-1217 output): evaluate a
prompt, generate `--decode` tokens, print the final top-N logits and one
KIPP_METRIC line.  The prompt is token ids (this engine has no tokenizer).

    python -m kipp_amd.cli --model DIR --tokens 5,17,3 --decode 16
    python -m kipp_amd.cli --model DIR --ppl tokens.u32 --ppl-window 512
    python -m kipp_amd.cli --write-random DIR --random tiny-a --seed-weights 7
    python -m kipp_amd.cli --random tiny-b --seed-weights 3 --tokens 5,17,3 --decode 8      (a model made for this run)
    python -m kipp_amd.cli --model DIR --path cpu-fp32 --tokens 5,17,3 --decode 8             (the C host's scalar path)

`--path` names the execution path as the reference's `--backend` names its own (never a fallback): gpu-bf16 and
gpu-fp32 are `--dtype bfloat16|float32`; cpu-fp32 is the scalar path of the C host, which needs no GPU.  `--host c`
runs the GPU paths through the C host as well.
"""
from __future__ import annotations

import argparse
import math
import struct
import sys
import time


def _parse_tokens(args) -> list:
    if args.tokens is not None:
        return [int(t) for t in args.tokens.replace(",", " ").split()]
    if args.tokens_file is not None:
        with open(args.tokens_file, "rb") as f:
            raw = f.read()
        if len(raw) % 4:
            raise SystemExit("kipp: --tokens-file must hold little-endian uint32 token ids")
        return list(struct.unpack(f"<{len(raw) // 4}I", raw))
    raise SystemExit("kipp: give --tokens or --tokens-file")


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="kipp", description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model", help="model folder (config.json, model.safetensors)")
    ap.add_argument("--tokens", help="prompt as token ids: 5,17,3")
    ap.add_argument("--tokens-file", help="prompt as little-endian uint32 token ids")
    ap.add_argument("--backend", default="hip", help="explicit backend; this engine has one, hip, and never falls back")
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16",
                    help="execution path (default bfloat16; float32 is the true 32-bit path)")
    ap.add_argument("--path", choices=["gpu-bf16", "gpu-fp32", "cpu-fp32"], default=None,
                    help="execution path by name: gpu-bf16, gpu-fp32 (as --dtype), or cpu-fp32, the scalar path of the C host")
    ap.add_argument("--host", choices=["python", "c"], default="python", help="the host that drives the kernels (cpu-fp32 is the C host's)")
    ap.add_argument("--max-context", type=int, default=0,
                    help="most tokens the session may hold (default: the model's positions); prompt + decode beyond it is refused")
    ap.add_argument("--kv-mib", type=float, default=0.0, help="size of the page pool in MiB (instead of --kv-pages)")
    ap.add_argument("--decode", type=int, default=0, help="greedy/sampled tokens to generate")
    ap.add_argument("--temperature", type=float, default=0.0, help="0 = greedy argmax (default)")
    ap.add_argument("--top-p", type=float, default=1.0, help="nucleus mass, 0 < F <= 1 (default 1)")
    ap.add_argument("--top-k", type=int, default=0, help="keep N highest logits (0 = off)")
    ap.add_argument("--min-p", type=float, default=0.0, help="min prob vs top, 0 <= F <= 1 (0 = off)")
    ap.add_argument("--seed", type=int, default=1, help="nonzero sampling seed (default 1)")
    ap.add_argument("--top", type=int, default=10, help="final top-N logits to print (default 10)")
    ap.add_argument("--ppl", metavar="FILE", help="perplexity over a little-endian uint32 token file")
    ap.add_argument("--ppl-window", type=int, default=512, help="tokens of one window; each starts from an empty context")
    ap.add_argument("--ppl-limit", type=int, default=0, help="score at most this many tokens of the file (0 = all)")
    ap.add_argument("--stop-token", type=int, action="append", default=None,
                    help="token that ends decoding (default: eos_token_id of config.json)")
    ap.add_argument("--page", type=int, default=16, help="tokens per cache page")
    ap.add_argument("--kv-pages", type=int, default=None, help="pages in the pool (default: enough for this run)")
    ap.add_argument("--prefill-chunk", type=int, default=512, help="largest portion of a prompt in one step")
    ap.add_argument("--warm-up", action="store_true",
                    help="run one portion of the prompt's first step's size before the clock starts: what a shape decides once a process "
                         "(the cut of a prompt product) then does not count as prefill time")
    ap.add_argument("--max-step-tokens", type=int, default=2048, help="token budget of one step")
    ap.add_argument("--random", metavar="SHAPE",
                    help="named shape (tiny-a, tiny-b, qwen3-4b, ...): with --write-random the folder to write, else the model of this run")
    ap.add_argument("--seed-weights", type=int, default=0, help="seed of the random weights")
    ap.add_argument("--write-random", metavar="DIR", help="write a random-weights model folder and exit")
    ap.add_argument("--weights-dtype", choices=["bfloat16", "float32"], default="bfloat16")
    return ap


def _ppl_stream(args) -> list:
    with open(args.ppl, "rb") as f:
        raw = f.read()
    if len(raw) % 4:
        raise SystemExit(f"kipp: ppl: '{args.ppl}' is not a uint32 token file")
    stream = list(struct.unpack(f"<{len(raw) // 4}I", raw))
    if args.ppl_limit:
        stream = stream[:args.ppl_limit]
    if len(stream) < 2:
        raise SystemExit("kipp: ppl: need at least two tokens to score")
    return stream


def run_perplexity_c(args, stream) -> int:
    """The same protocol through the C host: one session, reset before every window, every portion's rows from one step."""
    from .chost import CModel
    path = args.path or ("gpu-bf16" if args.dtype == "bfloat16" else "gpu-fp32")
    window = args.ppl_window
    with CModel(args.model, path=path, page_tokens=args.page, kv_pool_pages=args.kv_pages or -(-window // args.page), max_sessions=1,
                max_step_tokens=max(args.prefill_chunk, 1), share_prefixes=False) as model:
        if not 2 <= window <= model.context_length:
            raise SystemExit(f"kipp: --ppl-window must be between 2 and {model.context_length}")
        for index, token in enumerate(stream):
            if not 0 <= token < model.vocab_size:
                raise SystemExit(f"kipp: ppl: token {index} is out of range")
        windows = -(-len(stream) // window)
        nll, scored = 0.0, 0
        started = time.perf_counter()
        session = model.session(window)
        for w in range(windows):
            tokens = stream[w * window:(w + 1) * window]
            if len(tokens) < 2:
                break
            session.reset()
            for at in range(0, len(tokens), args.prefill_chunk):
                chunk = tokens[at:at + args.prefill_chunk]
                rows = [r for r in range(len(chunk)) if at + r + 1 < len(tokens)]
                # every row is scored in the step that makes it: only a number a row comes back
                nll += float(model.step_nll([(session, chunk, rows)], [tokens[at + r + 1] for r in rows]).sum())
                scored += len(rows)
            print(f"ppl: window {w + 1}/{windows} ppl={math.exp(nll / scored):.4f}", file=sys.stderr)
        print(f"KIPP_PPL backend={path} tokens={len(stream)} scored={scored} window={window} nll={nll:.9f} "
              f"ppl={math.exp(nll / scored):.6f} seconds={time.perf_counter() - started:.3f}", file=sys.stderr)
    return 0


def run_perplexity(args) -> int:
    """Windows of `--ppl-window` tokens that do not overlap, each from an empty
    context, no burn-in; a window of W tokens scores its W - 1 targets
    (/root/reference/src/kipp_cli.c:646-801: the protocol and the lines printed)."""
    stream = _ppl_stream(args)
    if args.host == "c":
        return run_perplexity_c(args, stream)
    import torch
    from .engine import Engine, StepEntry
    window = args.ppl_window
    engine = Engine.from_folder(args.model, dtype=args.dtype, page_size=args.page,
                                num_pages=args.kv_pages or -(-window // args.page), max_requests=1, share_prefixes=False)
    if not 2 <= window <= engine.model.spec.max_position:
        raise SystemExit(f"kipp: --ppl-window must be between 2 and {engine.model.spec.max_position}")
    for index, token in enumerate(stream):
        if not 0 <= token < engine.vocab_size:
            raise SystemExit(f"kipp: ppl: token {index} is out of range")
    windows = -(-len(stream) // window)
    nll, scored = 0.0, 0
    torch.cuda.synchronize()
    started = time.perf_counter()
    for w in range(windows):
        tokens = stream[w * window:(w + 1) * window]
        if len(tokens) < 2:
            break                                      # a tail of one token has nothing to score
        for at in range(0, len(tokens), args.prefill_chunk):
            chunk = tokens[at:at + args.prefill_chunk]
            rows = [r for r in range(len(chunk)) if at + r + 1 < len(tokens)]
            logits = engine.step([StepEntry("ppl", chunk, rows)])
            if rows:
                # every row's -log softmax at its target by the kernel that the C host scores with (the maximum in float32,
                # exponentials and their sum in float64): only a number a row comes back
                targets = torch.tensor([tokens[at + r + 1] for r in rows], dtype=torch.int32, device=logits.device)
                each = torch.empty(len(rows), dtype=torch.float64, device=logits.device)
                nll += float(engine.rt.ops.row_nll(logits.contiguous(), targets, each).sum())
                scored += len(rows)
        engine.close("ppl")
        print(f"ppl: window {w + 1}/{windows} ppl={math.exp(nll / scored):.4f}", file=sys.stderr)
    torch.cuda.synchronize()
    print(f"KIPP_PPL backend=hip-{args.dtype} tokens={len(stream)} scored={scored} window={window} nll={nll:.9f} "
          f"ppl={math.exp(nll / scored):.6f} seconds={time.perf_counter() - started:.3f}", file=sys.stderr)
    return 0


def main(argv=None) -> int:
    args = build_parser().parse_args(argv)
    if args.backend != "hip":
        raise SystemExit(f"kipp: backend {args.backend!r} is not built into this engine (only hip)")
    if args.write_random:
        from .config import shape_config
        from .weights import write_random_model
        if not args.random:
            raise SystemExit("kipp: --write-random needs --random SHAPE")
        write_random_model(args.write_random, shape_config(args.random), args.seed_weights, args.weights_dtype)
        print(f"kipp: wrote {args.random} (seed {args.seed_weights}, {args.weights_dtype}) to {args.write_random}", file=sys.stderr)
        return 0
    if args.path is not None:
        if args.path != "cpu-fp32":
            args.dtype = "bfloat16" if args.path == "gpu-bf16" else "float32"
        else:
            args.host = "c"
    made = None
    if not args.model and args.random:
        # a model with random weights made for this run, in a folder that goes away with it
        import tempfile
        from .config import shape_config
        from .weights import write_random_model
        made = tempfile.TemporaryDirectory(prefix="kipp-random-")
        args.model = write_random_model(made.name, shape_config(args.random), args.seed_weights, args.weights_dtype)
    if not args.model:
        raise SystemExit("kipp: --model (or --random SHAPE) is required")
    try:
        return _run(args)
    finally:
        if made is not None:
            made.cleanup()


def _pool_pages(args, capacity: int, bytes_per_page: int) -> int:
    """Pages of the pool: --kv-pages, or what --kv-mib holds (/root/reference/src/kipp_server.c:2681-2698), or enough for
    this run."""
    if args.kv_mib:
        pages = int(args.kv_mib * 1024 * 1024) // max(1, bytes_per_page)
        if pages < 1:
            raise SystemExit(f"kipp: --kv-mib {args.kv_mib:g} holds no page of {bytes_per_page} bytes")
        return pages
    return args.kv_pages or -(-capacity // args.page)


def _check_capacity(n_prompt: int, decode: int, limit: int) -> None:
    """/root/reference/src/kipp_cli.c:1057-1067: the session holds prompt + decode tokens, within the context length."""
    if n_prompt > limit or decode > limit - n_prompt:
        raise SystemExit(f"kipp: session: {n_prompt} prompt tokens and {decode} to decode exceed the context of {limit} tokens")


def run_c_host(args, tokens) -> int:
    """The same run through the C host (`kipp_amd/host`): prompt in portions, then one token a step, tokens chosen by
    the C sampler; `--path cpu-fp32` is its scalar path and needs no GPU."""
    import numpy as np
    from .chost import CModel, Rng, sample
    from .config import load_config
    path = args.path or ("gpu-bf16" if args.dtype == "bfloat16" else "gpu-fp32")
    _, cfg = load_config(args.model)
    spec = cfg.model_spec()
    limit = min(args.max_context or spec.max_position, spec.max_position)
    _check_capacity(len(tokens), max(args.decode, 0), limit)
    capacity = len(tokens) + max(args.decode, 0)
    from .engine.model import cache_bytes_per_page
    per_page = cache_bytes_per_page(spec, args.page, 2 if path == "gpu-bf16" else 4) if args.kv_mib else 0
    pages = _pool_pages(args, capacity, per_page)
    model = CModel(args.model, path=path, page_tokens=args.page, kv_pool_pages=pages, max_sessions=1,
                   max_step_tokens=max(args.prefill_chunk, 1), share_prefixes=False)
    stops = tuple(args.stop_token) if args.stop_token is not None else tuple(spec.stop_tokens)
    print(f"kipp: evaluating {len(tokens)} token{'s' if len(tokens) != 1 else ''} on {path} (C host)", file=sys.stderr)
    session = model.session(capacity)
    rng = Rng(args.seed)
    beside = path != "cpu-fp32" and args.decode > 0          # the GPU paths choose the token beside the logits

    def step_and_choose(chunk, place):
        """One step of the session; the token chosen from the row at `place`, and that row."""
        if beside:
            how = dict(temperature=args.temperature, top_p=args.top_p, top_k=args.top_k, min_p=args.min_p,
                       uniform=rng.uniform() if args.temperature > 0 else 0.0)
            chosen, rows = model.step_sample([(session, chunk, [place])], [how], logits=True)
            return chosen[0], rows[0]
        row = model.step([(session, chunk, [place])])[0]
        return (sample(row, args.temperature, args.top_p, args.top_k, args.min_p, rng=rng) if args.decode > 0 else None), row

    started = time.perf_counter()
    row = token = None
    for at in range(0, len(tokens), args.prefill_chunk):
        chunk = tokens[at:at + args.prefill_chunk]
        if at + len(chunk) == len(tokens):
            token, row = step_and_choose(chunk, len(chunk) - 1)
        else:
            model.step([(session, chunk, [])])
    prefill_seconds = time.perf_counter() - started
    started = time.perf_counter()
    output = []
    if args.decode > 0:
        sys.stdout.write("generated\t")
        while token not in stops:
            sys.stdout.write(("" if not output else " ") + str(token))
            sys.stdout.flush()
            output.append(token)
            if len(output) >= args.decode:
                break
            token, row = step_and_choose([token], 0)
        sys.stdout.write("\n")
    decode_seconds = time.perf_counter() - started
    order = sorted(range(len(row)), key=lambda i: (-float(row[i]), i))[:min(args.top, len(row))] if len(row) < 4096 else \
        sorted(np.argpartition(-row, args.top)[:args.top].tolist(), key=lambda i: (-float(row[i]), i))
    for rank, i in enumerate(order, 1):
        print(f"{rank}\t{int(i)}\t{float(row[i]):.9g}")
    decoded = max(0, len(output) - 1) if args.decode else 0
    print(f"KIPP_METRIC backend={path} prefill_tokens={len(tokens)} prefill_seconds={prefill_seconds:.9f} "
          f"decode_tokens={decoded} decode_seconds={decode_seconds:.9f}", file=sys.stderr)
    model.close()
    return 0


def _run(args) -> int:
    if args.ppl:
        return run_perplexity(args)
    if not 1 <= args.top <= 100:
        raise SystemExit("kipp: --top must be between 1 and 100")
    if args.seed == 0:
        raise SystemExit("kipp: --seed must be nonzero")
    tokens = _parse_tokens(args)
    if not tokens:
        raise SystemExit("kipp: the prompt is empty")

    if args.host == "c":
        return run_c_host(args, tokens)

    import torch
    from .config import load_config
    from .engine import Engine, StepEntry
    from .engine.model import cache_bytes_per_page
    from .engine.scheduler import Request, Scheduler
    from .sampling import SampleParams

    _, cfg = load_config(args.model)
    spec = cfg.model_spec()
    limit = min(args.max_context or spec.max_position, spec.max_position)
    _check_capacity(len(tokens), max(args.decode, 0), limit)
    capacity = len(tokens) + args.decode
    per_page = cache_bytes_per_page(spec, args.page, 2 if args.dtype == "bfloat16" else 4) if args.kv_mib else 0
    pages = _pool_pages(args, capacity, per_page)
    engine = Engine.from_folder(args.model, dtype=args.dtype, page_size=args.page, num_pages=pages, max_requests=1,
                                max_position=limit)
    if args.warm_up:
        engine.warm_up((min(len(tokens), args.prefill_chunk, args.max_step_tokens),))
    stops = tuple(args.stop_token) if args.stop_token is not None else tuple(engine.model.spec.stop_tokens)
    backend = f"hip-{args.dtype}"
    print(f"kipp: evaluating {len(tokens)} token{'s' if len(tokens) != 1 else ''} on {backend}", file=sys.stderr)

    # no running ahead: the logits printed at the end are those of the last token that counts;
    # the last logits row is kept for the top-N table
    last = {}

    def keep_last(requests, logits):
        last["row"] = logits[-1].clone()
    sched = Scheduler(engine, max_step_tokens=args.max_step_tokens, prefill_chunk=args.prefill_chunk, max_running=1,
                      lookahead=False, on_logits=keep_last)
    params = SampleParams(temperature=args.temperature, top_p=args.top_p, top_k=args.top_k, min_p=args.min_p)
    req = Request("cli", tokens, max(args.decode, 0), params, seed=args.seed, stop_tokens=stops)
    sched.add(req)

    torch.cuda.synchronize()
    started = time.perf_counter()
    while req.state in ("waiting", "prefill"):
        sched.step()
    torch.cuda.synchronize()
    prefill_seconds = time.perf_counter() - started
    started = time.perf_counter()
    if args.decode:
        sys.stdout.write("generated\t")
        shown = 0
        while True:
            for tok in req.output[shown:]:
                sys.stdout.write(("" if shown == 0 else " ") + str(tok))
                shown += 1
            sys.stdout.flush()
            if req.state == "finished":
                break
            sched.step()
        sys.stdout.write("\n")
    else:
        while req.state != "finished":
            sched.step()
    torch.cuda.synchronize()
    decode_seconds = time.perf_counter() - started

    row = last["row"].float().cpu()
    values, ids = torch.topk(row, min(args.top, row.numel()))
    order = sorted(range(len(ids)), key=lambda i: (-float(values[i]), int(ids[i])))
    for rank, i in enumerate(order, 1):
        print(f"{rank}\t{int(ids[i])}\t{float(values[i]):.9g}")
    decoded = max(0, len(req.output) - 1) if args.decode else 0
    print(f"KIPP_METRIC backend={backend} prefill_tokens={len(tokens)} prefill_seconds={prefill_seconds:.9f} "
          f"decode_tokens={decoded} decode_seconds={decode_seconds:.9f}", file=sys.stderr)
    return 0


if __name__ == "__main__":
    sys.exit(main())
