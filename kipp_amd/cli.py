"""Command line in the manner of the reference's `kipp`
(/root/reference/src/kipp_cli.c:571-610 options, :1145-1217 output): evaluate a
prompt, generate `--decode` tokens, print the final top-N logits and one
KIPP_METRIC line.  The prompt is token ids (this engine has no tokenizer).

    python -m kipp_amd.cli --model DIR --tokens 5,17,3 --decode 16
    python -m kipp_amd.cli --model DIR --ppl tokens.u32 --ppl-window 512
    python -m kipp_amd.cli --write-random DIR --random tiny-a --seed-weights 7
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
    ap.add_argument("--max-step-tokens", type=int, default=2048, help="token budget of one step")
    ap.add_argument("--random", metavar="SHAPE", help="with --write-random: named shape (tiny-a, tiny-b, qwen3-4b, ...)")
    ap.add_argument("--seed-weights", type=int, default=0, help="seed of the random weights")
    ap.add_argument("--write-random", metavar="DIR", help="write a random-weights model folder and exit")
    ap.add_argument("--weights-dtype", choices=["bfloat16", "float32"], default="bfloat16")
    return ap


def run_perplexity(args) -> int:
    """Windows of `--ppl-window` tokens that do not overlap, each from an empty
    context, no burn-in; a window of W tokens scores its W - 1 targets
    (/root/reference/src/kipp_cli.c:646-801: the protocol and the lines printed)."""
    import torch
    from .engine import Engine, StepEntry
    with open(args.ppl, "rb") as f:
        raw = f.read()
    if len(raw) % 4:
        raise SystemExit(f"kipp: ppl: '{args.ppl}' is not a uint32 token file")
    stream = list(struct.unpack(f"<{len(raw) // 4}I", raw))
    if args.ppl_limit:
        stream = stream[:args.ppl_limit]
    if len(stream) < 2:
        raise SystemExit("kipp: ppl: need at least two tokens to score")
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
                targets = torch.tensor([tokens[at + r + 1] for r in rows], device=logits.device)
                wide = logits.double()
                nll += float((torch.logsumexp(wide, dim=-1) - wide.gather(1, targets[:, None])[:, 0]).sum())
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
    if not args.model:
        raise SystemExit("kipp: --model is required")
    if args.ppl:
        return run_perplexity(args)
    if not 1 <= args.top <= 100:
        raise SystemExit("kipp: --top must be between 1 and 100")
    if args.seed == 0:
        raise SystemExit("kipp: --seed must be nonzero")
    tokens = _parse_tokens(args)
    if not tokens:
        raise SystemExit("kipp: the prompt is empty")

    import torch
    from .engine import Engine, StepEntry
    from .engine.scheduler import Request, Scheduler
    from .sampling import SampleParams

    capacity = len(tokens) + args.decode
    pages = args.kv_pages or -(-capacity // args.page)
    engine = Engine.from_folder(args.model, dtype=args.dtype, page_size=args.page, num_pages=pages, max_requests=1)
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
