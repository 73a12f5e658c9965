"""The Python entry point: token ids in, token ids out.

    from kipp_amd import generate
    outputs = generate("model_dir", [[1, 2, 3], [4, 5]], max_new_tokens=16)

Option names and meanings are those of the reference's command line
(/root/reference/src/kipp_cli.c:571-610): temperature 0 is greedy argmax, top_p
in (0, 1], top_k 0 = off, min_p 0 = off, seed nonzero.
"""
from __future__ import annotations

from typing import Optional, Sequence

from .engine import Engine
from .engine.scheduler import Request, Scheduler
from .sampling import SampleParams


def generate(model, prompts: Sequence[Sequence[int]], max_new_tokens: int = 16, temperature: float = 0.0,
             top_p: float = 1.0, top_k: int = 0, min_p: float = 0.0, seed: int = 1,
             stop_tokens: Optional[Sequence[int]] = None, dtype: str = "bfloat16", page_size: int = 16,
             kv_pages: Optional[int] = None, max_step_tokens: int = 2048, prefill_chunk: int = 512,
             return_requests: bool = False):
    """Generate for every prompt (a list of token ids) under continuous batching.
    `model` is a model folder or an `Engine`.  Request i samples with seed + i."""
    if isinstance(model, Engine):
        engine = model
    else:
        need = sum(-(-(len(p) + max_new_tokens) // page_size) for p in prompts)
        engine = Engine.from_folder(model, dtype=dtype, page_size=page_size,
                                    num_pages=kv_pages or max(need, 1), max_requests=max(len(prompts), 1))
    stops = tuple(stop_tokens) if stop_tokens is not None else tuple(engine.model.spec.stop_tokens)
    sched = Scheduler(engine, max_step_tokens=max_step_tokens, prefill_chunk=prefill_chunk,
                      max_running=engine.cache.max_requests)
    ids = []
    for i, prompt in enumerate(prompts):
        rid = f"gen-{id(sched)}-{i}"
        ids.append(rid)
        sched.add(Request(rid, list(prompt), max_new_tokens,
                          SampleParams(temperature=temperature, top_p=top_p, top_k=top_k, min_p=min_p),
                          seed=seed + i, stop_tokens=stops))
    done = sched.run()
    if return_requests:
        return [done[r] for r in ids]
    return [list(done[r].output) for r in ids]
