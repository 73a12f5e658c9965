"""The engine: a model, its cache manager, and ONE step function.

`step(entries)` runs exactly the tokens it is given, as one batch, from the
cache that earlier steps left: portions of prompts beside single decoded
tokens, cut anywhere.  It returns the float32 logits at the wanted places in
the order of the entries and of their `want` lists
(/root/reference/src/kipp.c:3984-4082 is the reference's batched call; there
one row per item, here any places).
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch

from ..cache import CacheManager, OutOfPages
from ..runtime import Runtime
from .batch import StepEntry, build_batch
from .graphs import DecodeGraphs
from .model import Model, load_model


class Engine:
    def __init__(self, model: Model, page_size: int = 16, num_pages: Optional[int] = None,
                 max_tokens: Optional[int] = None, max_requests: int = 64, share_prefixes: bool = True,
                 use_graphs: bool = True):
        """The pool of every cache group has `num_pages` pages, or as many as
        hold `max_tokens` tokens."""
        if num_pages is None:
            if max_tokens is None:
                raise ValueError("give num_pages or max_tokens")
            num_pages = (max_tokens + page_size - 1) // page_size
        self.model = model
        self.rt: Runtime = model.rt
        # what this model launches is compiled now, all at once, if it is not built yet
        from ..csrc import build
        from ..csrc.variants import model_variants
        build.build_all(model_variants(model.spec, self.rt.dtype))
        self.vocab_size = model.spec.vocab_size
        self.cache = CacheManager(model.kv_needs(), model.state_needs(), page_size, num_pages, max_requests,
                                  model.spec.max_position, runtime=self.rt, share_prefixes=share_prefixes)
        self.graphs = DecodeGraphs(self) if use_graphs else None

    @classmethod
    def from_folder(cls, model_dir: str, dtype: str = "bfloat16", device: str = "cuda:0", **kw) -> "Engine":
        return cls(load_model(model_dir, Runtime(dtype, device)), **kw)

    # -- requests ---------------------------------------------------------------------
    def open(self, request_id, prompt: Optional[Sequence[int]] = None, publish_early: bool = False):
        return self.cache.open(request_id, prompt, publish_early)

    def close(self, request_id) -> None:
        self.cache.close(request_id)

    def length(self, request_id) -> int:
        return self.cache.requests[request_id].length

    # -- the step ---------------------------------------------------------------------
    def step(self, entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        """Run one batch.  Requests not yet open are opened.  Raises OutOfPages
        (nothing changed) when the pools cannot hold the step."""
        if not entries:
            return None
        seen = set()
        requests = []
        for e in entries:
            if e.request in seen:
                raise ValueError(f"request {e.request!r} appears twice in one step")
            seen.add(e.request)
            if len(e.tokens) == 0:
                raise ValueError(f"request {e.request!r}: an entry needs at least one token")
            if min(e.tokens) < 0 or max(e.tokens) >= self.vocab_size:
                bad = [t for t in e.tokens if not 0 <= int(t) < self.vocab_size][0]
                raise ValueError(f"request {e.request!r}: token {bad} is outside the vocabulary of {self.vocab_size}")
            if e.want and (min(e.want) < 0 or max(e.want) >= len(e.tokens)):
                bad = [w for w in e.want if not 0 <= int(w) < len(e.tokens)][0]
                raise ValueError(f"request {e.request!r}: wanted place {bad} is not among its {len(e.tokens)} tokens")
        opened = []
        try:
            for e in entries:
                if e.request not in self.cache.requests:
                    self.cache.open(e.request)
                    opened.append(e.request)
                requests.append(self.cache.requests[e.request])
            self.cache.reserve([(r, len(e.tokens)) for r, e in zip(requests, entries)])
        except Exception:
            for rid in opened:
                self.cache.close(rid)
            raise
        try:
            if self.graphs is not None and self.graphs.applies(entries):
                logits = self.graphs.run(entries, requests)
            else:
                batch = build_batch(entries, requests, len(self.cache.groups), self.rt.device)
                logits = self.model.forward(batch, self.cache)
        except Exception:
            for r in requests:                  # the step did not happen: its pages go back
                self.cache.trim(r)
            for rid in opened:
                self.cache.close(rid)
            raise
        for r, e in zip(requests, entries):
            self.cache.commit(r, e.tokens)
        return logits

    # -- token choice -------------------------------------------------------------------
    def choose(self, logits: torch.Tensor, requests: Sequence[object]) -> List[int]:
        """One token for each row of `logits`; `requests[i]` carries the row's
        sampling parameters, generator and recent tokens.  Rows are chosen on the
        device in one launch (greedy and temperature rows alike; the uniform draw
        of a temperature row comes from its request's generator on the host).
        Only rows whose logits are changed first (bias, penalties) go through the
        host sampler."""
        from ..sampling import sample
        rows = logits.shape[0]
        if rows != len(requests):
            raise ValueError("one request for each row of logits")
        on_host = [i for i, r in enumerate(requests) if r.params.changes_logits]
        temperature, top_k, top_p, min_p, uniform = [], [], [], [], []
        for i, req in enumerate(requests):
            p = req.params
            sampled = not p.greedy and i not in on_host
            if sampled:
                p.validate()
            temperature.append(float(p.temperature) if sampled else 0.0)
            top_k.append(int(p.top_k) if sampled else 0)
            top_p.append(float(p.top_p) if sampled else 1.0)
            min_p.append(float(p.min_p) if sampled else 0.0)
            uniform.append(req.rng.uniform() if sampled else 0.0)
        dev = self.rt.device
        f32 = lambda v: torch.tensor(v, dtype=torch.float32, device=dev)
        picked = self.rt.ops.sample(logits, f32(temperature), torch.tensor(top_k, dtype=torch.int32, device=dev),
                                    f32(top_p), f32(min_p), torch.tensor(uniform, dtype=torch.float64, device=dev),
                                    self.rt.empty((rows,), torch.int32)).cpu().tolist()
        for i in on_host:
            req = requests[i]
            picked[i] = sample(logits[i].cpu().numpy(), req.params, req.rng, list(req.recent))
        return picked
