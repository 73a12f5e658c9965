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

import numpy as np
import torch

from ..cache import CacheManager
from ..runtime import Runtime
from .batch import StepEntry, build_batch
from .graphs import DecodeGraphs
from .model import Model, load_model


class Engine:
    def __init__(self, model: Model, page_size: int = 16, num_pages: Optional[int] = None,
                 max_tokens: Optional[int] = None, max_requests: int = 64, share_prefixes: bool = True,
                 use_graphs: bool = True, page_order=None, max_position: Optional[int] = None):
        """The pool of every cache group has `num_pages` pages, or as many as
        hold `max_tokens` tokens.  `page_order`: the order in which fresh pools hand
        out their pages (a permutation; results must not depend on it).  `max_position`:
        the longest context a request may reach (default: the model's own limit)."""
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
                                  max_position or model.spec.max_position, runtime=self.rt, share_prefixes=share_prefixes,
                                  page_order=page_order)
        self.graphs = DecodeGraphs(self) if use_graphs else None
        self._uncommitted = {}      # request -> tokens of a step run from device_tokens and not recorded yet

    @classmethod
    def from_folder(cls, model_dir: str, dtype: str = "bfloat16", device: str = "cuda:0", **kw) -> "Engine":
        return cls(load_model(model_dir, Runtime(dtype, device)), **kw)

    # -- requests ---------------------------------------------------------------------
    def open(self, request_id, prompt: Optional[Sequence[int]] = None, publish_early: bool = False):
        return self.cache.open(request_id, prompt, publish_early)

    def close(self, request_id) -> None:
        self._uncommitted.pop(request_id, None)     # a step that was never recorded leaves nothing behind
        self.cache.close(request_id)

    def warm_up(self, rows: Sequence[int] = (2048, 512, 256)) -> None:
        """Run a prompt portion of each of these sizes on a request of its own and forget it: what a shape decides at
        its first use (the cut of a prompt product is timed once a process) is decided now, not inside a request's
        first step.  Sizes that the pools or the positions cannot hold are left out; nothing is published."""
        share, self.cache.share = self.cache.share, False
        try:
            for n in rows:
                fits = 0 < n <= self.cache.max_position and all(-(-n // g.page_size) <= g.pool.free_count for g in self.cache.groups)
                if not fits or not self.cache.free_slots:
                    continue
                name = ("warm-up", n)
                try:
                    self.step([StepEntry(name, [0] * n, [n - 1])])
                finally:
                    if name in self.cache.requests:
                        self.close(name)
        finally:
            self.cache.share = share

    def length(self, request_id) -> int:
        return self.cache.requests[request_id].length

    # -- the step ---------------------------------------------------------------------
    def step(self, entries: Sequence[StepEntry], device_tokens: Optional[torch.Tensor] = None,
             borrow: bool = False) -> Optional[torch.Tensor]:
        """Run one batch.  Requests not yet open are opened.  Raises OutOfPages
        (nothing changed) when the pools cannot hold the step.

        With `borrow` the logits may lie in a buffer of the engine's own that a later
        step overwrites: for a caller that is done with them (has launched what reads
        them) before it calls `step` again, and saves a copy of [entries, vocab] floats.

        With `device_tokens` (int32 [entries] on the device) every entry brings one
        token that the host does not know yet, for instance the choice of the step
        before, which is still running: the step reads entry i's token from
        `device_tokens[i]` (the values in `entries` are ignored), and what the
        cache records is put off until `commit(request, tokens)` tells it, which
        must happen before the request's next step."""
        if not entries:
            return None
        if device_tokens is not None:
            if self.graphs is None or not self.graphs.applies(entries):
                raise ValueError("tokens on the device need a step of single tokens that is replayed as a graph")
            if device_tokens.dtype != torch.int32 or device_tokens.numel() != len(entries) \
                    or device_tokens.device != self.rt.device:
                raise ValueError("device_tokens must be int32 [entries] on the engine's device")
        seen = set()
        requests = []
        for e in entries:
            if e.request in seen:
                raise ValueError(f"request {e.request!r} appears twice in one step")
            if e.request in self._uncommitted:
                raise ValueError(f"request {e.request!r}: the tokens of its last step are not recorded yet (commit)")
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
                logits = self.graphs.run(entries, requests, device_tokens, borrow)
            else:
                batch = build_batch(entries, requests, len(self.cache.groups), self.rt.device)
                logits = self.model.forward(batch, self.cache)
        except Exception:
            self._after_failed_launches()
            for r in requests:                  # the step did not happen: its pages go back
                self.cache.trim(r)
            for rid in opened:
                self.cache.close(rid)
            raise
        if device_tokens is None:
            for r, e in zip(requests, entries):
                self.cache.commit(r, e.tokens)
        else:
            for r in requests:
                self._uncommitted[r.id] = 1
        return logits

    def _after_failed_launches(self) -> None:
        """A forward pass that stopped half way may have left counts of finished splits above zero in a decode
        workspace that outlives the step (a recorded shape keeps its own): the next launch on it would merge early or
        never.  They are set back to zero by a kernel; a recording that was under way is dropped with its shape."""
        if self.graphs is None:
            return
        for key, graph in list(self.graphs.graphs.items()):
            if graph.graph is None and graph.eager_runs >= 2:
                del self.graphs.graphs[key]                 # failed while recording: made anew when the shape returns
                continue
            for name, space in graph.batch.host.items():
                if isinstance(name, tuple) and name and name[0] == "decode_workspace" and len(space) > 2 and space[2] is not None:
                    try:
                        self.rt.ops.fill_zero(space[2])
                    except Exception:                       # noqa: BLE001 - the device itself is gone: nothing left to tidy
                        return

    def commit(self, request_id, tokens: Sequence[int]) -> None:
        """The tokens of a step that ran from `device_tokens` are known now."""
        if self._uncommitted.pop(request_id, 0) != len(tokens):
            raise ValueError(f"request {request_id!r} has no step of {len(tokens)} tokens waiting to be recorded")
        self.cache.commit(self.cache.requests[request_id], tokens)

    # -- token choice -------------------------------------------------------------------
    def choose(self, logits: torch.Tensor, requests: Sequence[object], wait: bool = True):
        """One token for each row of `logits`; `requests[i]` carries the row's
        sampling parameters, generator and recent tokens.  Rows are chosen on the
        device in one launch (greedy and temperature rows alike; the uniform draw
        of a temperature row comes from its request's generator on the host).
        Rows whose logits are changed first (bias, penalties over the request's
        recent tokens) are changed where they lie, by a kernel that walks each
        row's few entries in the host sampler's order (`logits` is overwritten
        there).  With `wait` false the choice is not waited for: the result
        is a `Picks` whose `device` tensor can feed the next step at once and whose
        `result()` gives the tokens when the host needs them (the recent tokens
        of a row with penalties must then be known: the scheduler waits for them)."""
        from ..sampling import logit_change_entries
        rows = logits.shape[0]
        if rows != len(requests):
            raise ValueError("one request for each row of logits")
        if any(r.params.changes_logits for r in requests):
            self._adjust_logits(logits, requests, logit_change_entries)
        picked = self.rt.empty((rows,), torch.int32)
        if all(r.params.greedy for r in requests):
            self.rt.ops.argmax(logits, picked)
        else:
            # all parameters in one pinned buffer and one copy: [temperature | top_p | min_p | top_k | uniform (8 bytes)]
            # (gathered in lists and written field by field: an assignment to one element of a tensor costs a microsecond)
            fields = ([], [], [], [], [])
            for req in requests:
                p = req.params
                if p.greedy:
                    row = (0.0, 1.0, 0.0, 0, 0.0)
                else:
                    p.validate()
                    row = (float(p.temperature), float(p.top_p), float(p.min_p), int(p.top_k), req.rng.uniform())
                for field, value in zip(fields, row):
                    field.append(value)
            packed = np.empty(rows * 24, dtype=np.uint8)
            packed[:rows * 12].view(np.float32)[:] = fields[0] + fields[1] + fields[2]
            packed[rows * 12:rows * 16].view(np.int32)[:] = fields[3]
            packed[rows * 16:].view(np.float64)[:] = fields[4]
            dev = torch.from_numpy(packed).pin_memory().to(self.rt.device, non_blocking=True)
            d32 = dev[:rows * 12].view(torch.float32)
            self.rt.ops.sample(logits, d32[:rows], dev[rows * 12:rows * 16].view(torch.int32), d32[rows:2 * rows],
                               d32[2 * rows:], dev[rows * 16:].view(torch.float64), picked)
        if not wait:
            return Picks(picked)
        return picked.cpu().tolist()

    def _adjust_logits(self, logits: torch.Tensor, requests: Sequence[object], entries_of) -> None:
        """Bias and penalties of every row that has them, in one launch: the rows' entries and parameters go up in one
        pinned buffer of 4-byte words [begin (rows + 1) | biases | tokens | values | repetition | presence | frequency]."""
        rows, vocab = logits.shape
        per_row = [entries_of(r.params, list(r.recent), vocab) if r.params.changes_logits else ([], [], 0) for r in requests]
        total = sum(len(tokens) for tokens, _, _ in per_row)
        words = 2 * rows + 1 + 2 * total + 3 * rows
        at_value = 2 * rows + 1 + total
        begin, biases, token, value = [], [], [], []
        for tokens, values, n_bias in per_row:
            begin.append(len(token))
            biases.append(n_bias)
            token += tokens
            value += values
        begin.append(len(token))
        at = len(token)
        packed = np.empty(words, dtype=np.int32)
        packed[:at_value] = begin + biases + token
        packed[at_value:].view(np.float32)[:] = (value + [float(r.params.repetition_penalty) for r in requests]
                                                 + [float(r.params.presence_penalty) for r in requests]
                                                 + [float(r.params.frequency_penalty) for r in requests])
        dev = torch.from_numpy(packed).pin_memory().to(self.rt.device, non_blocking=True)
        dev_float = dev.view(torch.float32)
        self.rt.ops.adjust_logits(logits, dev[:rows + 1], dev[rows + 1:2 * rows + 1], dev[2 * rows + 1:at_value],
                                  dev_float[at_value:at_value + total], dev_float[at_value + total:at_value + total + rows],
                                  dev_float[at_value + total + rows:at_value + total + 2 * rows], dev_float[at_value + total + 2 * rows:])


class Picks:
    """Tokens chosen on the device and on their way to the host."""

    def __init__(self, device: torch.Tensor):
        self.device = device
        self.host = torch.empty(device.shape, dtype=device.dtype).pin_memory()
        self.host.copy_(device, non_blocking=True)
        self.ready = torch.cuda.Event()
        self.ready.record()

    def result(self) -> List[int]:
        self.ready.synchronize()
        return self.host.tolist()
