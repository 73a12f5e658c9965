"""The scheduler above the step function: it admits requests, cuts prompts
into portions under a token budget, decodes, finishes and frees.

Policy (the reference's server loop lifted out of its HTTP code,
/root/reference/src/kipp_server.c:1623-1893 admission, :1900-2125 stepping):

* Waiting requests are admitted strictly in arrival order; the first that does
  not fit blocks those behind it.
* Requests publish their full pages as they go.  A waiting request whose prompt
  begins like that of a request still running its prompt waits until those pages
  are published and then adopts them instead of computing them again.
* A request is refused at `add` if its prompt plus `max_new_tokens` exceeds the
  model's positions, or if it could never fit the page pool even alone.
* Pages are reserved at admission: a request is admitted only if every pool
  still has its worst-case need plus what every running request may still
  claim.  So pages never run out in the middle of a generation; when they are
  short, requests wait (pressure delays, never corrupts).
* One step = one call of the step function: every decoding request gives its
  one next token first, then the remaining token budget goes to portions of
  prompts in arrival order; the last portion of a prompt asks for the logits of
  its last place.
* A sampled stop token ends the request and is neither kept nor fed back;
  reaching `max_new_tokens` ends it without running the last token.
* A step that fails (the step function raises) fails as a unit: every request that had
  tokens in it ends with `finish_reason="failed"` and its error, its pages go back, and
  the queue moves on (/root/reference/src/kipp_server.c:2081-2088).  The engine has
  already undone the step's own reservations by then.
* While every running request decodes and none waits, the scheduler runs one step
  ahead of what it knows (`lookahead`): the next step is launched with the tokens
  still on the device, and the tokens of the step before are read while it runs,
  so the GPU never waits for the host.  A request that a stop token ends has then
  run one step in vain; its cache goes back whole.  The tokens are the same.
"""
from __future__ import annotations

import time
from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, List, Optional, Sequence, Tuple

import numpy as np

from ..sampling import SampleParams, XorShift64Star
from .batch import StepEntry

RECENT_WINDOW = 64  # tokens the penalties look back over (/root/reference/src/kipp_server.c:848)


class RequestRefused(ValueError):
    """The request can never run on this engine."""


@dataclass
class Request:
    id: object
    prompt: Sequence[int]
    max_new_tokens: int
    params: SampleParams = field(default_factory=SampleParams)
    seed: int = 1
    stop_tokens: Tuple[int, ...] = ()
    # progress
    state: str = "waiting"          # waiting, prefill, decode, finished
    fed: int = 0                    # prompt tokens already in the cache
    output: List[int] = field(default_factory=list)
    next_token: Optional[int] = None
    finish_reason: Optional[str] = None
    rng: Optional[XorShift64Star] = None
    recent: Deque[int] = field(default_factory=lambda: deque(maxlen=RECENT_WINDOW))
    arrived: float = 0.0
    admitted_at: Optional[float] = None
    first_token_at: Optional[float] = None
    finished_at: Optional[float] = None
    error: Optional[str] = None     # what the step function said when a step with this request in it failed

    @property
    def budget_tokens(self) -> int:
        """Most tokens the cache will ever hold for it: the last sampled token is never run."""
        return len(self.prompt) + max(0, self.max_new_tokens - 1)


@dataclass
class SchedulerStats:
    requests: int = 0
    refused: int = 0
    finished: int = 0
    prompt_tokens: int = 0
    generated_tokens: int = 0
    prefix_tokens_reused: int = 0
    steps: int = 0
    waits_for_pages: int = 0
    waits_for_prefix: int = 0
    # what the reference's server counts beside these (/root/reference/src/kipp_server.c:71-84): requests that a
    # failed step ended, and sums of seconds with their counts, so that a reader derives averages and rates
    failed: int = 0
    failed_steps: int = 0
    queue_wait_seconds_sum: float = 0.0     # arrival -> admission
    queue_wait_count: int = 0
    ttft_seconds_sum: float = 0.0           # arrival -> first token known
    ttft_count: int = 0
    decode_seconds_sum: float = 0.0         # first token -> finish, of requests that ended without failing


def _rows_on_device(engine, tokens, rows):
    """tokens[rows] (int32 on the device), picked by the engine's own gather kernel."""
    import torch
    rt = engine.rt
    index = torch.tensor(list(rows), dtype=torch.int32).pin_memory().to(rt.device, non_blocking=True)
    return rt.ops.gather_rows(tokens.view(-1, 1), index, rt.empty((len(rows), 1), torch.int32)).view(-1)


class _PicksRows:
    """Some rows of a choice that is still on its way."""

    def __init__(self, engine, picks, rows):
        self.engine, self.picks, self.rows = engine, picks, list(rows)

    @property
    def device(self):
        return _rows_on_device(self.engine, self.picks.device, self.rows)

    def result(self):
        chosen = self.picks.result()
        return [chosen[i] for i in self.rows]


class Scheduler:
    def __init__(self, engine, max_step_tokens: int = 2048, prefill_chunk: int = 512, max_running: int = 64,
                 lookahead: bool = True, on_logits=None):
        """`on_logits(requests, logits)`: called after every step that asked for logits, before tokens are
        chosen from them, with the requests whose rows they are, in order, and the float32 tensor
        [rows, vocab] on the device.  The tensor may be overwritten by the next step: a caller that wants to
        keep a row copies it."""
        if max_step_tokens < 1 or prefill_chunk < 1 or max_running < 1:
            raise ValueError("budgets must be positive")
        self.on_logits = on_logits
        # running ahead needs an engine that takes a step's tokens from the device
        self.lookahead = lookahead and getattr(engine, "graphs", None) is not None
        self._ahead = None          # (requests, Picks) of the step launched last, its choice not yet read
        self.engine = engine
        self.cache = engine.cache
        self.max_step_tokens = max_step_tokens
        self.prefill_chunk = prefill_chunk
        self.max_running = min(max_running, self.cache.max_requests)
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []
        self.finished: Dict[object, Request] = {}
        self.stats = SchedulerStats()
        self._common: Dict[Tuple[object, object], int] = {}

    # -- page arithmetic -----------------------------------------------------------
    @property
    def _largest_step(self) -> int:
        """Most tokens one request brings in a step."""
        return min(self.prefill_chunk, self.max_step_tokens)

    def _still_to_claim(self, req: Request) -> List[int]:
        """Pages a running request may still claim in each group, beyond those it holds."""
        rc = self.cache.requests[req.id]
        return self.cache.pages_bound(rc, req.budget_tokens, self._largest_step)

    # -- interface -------------------------------------------------------------------
    def add(self, req: Request) -> None:
        # an id names one request at a time: a second one would fail at admission, stay first in line
        # and block the queue for good, and its result would replace the first one's
        if (req.id in self.cache.requests or req.id in self.finished
                or any(other.id == req.id for other in self.waiting) or any(other.id == req.id for other in self.running)):
            self.stats.refused += 1
            raise RequestRefused(f"request id {req.id!r} is already waiting, running, open in the engine, or finished and not collected")
        if len(req.prompt) == 0:
            raise RequestRefused(f"request {req.id!r}: empty prompt")
        if req.max_new_tokens < 0:
            raise RequestRefused(f"request {req.id!r}: max_new_tokens must be >= 0")
        if len(req.prompt) + req.max_new_tokens > self.cache.max_position:
            self.stats.refused += 1
            raise RequestRefused(
                f"request {req.id!r}: prompt {len(req.prompt)} + max_new_tokens {req.max_new_tokens} "
                f"exceeds the model's {self.cache.max_position} positions")
        for g, most in zip(self.cache.groups, self.cache.pages_bound(None, req.budget_tokens, self._largest_step)):
            if most > g.pool.num_pages:
                self.stats.refused += 1
                raise RequestRefused(f"request {req.id!r}: needs {most} pages of group {g.index}, more than its pool's {g.pool.num_pages}")
        for t in req.prompt:
            if not 0 <= int(t) < self.engine.vocab_size:
                self.stats.refused += 1
                raise RequestRefused(f"request {req.id!r}: token {t} is outside the vocabulary")
        req.params.validate()
        if not req.params.greedy:
            req.rng = XorShift64Star(req.seed if req.seed != 0 else 1)   # 0 mapped to 1 (kipp_server.c:1852-1862)
        req.state = "waiting"
        req.arrived = time.monotonic()
        self.waiting.append(req)
        self.stats.requests += 1

    def cancel(self, request_id) -> None:
        self._drain()
        for req in list(self.waiting):
            if req.id == request_id:
                self.waiting.remove(req)
                self._finish(req, "cancelled", opened=False)
                return
        for req in self.running:
            if req.id == request_id:
                self._finish(req, "cancelled")
                return

    @property
    def idle(self) -> bool:
        return not self.waiting and not self.running

    # -- admission ---------------------------------------------------------------------
    def _worth_waiting(self, req: Request) -> bool:
        """Is a running request about to publish pages that `req` could adopt?"""
        if not self.cache.share:
            return False
        page = self.cache.page_size
        for other in self.running:
            if other.state != "prefill":
                continue
            key = (req.id, other.id)
            if key not in self._common:
                n = min(len(req.prompt) - 1, len(other.prompt))
                a, b = np.asarray(req.prompt[:n]), np.asarray(other.prompt[:n])
                differ = np.nonzero(a != b)[0]
                self._common[key] = (int(differ[0]) if len(differ) else n) // page
            if self._common[key] > other.fed // page:
                return True
        return False

    def _admit(self) -> None:
        while self.waiting and len(self.running) < self.max_running:
            req = self.waiting[0]
            if self._worth_waiting(req):
                self.stats.waits_for_prefix += 1
                return
            rc = self.cache.open(req.id, req.prompt, publish_early=True)   # adopts the longest known beginning
            need = self.cache.pages_bound(rc, req.budget_tokens, self._largest_step)
            promised = [0] * len(self.cache.groups)
            for other in self.running:
                for g, n in enumerate(self._still_to_claim(other)):
                    promised[g] += n
            free = self.cache.free_pages()
            if any(need[g] + promised[g] > free[g] for g in range(len(free))):
                self.cache.close(req.id)                   # undo; stays first in line
                self.stats.waits_for_pages += 1
                return
            self.waiting.popleft()
            req.admitted_at = time.monotonic()
            self.stats.queue_wait_seconds_sum += req.admitted_at - req.arrived
            self.stats.queue_wait_count += 1
            req.fed = rc.length
            self.stats.prefix_tokens_reused += rc.length
            req.state = "prefill"
            self.running.append(req)

    # -- one step ------------------------------------------------------------------------
    def plan(self) -> List[Tuple[Request, List[int], List[int]]]:
        """(request, tokens, want) of the next step: decode tokens first, then
        portions of prompts in arrival order while the token budget lasts."""
        budget = self.max_step_tokens
        plan = []
        for req in self.running:
            if req.state == "decode" and budget > 0:
                plan.append((req, [req.next_token], [0]))
                budget -= 1
        for req in self.running:
            if req.state != "prefill" or budget <= 0:
                continue
            left = len(req.prompt) - req.fed
            n = min(self.prefill_chunk, left, budget)
            tokens = [int(t) for t in req.prompt[req.fed:req.fed + n]]
            plan.append((req, tokens, [n - 1] if n == left else []))
            budget -= n
        return plan

    def step(self) -> List[Tuple[object, int]]:
        """Admit, run one batch, sample.  Returns the (request id, token) pairs
        that became known in this step."""
        if self._ahead is not None:
            if not self.waiting:
                return self._step_ahead()
            produced = self._drain()                       # someone waits: back to steps that may bring prompts
        else:
            produced = []
        self._admit()
        plan = self.plan()
        if not plan:
            return produced
        entries = [StepEntry(req.id, tokens, want) for req, tokens, want in plan]
        try:
            logits = self.engine.step(entries, borrow=True)      # read by `choose` before the next step is launched
        except Exception as error:                               # noqa: BLE001 - whatever the step function raises fails the batch
            self._fail([req for req, _, _ in plan], error)
            return produced
        self.stats.steps += 1
        sampling = [req for req, _, want in plan if want]
        self._tell(sampling, logits)
        for req, tokens, want in plan:
            if req.state == "prefill":
                req.fed += len(tokens)
                self.stats.prompt_tokens += len(tokens)
        if sampling:
            if self._may_run_ahead(plan, sampling):
                self._ahead = (sampling, self.engine.choose(logits, sampling, wait=False))
                return produced
            chosen = self.engine.choose(logits, sampling)
            for req, token in zip(sampling, chosen):
                self._accept(req, int(token), produced)
        return produced

    def _tell(self, requests, logits) -> None:
        if self.on_logits is not None and logits is not None and requests:
            self.on_logits(requests, logits)

    # -- one step ahead --------------------------------------------------------------------
    def _may_run_ahead(self, plan, sampling) -> bool:
        return (self.lookahead and not self.waiting and len(sampling) == len(plan) == len(self.running)
                and all(req.state == "decode" and not req.params.changes_logits for req in sampling)
                and self.engine.graphs.applies([StepEntry(req.id, [0], [0]) for req in sampling]))

    def _step_ahead(self) -> List[Tuple[object, int]]:
        """The step launched last has not told its tokens yet.  Launch the next one
        from them where they are, then read them and settle the last step."""
        reqs, picks = self._ahead
        # requests that the length ends with the token still on its way need no further step
        go_on = [i for i, req in enumerate(reqs) if len(req.output) + 1 < req.max_new_tokens]
        nxt = None
        if go_on:
            cont = [reqs[i] for i in go_on]
            tokens = picks.device if len(go_on) == len(reqs) else _rows_on_device(self.engine, picks.device, go_on)
            try:
                logits = self.engine.step([StepEntry(req.id, [0], [0]) for req in cont], device_tokens=tokens, borrow=True)
            except Exception as error:                           # noqa: BLE001
                # the step before still holds good: its tokens are read and kept, then its requests fail with this one
                produced = self._drain()
                self._fail([req for req in cont if req.state != "finished"], error)
                return produced
            self._tell(cont, logits)
            self.stats.steps += 1
            nxt = (cont, self.engine.choose(logits, cont, wait=False))
        produced: List[Tuple[object, int]] = []
        chosen = picks.result()
        for req, token in zip(reqs, chosen):
            self._accept(req, int(token), produced)
        if nxt is not None:
            cont, ahead = nxt
            alive = []
            for i, req in enumerate(cont):
                if req.state == "decode":
                    self.engine.commit(req.id, [req.next_token])   # what the step just launched was fed
                    alive.append(i)
            # a request that its token has just ended ran that step in vain: its row is left out from here on
            if len(alive) == len(cont):
                self._ahead = nxt
            elif alive:
                self._ahead = ([cont[i] for i in alive], _PicksRows(self.engine, ahead, alive))
            else:
                self._ahead = None
        else:
            self._ahead = None
        return produced

    def _drain(self) -> List[Tuple[object, int]]:
        """Read the tokens of the step launched last and go back to knowing everything."""
        produced: List[Tuple[object, int]] = []
        if self._ahead is not None:
            reqs, picks = self._ahead
            self._ahead = None
            for req, token in zip(reqs, picks.result()):
                self._accept(req, int(token), produced)
        return produced

    def _fail(self, requests, error) -> None:
        """The step these requests had tokens in failed as a unit: each of them ends, failed, and its
        pages and slot go back; requests that were not in the step go on
        (/root/reference/src/kipp_server.c:2081-2088)."""
        self.stats.failed_steps += 1
        for req in requests:
            req.error = f"{type(error).__name__}: {error}"
            self._finish(req, "failed")

    def _accept(self, req: Request, token: int, produced) -> None:
        if req.max_new_tokens == 0:
            self._finish(req, "length")
            return
        if token in req.stop_tokens:
            self._finish(req, "stop")                      # not kept, not fed back
            return
        now = time.monotonic()
        if req.first_token_at is None:
            req.first_token_at = now
            self.stats.ttft_seconds_sum += now - req.arrived
            self.stats.ttft_count += 1
        req.output.append(token)
        req.recent.append(token)
        produced.append((req.id, token))
        self.stats.generated_tokens += 1
        if len(req.output) >= req.max_new_tokens:
            self._finish(req, "length")
            return
        req.next_token = token
        req.state = "decode"

    def _finish(self, req: Request, reason: str, opened: bool = True) -> None:
        req.state = "finished"
        req.finish_reason = reason
        req.finished_at = time.monotonic()
        if req in self.running:
            self.running.remove(req)
        if opened and req.id in self.cache.requests:
            self.engine.close(req.id)
        self.finished[req.id] = req
        self.stats.finished += 1
        if reason == "failed":
            self.stats.failed += 1
        elif req.first_token_at is not None:
            self.stats.decode_seconds_sum += req.finished_at - req.first_token_at
        self._common = {k: v for k, v in self._common.items() if req.id not in k}

    def run(self, max_steps: Optional[int] = None) -> Dict[object, Request]:
        """Step until every request has finished."""
        steps = 0
        while not self.idle:
            before = (len(self.waiting), len(self.running), self.stats.steps)
            self.step()
            steps += 1
            if max_steps is not None and steps >= max_steps:
                break
            if not self.running and self.waiting and (len(self.waiting), 0, self.stats.steps) == before:
                raise RuntimeError("scheduler stalled: a waiting request cannot be admitted although nothing is running")
        return self.finished
