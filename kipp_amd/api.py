"""The Python entry point in the manner of the reference's public interface
(/root/reference/src/kipp.h:99-295): a model, sessions that own a bounded
timeline of keys and values, evaluation of one session or of several in one
call, prefix adoption, truncation, and the sampler.  Names and meanings follow
kipp.h; handles are objects, errors are `KippError` with the reference's codes.

    model = Model.open("model_dir", dtype="bfloat16", kv_pool_blocks=4096)
    s = model.session_create(capacity=512)
    logits = s.eval([5, 17, 3])             # float32 row of the last token
    token = sample(logits, temperature=0.0)
"""
from __future__ import annotations

import itertools
from dataclasses import dataclass
from typing import List, Optional, Sequence

import numpy as np

from .cache import OutOfPages, OutOfSlots
from .engine import Engine, StepEntry
from .sampling import SampleParams, XorShift64Star
from .sampling import sample as _sample

EVAL_BATCH_LIMIT = 32   # /root/reference/src/kipp.h:245

# /root/reference/src/kipp.h:55-69
ERROR_ARGUMENT, ERROR_IO, ERROR_FORMAT, ERROR_UNSUPPORTED, ERROR_MEMORY, ERROR_RANGE, ERROR_INTERNAL = range(1, 8)
_NAMES = {1: "argument", 2: "io", 3: "format", 4: "unsupported", 5: "memory", 6: "range", 7: "internal"}


class KippError(Exception):
    def __init__(self, code: int, message: str):
        super().__init__(f"{_NAMES.get(code, code)}: {message}")
        self.code, self.message = code, message


def error_code_name(code: int) -> str:
    return _NAMES.get(code, "unknown")


@dataclass
class ModelInfo:
    architecture: str
    layers: int
    hidden_size: int
    vocab_size: int
    context_length: int
    dtype: str
    page_tokens: int
    kv_pool_blocks: int


@dataclass
class SessionInfo:
    capacity: int
    length: int
    cache_bytes: int


class Model:
    def __init__(self, engine: Engine):
        self.engine = engine
        self.sessions: List["Session"] = []
        self._ids = itertools.count()

    @classmethod
    def open(cls, path: str, dtype: str = "bfloat16", kv_pool_blocks: int = 1024, page_tokens: int = 16,
             max_sessions: int = EVAL_BATCH_LIMIT, device: str = "cuda:0") -> "Model":
        """Open a model folder.  Every session draws its pages from one pool of
        `kv_pool_blocks` pages of `page_tokens` tokens; finished sessions publish
        their full pages so that later ones can adopt a matching beginning."""
        from .config import ConfigError
        from .weights import SafetensorsError, WeightError
        if kv_pool_blocks <= 0:
            raise KippError(ERROR_ARGUMENT, "kv_pool_blocks must be nonzero")
        try:
            engine = Engine.from_folder(path, dtype=dtype, device=device, page_size=page_tokens,
                                        num_pages=kv_pool_blocks, max_requests=max_sessions)
        except ConfigError as e:
            raise KippError(ERROR_UNSUPPORTED if "registry" in str(e) else ERROR_FORMAT, str(e)) from e
        except (WeightError, SafetensorsError) as e:
            raise KippError(ERROR_FORMAT, str(e)) from e
        except OSError as e:
            raise KippError(ERROR_IO, str(e)) from e
        return cls(engine)

    def close(self) -> None:
        """Refuses while sessions are alive (/root/reference/src/kipp.c:1340-1344)."""
        if self.sessions:
            raise KippError(ERROR_ARGUMENT, f"{len(self.sessions)} sessions are still alive")
        self.engine = None

    def get_info(self) -> ModelInfo:
        spec, cache = self.engine.model.spec, self.engine.cache
        return ModelInfo(spec.architecture, len(spec.order), spec.hidden_size, spec.vocab_size, spec.max_position,
                         self.engine.rt.dtype, cache.page_size, cache.groups[0].pool.num_pages if cache.groups else 0)

    def is_stop_token(self, token: int) -> bool:
        return int(token) in self.engine.model.spec.stop_tokens

    def kv_pool_stats(self):
        return self.engine.cache.groups[0].pool.stats()

    def session_create(self, capacity: int) -> "Session":
        if capacity <= 0 or capacity > self.engine.model.spec.max_position:
            raise KippError(ERROR_RANGE, f"capacity must be in 1..{self.engine.model.spec.max_position}")
        return Session(self, capacity)

    def eval(self, tokens: Sequence[int]) -> np.ndarray:
        """Stateless: logits of the last of at most 256 tokens (/root/reference/src/kipp.h:164)."""
        if not 1 <= len(tokens) <= 256:
            raise KippError(ERROR_RANGE, "stateless evaluation takes 1..256 tokens")
        s = self.session_create(len(tokens))
        try:
            return s.eval(tokens)
        finally:
            s.destroy(publish=False)

    def eval_batch(self, items: Sequence[tuple]) -> List[np.ndarray]:
        """Several sessions in one step: items are (session, tokens); each gets the
        logits of its last token.  All or nothing (/root/reference/src/kipp.c:3984-4082)."""
        if not 1 <= len(items) <= EVAL_BATCH_LIMIT:
            raise KippError(ERROR_ARGUMENT, f"a batch holds 1..{EVAL_BATCH_LIMIT} items")
        sessions = [s for s, _ in items]
        if len({id(s) for s in sessions}) != len(sessions):
            raise KippError(ERROR_ARGUMENT, "a session appears twice in the batch")
        for s, tokens in items:
            if s.model is not self or s.dead:
                raise KippError(ERROR_ARGUMENT, "a session of another model, or a destroyed one")
            s._check(tokens)
        logits = self._step([StepEntry(s.id, list(t), [len(t) - 1]) for s, t in items])
        out = logits.float().cpu().numpy()
        return [out[i] for i in range(len(items))]

    def _step(self, entries):
        try:
            return self.engine.step(entries)
        except OutOfPages as e:
            raise KippError(ERROR_RANGE, f"KV pool exhausted: {e}") from e
        except OutOfSlots as e:
            raise KippError(ERROR_MEMORY, str(e)) from e
        except ValueError as e:
            raise KippError(ERROR_RANGE, str(e)) from e


class Session:
    def __init__(self, model: Model, capacity: int):
        self.model, self.capacity = model, capacity
        self.id = f"session-{next(model._ids)}"
        self.dead = False
        try:
            model.engine.open(self.id)
        except OutOfSlots as e:
            raise KippError(ERROR_MEMORY, str(e)) from e
        model.sessions.append(self)

    @property
    def _req(self):
        return self.model.engine.cache.requests[self.id]

    @property
    def length(self) -> int:
        return self._req.length

    def get_info(self) -> SessionInfo:
        cache = self.model.engine.cache
        element = 2 if self.model.engine.rt.dtype == "bfloat16" else 4
        per_token = sum(g.bytes_per_token(element) for g in cache.groups)
        return SessionInfo(self.capacity, self.length, per_token * self.capacity)

    def _check(self, tokens) -> None:
        if self.dead:
            raise KippError(ERROR_ARGUMENT, "the session was destroyed")
        if len(tokens) == 0:
            raise KippError(ERROR_ARGUMENT, "at least one token is required")
        if self.length + len(tokens) > self.capacity:
            raise KippError(ERROR_RANGE, f"{len(tokens)} tokens do not fit: {self.length} of {self.capacity} are used")

    def eval(self, tokens: Sequence[int]) -> np.ndarray:
        """Append the tokens; float32 logits [vocab] of the last one."""
        return self.eval_n(tokens, 1)[0]

    def eval_n(self, tokens: Sequence[int], rows: int) -> np.ndarray:
        """Append the tokens; logits [rows, vocab] of the last `rows` of them, each row the bits that
        evaluating its token alone would give (/root/reference/src/kipp.h:190-200: the primitive behind
        verification, where a greedy choice must not flip).  Under float32 every kernel gives a row the
        same bits however the tokens are cut, so one step serves.  Under bfloat16 a portion runs through
        other kernels than a single token does: the tokens before the wanted rows go in as one portion,
        the wanted ones one by one.  All or nothing: a failure leaves the session as it was."""
        self._check(tokens)
        n = len(tokens)
        if not 1 <= rows <= n:
            raise KippError(ERROR_ARGUMENT, "rows must be in 1..token_count")
        if self.model.engine.rt.dtype == "float32" or rows == 1:
            return self.eval_scored(tokens, rows)
        before = self.length
        try:
            if n > rows:
                self.model._step([StepEntry(self.id, list(tokens[:n - rows]), [])])
            out = [self.model._step([StepEntry(self.id, [int(t)], [0])]).float().cpu().numpy() for t in tokens[n - rows:]]
        except KippError:
            if self.length != before:
                self.truncate(before)
            raise
        return np.concatenate(out, axis=0)

    def eval_scored(self, tokens: Sequence[int], rows: int) -> np.ndarray:
        """As `eval_n`, but all tokens go through one step, whose rows agree with single-token evaluation
        within the precision's tolerance only (/root/reference/src/kipp.h:202-213: for scoring, where the
        logits feed arithmetic that tolerates it)."""
        self._check(tokens)
        n = len(tokens)
        if not 1 <= rows <= n:
            raise KippError(ERROR_ARGUMENT, "rows must be in 1..token_count")
        logits = self.model._step([StepEntry(self.id, list(tokens), list(range(n - rows, n)))])
        return logits.float().cpu().numpy()

    def match_prefix(self, tokens: Sequence[int]) -> int:
        """On a fresh session: adopt the longest published beginning of `tokens`
        (whole pages, at least one token left to run); returns the tokens adopted."""
        if self.length != 0:
            raise KippError(ERROR_ARGUMENT, "prefix adoption needs a fresh session")
        cache = self.model.engine.cache
        if not cache.share:
            raise KippError(ERROR_UNSUPPORTED, "this model's cache does not share prefixes")
        usable = list(tokens)[:self.capacity]
        cache.close(self.id)
        req = cache.open(self.id, usable)
        return req.length

    def truncate(self, length: int) -> None:
        try:
            self.model.engine.cache.truncate(self._req, length)
        except NotImplementedError as e:
            raise KippError(ERROR_UNSUPPORTED, str(e)) from e
        except ValueError as e:
            raise KippError(ERROR_RANGE, str(e)) from e

    def reset(self) -> None:
        """Forget the timeline; its full pages are published first."""
        cache = self.model.engine.cache
        cache.close(self.id)
        cache.open(self.id)

    def destroy(self, publish: bool = True) -> None:
        if self.dead:
            return
        cache = self.model.engine.cache
        if not publish:
            cache.requests[self.id].length = cache.requests[self.id].adopted_tokens   # nothing of its own to publish
            cache.requests[self.id].tokens = cache.requests[self.id].tokens[:cache.requests[self.id].length]
        cache.close(self.id)
        self.dead = True
        self.model.sessions.remove(self)


def sample(logits, temperature: float = 0.0, top_p: float = 1.0, rng: Optional[XorShift64Star] = None) -> int:
    """/root/reference/src/kipp.h:264-266."""
    return sample_ex(logits, SampleParams(temperature=temperature, top_p=top_p), rng)


def sample_ex(logits, params: SampleParams, rng: Optional[XorShift64Star] = None, recent: Sequence[int] = ()) -> int:
    """/root/reference/src/kipp.h:278-295."""
    try:
        return _sample(np.asarray(logits, dtype=np.float32), params, rng, recent)
    except ValueError as e:
        raise KippError(ERROR_ARGUMENT, str(e)) from e
