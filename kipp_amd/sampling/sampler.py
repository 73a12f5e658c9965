"""Token choice on the host, step for step as the reference's sampler
(/root/reference/src/kipp.c:3310-3571), in the same float widths: logits and
scaled logits float32, exponentials float32 (expf), sums and the draw float64.

Order: logit bias; repetition, presence and frequency penalties over the recent
tokens (each distinct token once); argmax with the lowest index winning ties;
temperature <= 0 returns the argmax and leaves the generator untouched;
otherwise scale by 1/T, keep candidates within 20 of the maximum, sort
descending (ties: lower id first), top-k, weights exp(l - max), min-p, top-p
(shortest prefix with mass >= top_p * total, at least one), one draw from
xorshift64*.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Sequence

import numpy as np

_MASK64 = (1 << 64) - 1


class XorShift64Star:
    """/root/reference/src/kipp.c:3322-3333."""

    def __init__(self, seed: int):
        if seed == 0 or not 0 <= seed <= _MASK64:
            raise ValueError("sampling requires a nonzero 64-bit RNG state")
        self.state = seed

    def next_u64(self) -> int:
        x = self.state
        x ^= x >> 12
        x ^= (x << 25) & _MASK64
        x ^= x >> 27
        self.state = x
        return (x * 2685821657736338717) & _MASK64

    def uniform(self) -> float:
        return (self.next_u64() >> 11) / 9007199254740992.0


@dataclass
class SampleParams:
    """/root/reference/src/kipp.h:278-291."""
    temperature: float = 0.0
    top_p: float = 1.0
    top_k: int = 0
    min_p: float = 0.0
    repetition_penalty: float = 1.0
    presence_penalty: float = 0.0
    frequency_penalty: float = 0.0
    logit_bias: Dict[int, float] = field(default_factory=dict)

    def validate(self) -> None:
        if self.temperature > 0:
            if not (0.0 < self.top_p <= 1.0):
                raise ValueError("top_p must be greater than 0 and at most 1")
            if not (0.0 <= self.min_p <= 1.0):
                raise ValueError("min_p must be between 0 and 1")
        if self.top_k < 0:
            raise ValueError("top_k must be >= 0")

    @property
    def greedy(self) -> bool:
        return self.temperature <= 0.0

    @property
    def has_penalty(self) -> bool:
        return (self.frequency_penalty != 0.0 or self.presence_penalty != 0.0
                or (self.repetition_penalty != 0.0 and self.repetition_penalty != 1.0))

    @property
    def changes_logits(self) -> bool:
        return bool(self.logit_bias) or self.has_penalty


def apply_bias_and_penalties(logits: np.ndarray, params: SampleParams, recent: Sequence[int]) -> np.ndarray:
    """/root/reference/src/kipp.c:3386-3431.  Returns a changed copy."""
    out = np.array(logits, dtype=np.float32, copy=True)
    n = out.shape[0]
    for token, bias in params.logit_bias.items():
        if 0 <= token < n:
            out[token] = np.float32(out[token] + np.float32(bias))
    if not params.has_penalty or not recent:
        return out
    seen = set()
    for token in recent:
        if token >= n or token < 0 or token in seen:
            continue
        seen.add(token)
        count = sum(1 for other in recent if other == token)
        v = out[token]
        if params.repetition_penalty != 0.0 and params.repetition_penalty != 1.0:
            rp = np.float32(params.repetition_penalty)
            v = np.float32(v / rp) if v > 0 else np.float32(v * rp)
        v = np.float32(v - np.float32(params.presence_penalty))
        v = np.float32(v - np.float32(params.frequency_penalty) * np.float32(count))
        out[token] = v
    return out


def logit_change_entries(params: SampleParams, recent: Sequence[int], vocab: int):
    """What `apply_bias_and_penalties` does to one row, as the entries the device kernel walks (`ops.adjust_logits`):
    (tokens, values, how many of them are biases).  A bias entry's value is the bias; the others are the distinct recent
    tokens in their order, each with its count.  Tokens outside the vocabulary are dropped, as there."""
    tokens, values = [], []
    for token, bias in params.logit_bias.items():
        if 0 <= token < vocab:
            tokens.append(int(token))
            values.append(float(np.float32(bias)))
    biases = len(tokens)
    if params.has_penalty and recent:
        seen = set()
        for token in recent:
            if token >= vocab or token < 0 or token in seen:
                continue
            seen.add(token)
            tokens.append(int(token))
            values.append(float(sum(1 for other in recent if other == token)))
    return tokens, values, biases


def argmax(values: np.ndarray) -> int:
    """Strict '>' in index order: the lowest index among equals (kipp.c:3459-3464)."""
    return int(np.argmax(values))


def sample(logits: np.ndarray, params: SampleParams, rng: XorShift64Star | None, recent: Sequence[int] = ()) -> int:
    values = np.asarray(logits, dtype=np.float32)
    if values.ndim != 1 or values.shape[0] == 0:
        raise ValueError("logits must be a non-empty vector")
    if params.changes_logits:
        values = apply_bias_and_penalties(values, params, recent)
    best = argmax(values)
    if params.temperature <= 0.0:
        return best
    params.validate()
    if rng is None or rng.state == 0:      # /root/reference/src/kipp.c:3477-3480
        raise ValueError("sampling requires a nonzero RNG state")
    inverse_temperature = np.float32(1.0) / np.float32(params.temperature)
    scaled = values * inverse_temperature                      # float32
    scaled_maximum = np.float32(values[best] * inverse_temperature)
    cutoff = np.float32(scaled_maximum - np.float32(20.0))
    ids = np.nonzero(scaled >= cutoff)[0]
    cand = scaled[ids]
    order = np.lexsort((ids, -cand.astype(np.float64)))        # descending logit, then lower id
    ids, cand = ids[order], cand[order]
    if params.top_k != 0 and params.top_k < ids.shape[0]:
        ids, cand = ids[:params.top_k], cand[:params.top_k]
    weights = np.exp((cand - scaled_maximum).astype(np.float32)).astype(np.float32)
    if params.min_p > 0.0 and weights.shape[0] > 0:
        threshold = float(np.float32(params.min_p)) * float(weights[0])
        below = np.nonzero(weights[1:].astype(np.float64) < threshold)[0]
        if below.shape[0]:
            keep = int(below[0]) + 1
            ids, weights = ids[:keep], weights[:keep]
    w64 = weights.astype(np.float64)
    cumulative = np.cumsum(w64)                                # sequential float64 sums, as in C
    total = float(cumulative[-1])
    target = float(np.float32(params.top_p)) * total
    nucleus = int(np.searchsorted(cumulative, target, side="left")) + 1   # first count with kept >= target
    nucleus = max(1, min(nucleus, ids.shape[0]))
    kept = float(cumulative[nucleus - 1])
    draw = rng.uniform() * kept
    index = int(np.searchsorted(cumulative[:nucleus], draw, side="right"))  # first with draw < cumulative
    if index >= nucleus:
        index = nucleus - 1
    return int(ids[index])
