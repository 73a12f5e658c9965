"""One step's batch, flattened: the tokens of every entry one after another,
with what each kernel needs to find a token's sequence, position and pages.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Sequence

import torch


@dataclass
class StepEntry:
    """A request's next tokens and the places among them whose logits are wanted."""
    request: object
    tokens: Sequence[int]
    want: Sequence[int] = ()


@dataclass
class StepBatch:
    n_tokens: int
    n_seqs: int
    n_want: int
    tokens: torch.Tensor          # int32 [tokens]
    positions: torch.Tensor       # int32 [tokens]   absolute position of each token in its sequence
    seq_of_token: torch.Tensor    # int32 [tokens]   index of the token's entry in this batch
    q_start: torch.Tensor         # int32 [seqs]     first row of each entry
    q_len: torch.Tensor           # int32 [seqs]
    ctx_len: torch.Tensor         # int32 [seqs]     tokens of the sequence after this step
    slots: torch.Tensor           # int32 [seqs]     state slot of each entry's request
    want_rows: torch.Tensor       # int32 [wanted]   rows whose logits are returned
    block_tables: Dict[int, torch.Tensor]  # group -> int32 [seqs, blocks]
    decode_rows: torch.Tensor = None     # int32 rows of the entries that bring one token
    n_decode: int = 0                    # entries that bring one token
    n_portions: int = 0                  # entries that bring more than one
    max_decode_ctx: int = 0
    max_q_len: int = 0
    max_ctx_len: int = 0
    want_every_row: bool = False         # want_rows is 0, 1, ... n_tokens - 1
    # per entry, as Python lists: "q_start", "q_len", "ctx_len"; parts may also keep buffers here that live as long as the batch
    host: dict = field(default_factory=dict)
    step_cache: dict = field(default_factory=dict)   # device values of this forward that parts share; emptied by every forward

    def upload(self, *lists):
        """int32 tensors on the batch's device holding `lists`, sent in one copy that nothing waits for:
        for a part that derives work lists of its own from `host` (it keeps them in `step_cache`)."""
        flat = torch.tensor([v for values in lists for v in values], dtype=torch.int32)
        if self.tokens.is_cuda:
            flat = flat.pin_memory()
        dev = flat.to(self.tokens.device, non_blocking=True)
        out, at = [], 0
        for values in lists:
            out.append(dev[at:at + len(values)])
            at += len(values)
        return out


def build_batch(entries: Sequence[StepEntry], requests: Sequence[object], n_groups: int, device) -> StepBatch:
    """`requests[i]` is the RequestCache of `entries[i]` (pages already reserved).
    All integers go to the device in one copy."""
    tokens: List[int] = []
    positions: List[int] = []
    seq_of: List[int] = []
    q_start: List[int] = []
    q_len: List[int] = []
    ctx_len: List[int] = []
    slots: List[int] = []
    want_rows: List[int] = []
    for i, (entry, req) in enumerate(zip(entries, requests)):
        n = len(entry.tokens)
        q_start.append(len(tokens))
        q_len.append(n)
        ctx_len.append(req.length + n)
        slots.append(req.slot)
        for w in entry.want:
            if not 0 <= w < n:
                raise ValueError(f"request {entry.request!r}: wanted place {w} is not among its {n} tokens")
            want_rows.append(len(tokens) + w)
        tokens.extend(int(t) for t in entry.tokens)
        positions.extend(range(req.length, req.length + n))
        seq_of.extend([i] * n)
    n_seqs = len(entries)
    decode_rows = [q_start[i] for i in range(n_seqs) if q_len[i] == 1]
    decode_ctx = [ctx_len[i] for i in range(n_seqs) if q_len[i] == 1]
    max_blocks = max(1, max(len(req.tables[g]) for req in requests for g in range(n_groups)) if n_groups else 1)
    tables = []
    for g in range(n_groups):
        for req in requests:
            row = [p if p >= 0 else 0 for p in req.tables[g]]
            tables.extend(row + [0] * (max_blocks - len(row)))
    sections = [tokens, positions, seq_of, q_start, q_len, ctx_len, slots, want_rows, decode_rows, tables]
    flat = torch.tensor([v for s in sections for v in s], dtype=torch.int32).pin_memory() \
        if torch.cuda.is_available() else torch.tensor([v for s in sections for v in s], dtype=torch.int32)
    dev = flat.to(device, non_blocking=True)
    parts = []
    offset = 0
    for s in sections:
        parts.append(dev[offset:offset + len(s)])
        offset += len(s)
    t_tokens, t_pos, t_seq, t_qs, t_ql, t_cl, t_slots, t_want, t_dec, t_tables = parts
    block_tables = {g: t_tables[g * n_seqs * max_blocks:(g + 1) * n_seqs * max_blocks].view(n_seqs, max_blocks)
                    for g in range(n_groups)}
    return StepBatch(
        n_tokens=len(tokens), n_seqs=n_seqs, n_want=len(want_rows),
        tokens=t_tokens, positions=t_pos, seq_of_token=t_seq, q_start=t_qs, q_len=t_ql, ctx_len=t_cl,
        slots=t_slots, want_rows=t_want, block_tables=block_tables,
        decode_rows=t_dec, n_decode=len(decode_rows), n_portions=n_seqs - len(decode_rows), max_decode_ctx=max(decode_ctx) if decode_ctx else 0,
        max_q_len=max(q_len) if q_len else 0, max_ctx_len=max(ctx_len) if ctx_len else 0,
        want_every_row=want_rows == list(range(len(tokens))),
        host={"q_start": q_start, "q_len": q_len, "ctx_len": ctx_len})
