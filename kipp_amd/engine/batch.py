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
    prefill_seq: torch.Tensor = None     # int32 per work item: entry that brings a portion ...
    prefill_tile: torch.Tensor = None    # ... and which tile of PREFILL_TILE rows of it
    n_decode: int = 0
    n_prefill_items: int = 0
    max_decode_ctx: int = 0
    max_q_len: int = 0
    max_ctx_len: int = 0
    want_every_row: bool = False         # want_rows is 0, 1, ... n_tokens - 1
    host: dict = field(default_factory=dict)
    step_cache: dict = field(default_factory=dict)   # device values of this forward that parts share; emptied by every forward


PREFILL_TILE = 128   # query rows of one work item of the prefill attention kernel


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
    items = []
    for i in range(n_seqs):
        if q_len[i] > 1:
            start = ctx_len[i] - q_len[i]
            for tile in range((q_len[i] + PREFILL_TILE - 1) // PREFILL_TILE):
                keys = start + min((tile + 1) * PREFILL_TILE, q_len[i])     # keys the tile's last row sees
                items.append((-keys, i, tile))
    items.sort()                                                          # longest key range first
    prefill_seq = [i for _, i, _ in items]
    prefill_tile = [t for _, _, t in items]
    max_blocks = max(1, max(len(req.tables[g]) for req in requests for g in range(n_groups)) if n_groups else 1)
    tables = []
    for g in range(n_groups):
        for req in requests:
            row = [p if p >= 0 else 0 for p in req.tables[g]]
            tables.extend(row + [0] * (max_blocks - len(row)))
    sections = [tokens, positions, seq_of, q_start, q_len, ctx_len, slots, want_rows, decode_rows, prefill_seq,
                prefill_tile, tables]
    flat = torch.tensor([v for s in sections for v in s], dtype=torch.int32).pin_memory() \
        if torch.cuda.is_available() else torch.tensor([v for s in sections for v in s], dtype=torch.int32)
    dev = flat.to(device, non_blocking=True)
    parts = []
    offset = 0
    for s in sections:
        parts.append(dev[offset:offset + len(s)])
        offset += len(s)
    t_tokens, t_pos, t_seq, t_qs, t_ql, t_cl, t_slots, t_want, t_dec, t_pfs, t_pft, t_tables = parts
    block_tables = {g: t_tables[g * n_seqs * max_blocks:(g + 1) * n_seqs * max_blocks].view(n_seqs, max_blocks)
                    for g in range(n_groups)}
    return StepBatch(
        n_tokens=len(tokens), n_seqs=n_seqs, n_want=len(want_rows),
        tokens=t_tokens, positions=t_pos, seq_of_token=t_seq, q_start=t_qs, q_len=t_ql, ctx_len=t_cl,
        slots=t_slots, want_rows=t_want, block_tables=block_tables,
        decode_rows=t_dec, prefill_seq=t_pfs, prefill_tile=t_pft, n_decode=len(decode_rows),
        n_prefill_items=len(prefill_seq), max_decode_ctx=max(decode_ctx) if decode_ctx else 0,
        max_q_len=max(q_len) if q_len else 0, max_ctx_len=max(ctx_len) if ctx_len else 0,
        want_every_row=want_rows == list(range(len(tokens))),
        host={"q_start": q_start, "q_len": q_len, "ctx_len": ctx_len})
