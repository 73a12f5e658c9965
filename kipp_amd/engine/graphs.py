"""Decode steps as HIP graphs.

A step in which every entry brings one token launches a few hundred small
kernels; recorded once into a HIP graph and replayed, the launches cost the
host almost nothing.  A graph is kept for each (number of entries, context
bucket): shapes, grids and buffer addresses of a decode step depend on nothing
else.  What changes from step to step (tokens, positions, slots, block
tables) lives in one static int32 buffer that is overwritten before a replay.

A graph holds our own kernels only: nothing that reads back to the host, no
library call, no memset node.  A model with a part that does not declare
`graph_safe`, or a step that went to a library product, runs eagerly instead.

The number of rows is rounded up to one of a few sizes (exact up to 16, then 24, 32,
48, ... 256), so that a batch whose size changes from step to step still finds its
graph: the rows that fill up bring token 0 at position 0 of a sequence of their own,
whose block table names the cache's scratch page and whose state is the scratch slot;
their logits are dropped.

A shape is recorded when it comes a second time (recording costs the host a
whole forward pass: under continuous batching the number of decoding requests
often changes from step to step, and a shape seen once may never return), and
only the most recently used shapes are kept.
"""
from __future__ import annotations

import gc
import weakref
from collections import OrderedDict
from typing import Dict, Optional, Sequence, Tuple

import numpy as np
import torch

from .batch import StepBatch

CONTEXT_BUCKET = 1024
MAX_GRAPHS = 48              # shapes kept (each holds its recorded launches and small static buffers)
MAX_GRAPH_ENTRIES = 256     # rows up to which every product of a step is one of our own kernels (none goes to a library)


GRAPH_SIZES = [1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16, 24, 32, 48, 64, 96, 128, 192, 256]   # exact up to 16 rows (every row costs there: 13 rows on a recording of 16 took 3.23 ms, of 13 rows 3.12)


def padded_size(n: int) -> int:
    for size in GRAPH_SIZES:
        if size >= n:
            return size
    raise ValueError(f"{n} rows are more than a recorded step takes")


class DecodeGraph:
    def __init__(self, engine, n_seqs: int, max_context: int):
        cache = engine.cache
        rt = engine.rt
        self.n = n = n_seqs
        self.groups = len(cache.groups)
        # a table row is as wide as the contexts of this shape, not as the model's longest possible one:
        # kernels choose by it what they can do, and it is copied whenever a row changes
        self.blocks = [max(1, -(-max_context // g.page_size)) for g in cache.groups]     # of a table row, per group
        self.table_at = [4 * n + n * sum(self.blocks[:g]) for g in range(self.groups)]     # where a group's tables begin
        self.max_context = max_context
        table_ints = n * sum(self.blocks)
        # [tokens | positions | ctx_len | slots | tables | arange | ones]
        self.layout = {"tokens": 0, "positions": n, "ctx_len": 2 * n, "slots": 3 * n, "tables": 4 * n}
        var_ints = 4 * n + table_ints
        total = var_ints + 2 * n
        self.var_ints = var_ints
        self.host = torch.zeros(total, dtype=torch.int32).pin_memory()
        self.host_np = self.host.numpy()
        self.host_np[var_ints:var_ints + n] = np.arange(n, dtype=np.int32)
        self.host_np[var_ints + n:] = 1
        self.dev = torch.zeros(total, dtype=torch.int32, device=rt.device)
        self.dev.copy_(self.host)
        d = self.dev
        arange = d[var_ints:var_ints + n]
        ones = d[var_ints + n:]
        tables = {g: d[self.table_at[g]:self.table_at[g] + n * self.blocks[g]].view(n, self.blocks[g])
                  for g in range(self.groups)}
        self.batch = StepBatch(
            n_tokens=n, n_seqs=n, n_want=n, tokens=d[0:n], positions=d[n:2 * n], seq_of_token=arange, q_start=arange,
            q_len=ones, ctx_len=d[2 * n:3 * n], slots=d[3 * n:4 * n], want_rows=arange, block_tables=tables,
            decode_rows=arange, n_decode=n, n_portions=0,
            max_decode_ctx=max_context, max_q_len=1, max_ctx_len=max_context, want_every_row=True,
            host={"q_start": list(range(n)), "q_len": [1] * n, "ctx_len": [max_context] * n})
        self.graph: Optional[torch.cuda.CUDAGraph] = None
        self.logits: Optional[torch.Tensor] = None
        self.copied: Optional[torch.cuda.Event] = None
        self.row_marks = [None] * n
        self.eager_runs = 0
        self.scratch_pages = [cache.scratch_page(g) for g in range(self.groups)]
        self.scratch_slot = cache.scratch_slot

    def fill(self, entries, requests, device_tokens=None) -> None:
        n, h = self.n, self.host_np
        live = len(entries)                  # rows beyond them only fill the batch up to the recorded size
        if self.copied is not None:
            self.copied.synchronize()     # the copy of the step before has left the pinned buffer
        h[0:n] = 0
        if device_tokens is None:
            h[0:live] = [e.tokens[0] for e in entries]
        h[n:n + live] = [r.length for r in requests]
        h[n + live:2 * n] = 0
        h[2 * n:3 * n] = h[n:2 * n] + 1
        h[3 * n:3 * n + live] = [r.slot for r in requests]
        h[3 * n + live:4 * n] = self.scratch_slot
        # a row of a block table changes only when its request got a page (or another request
        # took the row): only then is it written again, and only then are the tables copied
        changed = False
        for i in range(n):
            r = requests[i] if i < live else None
            # the serial, not the id: an id that was closed and opened again names another request with other pages
            mark = (r.serial, r.table_version) if r is not None else "fills up"
            if self.row_marks[i] != mark:
                self.row_marks[i] = mark
                changed = True
                for g in range(self.groups):
                    at, width = self.table_at[g] + i * self.blocks[g], self.blocks[g]
                    h[at:at + width] = r.rows[g][:width] if r is not None else self.scratch_pages[g]
        upto = self.var_ints if changed else 4 * n
        self.dev[:upto].copy_(self.host[:upto], non_blocking=True)
        self.copied = torch.cuda.Event()
        self.copied.record()
        if device_tokens is not None:
            self.dev[:live].copy_(device_tokens)  # on the device, after the copy above: the tokens the host does not know

    def run(self, engine, entries, requests, device_tokens=None, borrow: bool = False) -> torch.Tensor:
        self.fill(entries, requests, device_tokens)
        if self.graph is None:
            # a shape runs eagerly until it has come twice (that also makes every workspace the
            # kernels keep); if nothing in it went to a library, the same launches are then
            # recorded for the steps to come
            before = engine.rt.library_products
            engine.rt.for_a_graph = True        # the products of these rows keep to kernels that can be recorded
            try:
                logits = engine.model.forward(self.batch, engine.cache)
            finally:
                engine.rt.for_a_graph = False
            self.eager_runs += 1
            if engine.rt.library_products != before or self.eager_runs < 2:
                return logits[:len(entries)]
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            # nothing may be freed on the device while the stream records: the collector stays
            # off until the recording ends (it runs once before, inside torch.cuda.graph)
            was_enabled = gc.isenabled()
            gc.disable()
            engine.rt.for_a_graph = True
            try:
                with torch.cuda.graph(graph):
                    self.logits = engine.model.forward(self.batch, engine.cache)
            finally:
                engine.rt.for_a_graph = False
                if was_enabled:
                    gc.enable()
            self.graph = graph
            return logits[:len(entries)]
        self.graph.replay()
        rows = self.logits[:len(entries)]
        if borrow:
            return rows                 # the graph's own output buffer: the next replay of this shape overwrites it
        return engine.rt.ops.copy(rows, engine.rt.empty(rows.shape, rows.dtype))


class DecodeGraphs:
    """The graphs of one engine, made when a shape is first seen."""

    def __init__(self, engine):
        self._engine = weakref.ref(engine)     # no cycle: an engine and its graphs go away together, at once
        self.graphs: "OrderedDict[Tuple[int, int], DecodeGraph]" = OrderedDict()
        model = engine.model
        self.possible = all(getattr(b, "graph_safe", False) for b in model.blocks) and all(
            getattr(p, "graph_safe", False) for p in (model.embedding, model.final_norm, model.head)
            + ((model.input_position,) if model.input_position is not None else ()))
        self.replays = 0

    def applies(self, entries: Sequence) -> bool:
        return (self.possible and 0 < len(entries) <= MAX_GRAPH_ENTRIES
                and all(len(e.tokens) == 1 and list(e.want) == [0] for e in entries))

    def run(self, entries, requests, device_tokens=None, borrow: bool = False) -> torch.Tensor:
        engine = self._engine()
        cache = engine.cache
        longest = max(r.length for r in requests) + 1
        bucket = min(-(-longest // CONTEXT_BUCKET) * CONTEXT_BUCKET, max(cache.max_position, 1))
        key = (padded_size(len(entries)), bucket)
        graph = self.graphs.get(key)
        if graph is None:
            graph = self.graphs[key] = DecodeGraph(engine, key[0], bucket)
            if len(self.graphs) > MAX_GRAPHS:
                self.graphs.popitem(last=False)        # the shape used longest ago
        else:
            self.graphs.move_to_end(key)
        if graph.graph is not None:
            self.replays += 1
        return graph.run(engine, entries, requests, device_tokens, borrow)
