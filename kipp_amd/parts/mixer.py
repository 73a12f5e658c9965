"""Token mixers.  Interface of a mixer:

    params(spec) -> {local name: ParamSpec}
    load(tensors)
    cache_need() -> KVNeed or None      what it keeps per token, in pages
    state_need() -> StateNeed or None   what it keeps per request, of fixed size
    forward(x, batch, cache, state) -> delta
        x      [tokens, hidden] in the activation type (the normed residual)
        batch  the step's StepBatch (positions, sequence of each token, tables)
        cache  the KVCacheView of this run (None if cache_need() is None)
        state  tensor [slots, ...] of this run (None if state_need() is None)
        delta  float32 [tokens, hidden], added to the residual by the block
               (or slabs of it, or a product deferred by `Runtime.linear`)

A mixer with `takes_scaled_rows = True` passes x on to `Runtime.linear` only,
which also takes rows whose norm scale is still to be applied.
"""
from __future__ import annotations

import math

from ..cache.needs import KVNeed
from .base import ParamSpec, build_part, register



@register("mixer", "attention")
class Attention:
    """Causal grouped-query attention with optional per-head q/k RMSNorm, a
    rotary position part and an optional window, over the paged cache
    (/root/reference/src/kipp.c:2950-2993).  Query head h reads key/value head
    h // (n_q / n_kv)."""

    graph_safe = True   # forward launches kernels only: no host reads, no data-dependent launches
    takes_scaled_rows = True

    def __init__(self, spec, runtime):
        self.spec = spec
        self.rt = runtime
        self.position = build_part("position", spec.position, runtime)
        self.scale = spec.scale if spec.scale is not None else 1.0 / math.sqrt(spec.head_dim)
        self.w_qkv = self.w_o = self.q_norm = self.k_norm = None

    @staticmethod
    def params(spec):
        p = {
            "q_proj.weight": ParamSpec((spec.q_dim, spec.hidden_size)),
            "k_proj.weight": ParamSpec((spec.kv_dim, spec.hidden_size)),
            "v_proj.weight": ParamSpec((spec.kv_dim, spec.hidden_size)),
            "o_proj.weight": ParamSpec((spec.hidden_size, spec.q_dim)),
        }
        if spec.qk_norm_eps is not None:
            p["q_norm.weight"] = ParamSpec((spec.head_dim,), "float", ("one_plus_normal", 0.05))
            p["k_norm.weight"] = ParamSpec((spec.head_dim,), "float", ("one_plus_normal", 0.05))
        return p

    @staticmethod
    def placement(spec):
        return {"q_norm.weight": "float32", "k_norm.weight": "float32"}

    @staticmethod
    def variants(spec, dtype):
        """The builds of its specialised kernels (one per head size; decode also per number of query heads
        that share a key/value head).  Under float32, and for more than 16 heads a group, the generic
        attention kernel runs, which every model has."""
        if dtype != "bfloat16" or spec.head_dim % 16:
            return []
        group = spec.num_heads // spec.num_kv_heads
        out = [("attention_prefill", {"HEAD_DIM": spec.head_dim})]
        if group <= 16:
            out.append(("attention_decode", {"HEAD_DIM": spec.head_dim, "GROUP": group}))
        return out

    def load(self, tensors):
        import torch
        q, k, v = tensors["q_proj.weight"], tensors["k_proj.weight"], tensors["v_proj.weight"]
        if not (q.dtype == k.dtype == v.dtype):
            q, k, v = (t.float() for t in (q, k, v))
        # rows concatenated: one product serves q, k and v; no output element changes
        self.w_qkv = self.rt.weight(torch.cat([q, k, v], dim=0).contiguous())
        self.w_o = self.rt.weight(tensors["o_proj.weight"])
        if self.spec.qk_norm_eps is not None:
            self.q_norm = tensors["q_norm.weight"]
            self.k_norm = tensors["k_norm.weight"]

    @staticmethod
    def need_of(spec):
        """What a mixer of this spec keeps per token, known without building it."""
        return KVNeed(num_kv_heads=spec.num_kv_heads, head_dim=spec.head_dim, window=spec.window, page_size=spec.page_size)

    def cache_need(self):
        return self.need_of(self.spec)

    def state_need(self):
        return None

    def forward(self, x, batch, cache, state=None):
        s, rt = self.spec, self.rt
        n = x.shape[0]
        inv_freq, rotary_dim = self.position.rotary_table()
        angles = self.position.angles(batch) if hasattr(self.position, "angles") and hasattr(batch, "step_cache") else None
        table = batch.block_tables[cache.group]
        eps = s.qk_norm_eps if s.qk_norm_eps is not None else 0.0
        pairing = getattr(self.position, "pairing", "half")
        # a table row is as wide as the longest context of this step, so what decides is what the step needs
        fast = rt.dtype == "bfloat16" and s.head_dim % 16 == 0 \
            and rt.ops.attention_fast_ok(s.num_heads, s.num_kv_heads, cache.page_size, table.shape[1])
        if rt.dtype == "bfloat16" and not fast:
            rt.generic_attention_launches += 1      # the slow kernel class: a measurement must know it ran
        # single tokens only: norm, rotation, cache write and attention in one kernel, for a few of them (with
        # more rows or long contexts every split's workgroup would prepare the queries again, which costs more
        # than the rotary kernel it saves) and wherever the kernel that walks whole contexts or long ranges runs
        fused = fast and not batch.n_portions and batch.n_decode == n and pairing == "half" \
            and rt.ops.attention_decode_fused_ok(s.head_dim, rotary_dim, inv_freq is not None) \
            and ((n <= rt.fused_decode_rows and batch.max_decode_ctx < rt.fused_decode_keys)
                 or rt.ops.attention_decode_streams(n, s.num_kv_heads, s.head_dim, s.num_heads // s.num_kv_heads,
                                                    cache.page_size, batch.max_decode_ctx, s.window or 0))
        qkv = rt.linear(x, self.w_qkv, slabs=rt.ops.DECODE_FUSED_SLABS if fused else True)
        if fused:
            out = rt.empty((n, s.q_dim), rt.act_dtype)
            # the mixed heads go to the output projection alone: in the order that product reads fastest, if it is a few-rows one
            major = rt.steps_major_rows and n > 1 and rt._few_rows(n, s.q_dim, self.w_o)
            rt.ops.attention_decode_fused(qkv, cache.k, cache.v, out, batch.decode_rows, batch.positions,
                                          batch.seq_of_token, table, s.num_heads, s.num_kv_heads, s.head_dim,
                                          self.q_norm, self.k_norm, eps, inv_freq, rotary_dim, cache.writable,
                                          self.scale, s.window or 0, batch.max_decode_ctx, self._workspace(batch),
                                          angles=angles, out_steps_major=major)
            return rt.linear(out, self.w_o, slabs=True, defer=True, x_steps_major=major)
        q = rt.ops.qk_norm_rope_kv_write(
            qkv, rt.empty((n, s.q_dim), rt.act_dtype), cache.k, cache.v,
            batch.positions, batch.seq_of_token, table, s.num_heads, s.num_kv_heads, s.head_dim,
            self.q_norm, self.k_norm, eps, inv_freq, rotary_dim, write_kv=cache.writable, angles=angles, pairing=pairing)
        out = rt.empty((n, s.q_dim), rt.act_dtype)
        if fast:
            if batch.n_portions:
                item_seq, item_tile, cuts = self._prefill_work(batch)
                rt.ops.attention_prefill(q, cache.k, cache.v, out, item_seq, item_tile, batch.q_start,
                                         batch.q_len, batch.positions, table, s.num_heads, s.num_kv_heads, s.head_dim,
                                         self.scale, s.window or 0, cuts=cuts)
            if batch.n_decode:
                rt.ops.attention_decode(q, cache.k, cache.v, out, batch.decode_rows, batch.positions, batch.seq_of_token,
                                        table, s.num_heads, s.num_kv_heads, s.head_dim, self.scale, s.window or 0,
                                        batch.max_decode_ctx, self._workspace(batch))
        else:
            # the float32 path, and geometries the matrix-core kernels refuse (groups above 16, odd page sizes)
            rt.ops.paged_attention_generic(q, cache.k, cache.v, out, batch.positions, batch.seq_of_token, table,
                                           s.num_heads, s.num_kv_heads, s.head_dim, self.scale, s.window or 0)
        return rt.linear(out, self.w_o, slabs=True, defer=True)

    def _prefill_work(self, batch):
        """The work list of the prefill kernel: (entry, tile of 128 query rows) for every entry that brings a
        portion, the longest key range first (the kernel folds the list so that workgroups sharing a
        compute unit carry about the same load).

        A workgroup walks all keys its tile sees, one after the other.  Where the tiles times the heads are
        fewer workgroups than two a compute unit and the contexts are long (a portion of a few hundred rows
        behind thousands of keys), the keys are cut as well, at multiples of a length chosen so that the
        GPU is filled about twice: a work item is then (entry, tile, cut), and the cuts of a row are merged
        in order afterwards.  The cuts follow from the step's shape, not from a row's place in it, so a row's
        result may differ in its last bits between steps of different shapes, as between the kernels for
        portions and for single tokens.  Made by the first attention layer of a forward pass and shared by
        the others of the same geometry."""
        s, ops = self.spec, self.rt.ops
        key = ("attention_prefill_work", s.num_heads, s.head_dim, s.window)
        work = batch.step_cache.get(key)
        if work is None:
            tile = ops.PREFILL_ROWS
            q_start = batch.host["q_start"]
            portions = [(i, n, ctx) for i, (n, ctx) in enumerate(zip(batch.host["q_len"], batch.host["ctx_len"])) if n > 1]
            tiles = [(i, t, ctx - n + min((t + 1) * tile, n) - 1, q_start[i] + t * tile, min(tile, n - t * tile))
                     for i, n, ctx in portions for t in range((n + tile - 1) // tile)]     # (entry, tile, last key, first row, rows)
            workgroups = len(tiles) * s.num_heads
            longest = max(last for _, _, last, _, _ in tiles) + 1
            split_keys = 0
            units = ops.compute_units(self.rt.device)
            if s.window is None and workgroups < 2 * units:
                want = -(-2 * units // workgroups)
                split_keys = max(ops.PREFILL_MIN_CUT, -(-longest // want // 64) * 64)
                if longest <= split_keys:
                    split_keys = 0
            if not split_keys:
                items = sorted((-last, i, t) for i, t, last, _, _ in tiles)
                work = tuple(batch.upload([i for _, i, _ in items], [t for _, _, t in items])) + (None,)
            else:
                items, merge_rows, merge_cuts = [], [], []
                for i, t, last, row0, rows in tiles:
                    cuts = last // split_keys + 1
                    items.extend((-(min(last + 1, (c + 1) * split_keys) - c * split_keys), i, t, c) for c in range(cuts))
                    merge_rows.extend(range(row0, row0 + rows))
                    merge_cuts.extend([cuts] * rows)
                items.sort()
                most = max(merge_cuts)
                seq, til, cut, rows_d, cuts_d = batch.upload([i for _, i, _, _ in items], [t for _, _, t, _ in items],
                                                             [c for _, _, _, c in items], merge_rows, merge_cuts)
                space = ops.attention_prefill_workspace(batch.n_tokens, s.num_heads, s.head_dim, most, self.rt.device)
                work = (seq, til, (split_keys, cut, rows_d, cuts_d, space))
            batch.step_cache[key] = work
        return work

    def _workspace(self, batch):
        """Partial results of the split decode kernel, shared by the layers of one geometry and kept
        while the batch object lives (a recorded step keeps its own)."""
        s = self.spec
        key = ("decode_workspace", batch.n_decode, batch.max_decode_ctx, s.num_heads, s.head_dim)
        ws = batch.host.get(key)
        if ws is None:
            ws = self.rt.ops.attention_decode_workspace(batch.n_decode, s.num_heads, s.head_dim,
                                                        batch.max_decode_ctx, self.rt.device)
            if not self.rt.merge_in_kernel:
                ws = ws[:2]         # without the counts the splits are merged by a launch of its own
            batch.host[key] = ws
        return ws
