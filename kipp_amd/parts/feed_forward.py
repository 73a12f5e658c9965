"""Feed-forward parts.  Interface:

    params(spec) -> {local name: ParamSpec}
    load(tensors)
    forward(x, batch) -> delta      x [tokens, hidden] activation type,
                                    delta float32 [tokens, hidden] (or slabs of it,
                                    or a product deferred by `Runtime.linear`)

A feed-forward with `takes_scaled_rows = True` also takes `ScaledRows` for x.
"""
from __future__ import annotations

import torch

from ..runtime import ScaledRows
from .base import ParamSpec, register


@register("feed_forward", "gated_mlp")
class GatedMLP:
    """delta = W_down (silu(W_gate x) * (W_up x))  (/root/reference/src/kipp.c:2633-2653)."""

    graph_safe = True   # forward launches kernels only: no host reads, no data-dependent launches
    takes_scaled_rows = True

    def __init__(self, spec, runtime):
        self.spec = spec
        self.rt = runtime
        self.w_gate_up = self.w_down = None

    @staticmethod
    def params(spec):
        return {
            "gate_proj.weight": ParamSpec((spec.intermediate_size, spec.hidden_size)),
            "up_proj.weight": ParamSpec((spec.intermediate_size, spec.hidden_size)),
            "down_proj.weight": ParamSpec((spec.hidden_size, spec.intermediate_size)),
        }

    def load(self, tensors):
        g, u = tensors["gate_proj.weight"], tensors["up_proj.weight"]
        if g.dtype != u.dtype:
            g, u = g.float(), u.float()
        self.w_gate_up = self.rt.weight(torch.cat([g, u], dim=0).contiguous(), gate_up=True)
        self.w_down = self.rt.weight(tensors["down_proj.weight"])

    def forward(self, x, batch=None):
        rt = self.rt
        rows, inner = x.shape[0], self.spec.intermediate_size
        act = rt.empty((rows, inner), rt.act_dtype)
        w = self.w_gate_up
        ours = w.dtype == x.dtype == torch.bfloat16 and rt.streams(rows, x.shape[1], 2 * inner)
        if ours and rows <= rt.few_rows:
            # both products and the activation in one kernel (and the norm's scale, if it was left to us)
            scaled = isinstance(x, ScaledRows)
            # the activation goes to the down projection alone: written in the order that product reads fastest
            major = rt.steps_major_rows and inner % 32 == 0 and rows > 1 and rt._few_rows(rows, inner, self.w_down)
            rt.ops.gemm_skinny_swiglu(x.rows if scaled else x, w.rows, act, tiles=w.tiles,
                                      row_scale=x.scale if scaled else None,
                                      x_steps_major=scaled and x.steps_major, out_steps_major=major)
            return rt.linear(act, self.w_down, slabs=True, defer=True, x_steps_major=major)
        x = rt.rows_of(x)
        if ours and w.pairs and rt.ops.gemm_rows_swiglu_pays(rows, 2 * inner, x.shape[1]):
            # a few dozen rows against a weight with rows enough for every compute unit: the activation at the product's end
            rt.ops.gemm_rows_swiglu(x, w.tiles, act)
        elif ours and w.pairs:
            # streamed from the paired tiles: the columns come out gate tile by gate tile
            rt.ops.swiglu(rt.ops.gemm_rows(x, w.rows, max_parts=12, tiles=w.tiles, pairs=True), act, pairs=True)
        elif w.dtype == x.dtype == torch.bfloat16 and not ours:
            act = rt.gated(x, w, act)       # many rows: both products and the activation, by whichever way is faster
        else:
            rt.ops.swiglu(rt.linear(x, w, slabs=True), act)
        return rt.linear(act, self.w_down, slabs=True, defer=True)
