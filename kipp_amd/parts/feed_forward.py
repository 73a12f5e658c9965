"""Feed-forward parts.  Interface:

    params(spec) -> {local name: ParamSpec}
    load(tensors)
    forward(x, batch) -> delta      x [tokens, hidden] activation type,
                                    delta float32 [tokens, hidden]
"""
from __future__ import annotations

import torch

from .base import ParamSpec, register


@register("feed_forward", "gated_mlp")
class GatedMLP:
    """delta = W_down (silu(W_gate x) * (W_up x))  (/root/reference/src/kipp.c:2633-2653)."""

    graph_safe = True   # forward launches kernels only: no host reads, no data-dependent launches

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
        self.w_gate_up = self.rt.weight(torch.cat([g, u], dim=0).contiguous(), split=2)
        self.w_down = self.rt.weight(tensors["down_proj.weight"])

    def forward(self, x, batch=None):
        rt = self.rt
        rows, inner = x.shape[0], self.spec.intermediate_size
        act = rt.empty((rows, inner), rt.act_dtype)
        if self.w_gate_up.dtype == x.dtype == torch.bfloat16 and rows <= 16 and rt.ops.gemm_skinny_ok(rows, x.shape[1]):
            # both products and the activation in one kernel
            rt.ops.gemm_skinny_swiglu(x, self.w_gate_up.rows, act, tiles=self.w_gate_up.tiles)
        else:
            rt.ops.swiglu(rt.linear(x, self.w_gate_up, slabs=True, low_precision_out=True), act)
        return rt.linear(act, self.w_down, slabs=True)
