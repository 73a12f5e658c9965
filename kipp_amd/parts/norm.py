"""Norm parts.  Interface of a norm:

    params(spec) -> {local name: ParamSpec}
    load(tensors)                       tensors by local name, already on the device
    forward(x, out_dtype) -> y          x float32 [rows, width]
    add_forward(x, delta, out_dtype)    x += delta in place, then y = norm(x)

A norm with `fuses_products = True` also takes a delta that `Runtime.linear(...,
defer=True)` has not launched yet and may return `ScaledRows` (its rows without
their scale, which the product that follows applies); blocks settle both for
parts that do not say they take them.
"""
from __future__ import annotations

from ..runtime import Deferred
from .base import ParamSpec, register


@register("norm", "rms_norm")
class RMSNorm:
    """y = x * rsqrt(mean(x^2) + eps) * w  (/root/reference/src/kipp.c:2221-2231)."""

    graph_safe = True   # forward launches kernels only: no host reads, no data-dependent launches
    fuses_products = True

    def __init__(self, spec, runtime):
        self.spec = spec
        self.rt = runtime
        self.weight = None

    @staticmethod
    def params(spec):
        return {"weight": ParamSpec((spec.width,), "float", ("one_plus_normal", 0.05))}

    @staticmethod
    def placement(spec):
        """Norm weights are widened to float32 on the device (exact)."""
        return {"weight": "float32"}

    def load(self, tensors):
        self.weight = tensors["weight"]

    def forward(self, x, out_dtype):
        return self.rt.ops.rmsnorm(x, self.weight, self.spec.eps, self.rt.empty(x.shape, out_dtype))

    def add_forward(self, x, delta, out_dtype):
        if isinstance(delta, Deferred):       # a product not launched yet: add and norm ride on it where they can
            fused = self.rt.product_add_norm(delta, x, self.weight, self.spec.eps) if out_dtype == self.rt.act_dtype else None
            if fused is not None:
                return fused
            delta = delta.run()
        return self.rt.ops.rmsnorm(x, self.weight, self.spec.eps, self.rt.empty(x.shape, out_dtype), delta=delta)
