"""Block arrangements: how the parts of one layer are put together.

Interface of a block:

    roles: tuple of (role, category) the arrangement needs in LayerSpec.parts
    forward(x, pending, batch, cache, state) -> (x, pending)
        x        float32 [tokens, hidden], the residual stream (updated in place)
        pending  a delta not yet added to x (or None); the block adds it inside
                 its first norm and hands its own last delta on the same way,
                 so that residual add and norm are one kernel.  A delta may
                 be a product that the runtime has not launched yet
                 (`Runtime.linear(..., defer=True)`), and a norm may leave its
                 scale to the product that follows (`ScaledRows`): the block
                 settles either for a part that does not declare it takes it
                 (`fuses_products` of a norm, `takes_scaled_rows` of a mixer
                 or feed-forward).
"""
from __future__ import annotations

from .base import build_part, register


@register("block", "pre_norm")
class PreNormBlock:
    """x += mixer(mixer_norm(x)); x += ffn(ffn_norm(x))
    (/root/reference/docs/ARCHITECTURE.md:77-92)."""

    roles = (("mixer_norm", "norm"), ("mixer", "mixer"), ("ffn_norm", "norm"), ("ffn", "feed_forward"))

    def __init__(self, layer_spec, runtime):
        self.rt = runtime
        self.parts = {role: build_part(cat, layer_spec.part(role), runtime) for role, cat in self.roles}
        self.mixer = self.parts["mixer"]
        self.graph_safe = all(getattr(part, "graph_safe", False) for part in self.parts.values())

    def forward(self, x, pending, batch, cache, state):
        act = self.rt.act_dtype
        norm1, norm2 = self.parts["mixer_norm"], self.parts["ffn_norm"]
        rt, ffn = self.rt, self.parts["ffn"]
        if pending is not None and not getattr(norm1, "fuses_products", False):
            pending = rt.settle(pending)
        h = norm1.forward(x, act) if pending is None else norm1.add_forward(x, pending, act)
        if not getattr(self.mixer, "takes_scaled_rows", False):
            h = rt.rows_of(h)
        delta = self.mixer.forward(h, batch, cache, state)
        if not getattr(norm2, "fuses_products", False):
            delta = rt.settle(delta)
        h = norm2.add_forward(x, delta, act)
        if not getattr(ffn, "takes_scaled_rows", False):
            h = rt.rows_of(h)
        return x, ffn.forward(h, batch)
