"""Position-encoding parts.  A position part is owned by a mixer, which applies
it inside its own kernel; the interface is what that kernel needs:

    rotary_table() -> (inv_freq float32 [rotary_dim / 2] on the device, rotary_dim)
                      or (None, 0) when the part does not rotate
    pairing           "half" (dim i turns with dim i + rotary_dim / 2; the default when
                      the attribute is missing) or "interleaved" (dim 2i with dim 2i + 1)
    angles(batch)  -> float32 [tokens, rotary_dim] (cosines, then sines) of the
                      batch's positions, or None; optional: a mixer computes
                      the angles itself from `inv_freq` where it is missing.
                      Parts with the same frequencies share one table a step
                      (`batch.step_cache`, emptied at the start of every forward).

A rotary part of another kind (scaled frequencies, another base) only has to
produce its own table.

A position encoding that is no rotation inside a mixer (a learned table, an
additive code) is a part of the same category that the model applies to the
residual stream once, after the embedding: `ModelSpec.input_position` names
its spec, and its interface is

    params(spec), load(tensors)
    forward(x, batch) -> x          x float32 [tokens, hidden], changed in place or anew;
                                    batch.positions holds every token's position
"""
from __future__ import annotations

import torch

from .base import register


@register("position", "none")
class NoPosition:
    graph_safe = True   # forward launches kernels only: no host reads, no data-dependent launches
    def __init__(self, spec, runtime):
        self.spec = spec

    @staticmethod
    def params(spec):
        return {}

    def load(self, tensors):
        pass

    def rotary_table(self):
        return None, 0

    def angles(self, batch):
        return None


@register("position", "rope")
class Rope:
    """inv_freq[i] = theta^(-2i / rotary_dim), angle = float32(pos) * inv_freq[i]
    (/root/reference/src/kipp.c:2368-2382).  The table is computed once in
    float64 and rounded to float32; the angle product is float32."""

    graph_safe = True   # forward launches kernels only: no host reads, no data-dependent launches

    def __init__(self, spec, runtime):
        if spec.pairing not in ("half", "interleaved"):
            raise ValueError(f"rope pairing {spec.pairing!r} is not implemented (half, interleaved)")
        self.spec = spec
        self.pairing = spec.pairing
        self.rt = runtime
        self.rotary_dim = spec.head_dim if spec.rotary_dim is None else spec.rotary_dim
        self.inv_freq = self.frequencies().to(device=runtime.device, dtype=torch.float32)

    def frequencies(self) -> torch.Tensor:
        half = self.rotary_dim // 2
        i = torch.arange(half, dtype=torch.float64)
        return torch.pow(torch.tensor(float(self.spec.theta), dtype=torch.float64), -(2.0 * i) / self.rotary_dim)

    @staticmethod
    def params(spec):
        return {}

    def load(self, tensors):
        pass

    def rotary_table(self):
        return self.inv_freq, self.rotary_dim

    def angles(self, batch):
        key = ("rotary_angles", float(self.spec.theta), self.rotary_dim)
        table = batch.step_cache.get(key)
        if table is None:
            table = self.rt.ops.rotary_angles(batch.positions, self.inv_freq,
                                              self.rt.empty((batch.n_tokens, self.rotary_dim), torch.float32))
            batch.step_cache[key] = table
        return table
