"""Token embedding and output head."""
from __future__ import annotations

from .base import ParamSpec, register


@register("embedding", "embedding")
class Embedding:
    """x[t] = E[token_t], widened to float32, no scaling (/root/reference/src/kipp.c:2579-2585)."""

    graph_safe = True   # forward launches kernels only: no host reads, no data-dependent launches

    def __init__(self, spec, runtime):
        self.spec = spec
        self.rt = runtime
        self.weight = None

    @staticmethod
    def params(spec):
        return {"weight": ParamSpec((spec.vocab_size, spec.hidden_size))}

    def load(self, tensors):
        self.weight = tensors["weight"]

    def forward(self, tokens):
        import torch
        return self.rt.ops.embed(self.weight, tokens, self.rt.empty((tokens.numel(), self.spec.hidden_size), torch.float32))


@register("head", "lm_head")
class Head:
    """logits = W x, float32, no bias (/root/reference/src/kipp.c:2660-2661).  A tied
    head has no tensor of its own and uses the embedding table."""

    graph_safe = True   # forward launches kernels only: no host reads, no data-dependent launches

    def __init__(self, spec, runtime):
        self.spec = spec
        self.rt = runtime
        self.weight = None

    @staticmethod
    def params(spec):
        return {} if spec.tied else {"weight": ParamSpec((spec.vocab_size, spec.hidden_size))}

    def load(self, tensors, embedding=None):
        self.weight = self.rt.weight(embedding.weight if self.spec.tied else tensors["weight"])

    def forward(self, x):
        return self.rt.linear(x, self.weight)
