"""A decoder built from a `ModelSpec`: the parts of every layer, the run order,
and the forward pass over one flattened batch of tokens.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..config import ModelSpec, load_config, parse_config
from ..parts import ParamSpec, build_part, part_class, part_params
from ..weights.loader import check_tensors, read_model_tensors


def _part_specs(spec: ModelSpec):
    """(category, part spec) of every part that owns tensors, in file order."""
    yield "embedding", spec.embedding
    if spec.input_position is not None:
        yield "position", spec.input_position
    for layer in spec.layers:
        block_cls = part_class("block", layer.block)
        for role, category in block_cls.roles:
            yield category, layer.part(role)
    yield "norm", spec.final_norm
    yield "head", spec.head


def model_params(spec: ModelSpec) -> Dict[str, ParamSpec]:
    """Every tensor the model needs, by file name.  No device is touched."""
    out: Dict[str, ParamSpec] = {}
    for category, part_spec in _part_specs(spec):
        for name, p in part_params(category, part_spec).items():
            if name in out:
                raise ValueError(f"two parts declare the tensor {name!r}")
            out[name] = p
    return out


def cache_bytes_per_page(spec: ModelSpec, page_size: int, element_size: int) -> int:
    """Bytes one page of every cache group takes together, from what the mixers of the spec declare (`need_of(spec)`, a
    static method of a mixer class that keeps keys and values); no device is touched.  Sizes a pool given in bytes."""
    from ..cache import CacheManager
    needs = []
    for run in spec.order:
        mixer = dict(spec.layers[run.layer].parts).get("mixer")
        need_of = getattr(part_class("mixer", mixer.kind), "need_of", None) if mixer is not None else None
        needs.append(need_of(mixer) if need_of is not None and run.cache_of is None else None)
    groups = CacheManager(needs, [None] * len(needs), page_size, 1, 1, spec.max_position, runtime=None).groups
    return sum(g.bytes_per_token(element_size) * g.page_size for g in groups)


class Model:
    def __init__(self, spec: ModelSpec, runtime):
        self.spec = spec
        self.rt = runtime
        self.embedding = build_part("embedding", spec.embedding, runtime)
        self.input_position = (build_part("position", spec.input_position, runtime)
                               if spec.input_position is not None else None)
        self.blocks = [build_part("block", layer, runtime) for layer in spec.layers]
        self.final_norm = build_part("norm", spec.final_norm, runtime)
        self.head = build_part("head", spec.head, runtime)
        self.loaded = False

    # -- what the cache manager has to provide, per run of the order -----------------
    def kv_needs(self):
        return [None if run.cache_of is not None else self.blocks[run.layer].mixer.cache_need()
                for run in self.spec.order]

    def state_needs(self):
        return [self.blocks[run.layer].mixer.state_need() for run in self.spec.order]

    # -- weights ------------------------------------------------------------------------
    def _owners(self):
        yield "embedding", self.spec.embedding, self.embedding
        if self.input_position is not None:
            yield "position", self.spec.input_position, self.input_position
        for layer, block in zip(self.spec.layers, self.blocks):
            for role, category in block.roles:
                yield category, layer.part(role), block.parts[role]
        yield "norm", self.spec.final_norm, self.final_norm
        yield "head", self.spec.head, self.head

    def bind(self, tensors) -> "Model":
        """Give every part its tensors: `tensors[file name]` (a mapping; it may make a tensor when it is asked for it)
        is put on the device as the part's class says and handed over under the part's local name.  The one place where
        a part category's tensors reach its part, whatever their source."""
        for category, part_spec, part in self._owners():
            cls = part_class(category, part_spec.kind)
            forced = getattr(cls, "placement", lambda s: {})(part_spec)
            prefix = getattr(part_spec, "prefix", "")
            local = {}
            for name, p in cls.params(part_spec).items():
                force = {"float32": torch.float32, None: None}[forced.get(name)]
                local[name] = self.rt.place(tensors[prefix + name], p.kind, force)
            if category == "head":
                part.load(local, embedding=self.embedding)
            else:
                part.load(local)
        self.loaded = True
        return self

    def load_tensors(self, tensors: Dict[str, torch.Tensor], where: str = "the given tensors") -> "Model":
        """Bind tensors by name, checked first against what the parts declare."""
        check_tensors(where, tensors, model_params(self.spec))
        return self.bind(tensors)

    # -- forward ---------------------------------------------------------------------------
    def forward(self, batch, cache) -> Optional[torch.Tensor]:
        """Run the batch's tokens through every run of the order; float32 logits
        [wanted, vocab] at `batch.want_rows`, or None if nothing is wanted."""
        batch.step_cache.clear()
        x = self.embedding.forward(batch.tokens)
        if self.input_position is not None:
            x = self.input_position.forward(x, batch)
        pending = None
        for index, run in enumerate(self.spec.order):
            block = self.blocks[run.layer]
            view = cache.view(index, run.cache_of)
            x, pending = block.forward(x, pending, batch, view, cache.state(index))
        if batch.n_want == 0:
            return None
        ops = self.rt.ops
        if pending is not None and not (batch.want_every_row and getattr(self.final_norm, "fuses_products", False)):
            pending = self.rt.settle(pending)
        if batch.want_every_row:
            # every row in order (a step of single tokens): no gather, and the last delta is added inside the norm
            normed = (self.final_norm.forward(x, self.rt.act_dtype) if pending is None
                      else self.final_norm.add_forward(x, pending, self.rt.act_dtype))
            return self.head.forward(normed)
        if pending is not None:
            ops.residual_add(x, pending)
        rows = ops.gather_rows(x, batch.want_rows, self.rt.empty((batch.n_want, x.shape[1]), torch.float32))
        normed = self.final_norm.forward(rows, self.rt.act_dtype)
        return self.head.forward(normed)


def load_model(model_dir: str, runtime) -> Model:
    """The model of a folder with config.json and model.safetensors."""
    _, cfg = load_config(model_dir)
    model = Model(cfg.model_spec(), runtime)
    model.load_tensors(read_model_tensors(model_dir), where=model_dir)
    model.config = cfg
    return model


def random_model(config: dict, seed: int, runtime) -> Model:
    """A model with random weights made on the device, without a folder (for
    measurements at sizes whose file would be many gigabytes)."""
    from ..weights.random_init import random_tensor
    _, cfg = parse_config(config)
    spec = cfg.model_spec()
    model = Model(spec, runtime)
    expected = model_params(spec)

    class _Made(dict):
        def __missing__(self, name):
            return random_tensor(seed, name, expected[name], torch.bfloat16, device=str(runtime.device))
    model.bind(_Made())
    model.config = cfg
    return model
