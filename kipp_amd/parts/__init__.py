"""The parts a layer is put together from, each chosen by the `kind` of its spec."""
from .base import (CATEGORIES, ParamSpec, build_part, part_class, part_params,
                   register, unregister)
from . import norm, position, mixer, feed_forward, block, embedding  # noqa: F401  (register the parts)
