"""kipp_amd: a small, whole inference engine for one GPU (MI355X, gfx950).

config/    typed configurations, the decoder as data, the architecture registry
weights/   safetensors by tensor name, random-weights model folders
parts/     mixer, feed-forward, norm, position encoding, block arrangements
cache/     paged key/value pools per layer group, block tables, state slots
engine/    the step function, the scheduler, generation
sampling/  greedy and temperature sampling
csrc/      hand-written HIP kernels for gfx950 and their build
"""
__version__ = "0.1.0"


def generate(*args, **kwargs):
    from .generation import generate as _generate
    return _generate(*args, **kwargs)
