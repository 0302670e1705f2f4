"""A small, whole inference engine for one MI355X GPU: the Qwen2 dense decoder from a request's
tokens to its next token.

Subpackages: ``config`` (typed configuration, architecture registry), ``weights`` (safetensors by
tensor name, seeded random weights), ``parts`` (mixer, feed-forward, norm, position encoding,
block), ``models`` (the generic decoder and the registered architectures), ``cache`` (pages, block
tables, state slots), ``engine`` (step function, scheduler, generation), ``sampling``, ``ops``
(bindings of the HIP kernels in ``csrc``).
"""
from . import errors  # noqa: F401

__version__ = "0.1.0"


def __getattr__(name):
    # heavy parts are imported on first use
    if name == "Engine":
        from .engine.engine import Engine
        return Engine
    if name == "SamplingParams":
        from .sampling.sampler import SamplingParams
        return SamplingParams
    if name == "ModelRunner":
        from .engine.runner import ModelRunner
        return ModelRunner
    raise AttributeError(name)
