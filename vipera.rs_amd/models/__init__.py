"""Models by architecture name."""
from __future__ import annotations

from .. import parts  # noqa: F401  (registers the built-in parts)
from ..config.base import ModelConfig
from ..config.registry import lookup_architecture
from . import qwen2  # noqa: F401  (registers the architecture)
from .decoder import CacheNeed, DecoderModel, check_model, declare_cache_needs, declare_model


def build_model(config: ModelConfig, runtime):
    """The model of ``config``'s architecture, without weights."""
    _, builder = lookup_architecture(config.architecture)
    return builder(config, runtime)


__all__ = ["CacheNeed", "DecoderModel", "build_model", "check_model", "declare_cache_needs", "declare_model"]
