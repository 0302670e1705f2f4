"""Qwen2 dense decoder: the architecture name, its configuration class, and its builder.

Everything specific to the architecture is in :class:`~vipera_rs_amd.config.Qwen2Config`, which
describes the layers as data; the model itself is the generic decoder.
"""
from __future__ import annotations

from ..config.qwen2 import Qwen2Config
from ..config.registry import register_architecture
from .decoder import DecoderModel


def build_qwen2(config: Qwen2Config, runtime) -> DecoderModel:
    return DecoderModel(config, runtime)


register_architecture("Qwen2ForCausalLM", Qwen2Config, build_qwen2)
