"""Arrangements of a layer's parts.

``prenorm``: ``x += mixer(norm_1(x)); x += ffn(norm_2(x))``, the pre-norm residual block of the
reference (crates/vipera-backend-cpu/src/model.rs:3-4, 975-1198).
"""
from __future__ import annotations

from typing import List

from ..config.base import LayerSpec
from ..weights.checkpoint import TensorSpec
from .base import Block, part_class, register_block


class PreNormBlock(Block):
    def __init__(self, spec: LayerSpec, runtime):
        super().__init__(spec, runtime)
        self.mixer_norm = part_class("norm", spec.mixer_norm.kind)(spec.mixer_norm, spec.prefix, runtime)
        self.mixer = part_class("mixer", spec.mixer.kind)(spec.mixer, spec.prefix, runtime)
        self.ffn_norm = part_class("norm", spec.ffn_norm.kind)(spec.ffn_norm, spec.prefix, runtime)
        self.ffn = part_class("ffn", spec.ffn.kind)(spec.ffn, spec.prefix, runtime)
        self.position = part_class("position", spec.position.kind)(spec.position, spec.prefix, runtime)

    @classmethod
    def declare(cls, spec: LayerSpec) -> List[TensorSpec]:
        out: List[TensorSpec] = []
        out += part_class("norm", spec.mixer_norm.kind).declare(spec.mixer_norm, spec.prefix)
        out += part_class("mixer", spec.mixer.kind).declare(spec.mixer, spec.prefix)
        out += part_class("norm", spec.ffn_norm.kind).declare(spec.ffn_norm, spec.prefix)
        out += part_class("ffn", spec.ffn.kind).declare(spec.ffn, spec.prefix)
        out += part_class("position", spec.position.kind).declare(spec.position, spec.prefix)
        return out

    def load(self, tensors) -> None:
        for part in (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn, self.position):
            part.load(tensors)

    def forward(self, x, batch, cache, state, reads_only: bool = False) -> None:
        h = self.mixer_norm.forward(x)
        # with a few tokens the second norm may be split between the mixer's last product and the feed-forward's
        # first, if all three can (see NormHandoff); otherwise it is a kernel of its own
        handoff = None
        if self.mixer.fills_handoff and self.ffn.accepts_handoff(x.shape[0]):
            handoff = self.ffn_norm.handoff(x.shape[0])
        if handoff is None:
            self.mixer.forward(h, batch, cache, state, self.position, x, reads_only)
        else:
            self.mixer.forward(h, batch, cache, state, self.position, x, reads_only, handoff=handoff)
        if handoff is not None and handoff.groups:
            self.ffn.forward(None, batch, x, handoff=handoff)
        else:
            h = self.ffn_norm.forward(x)
            self.ffn.forward(h, batch, x)


register_block("prenorm", PreNormBlock)
