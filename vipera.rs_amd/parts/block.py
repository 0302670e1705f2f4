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

    hands_off = True

    def accepts_incoming(self, tokens: int, batch):
        """A :class:`NormHandoff` of this block's first norm for the layer before to fill, or None."""
        if not self.mixer.accepts_handoff(tokens, self.position, batch):
            return None
        return self.mixer_norm.handoff(tokens)

    def fills_outgoing(self) -> bool:
        return self.ffn.fills_handoff

    def forward(self, x, batch, cache, state, reads_only: bool = False, incoming=None, outgoing=None) -> None:
        """With a few tokens a norm may be split between the product before it and the product after it, if all
        three can (see NormHandoff); otherwise it is a kernel of its own. ``incoming``: this block's first norm,
        filled by the layer before (``groups`` > 0) or not; ``outgoing``: the next layer's first norm, for this
        block's feed-forward to fill."""
        if incoming is not None and incoming.groups:
            h = None
            mixer_kwargs = {"incoming": incoming}
        else:
            h = self.mixer_norm.forward(x)
            mixer_kwargs = {}
        between = None
        if self.mixer.fills_handoff and self.ffn.accepts_handoff(x.shape[0]):
            between = self.ffn_norm.handoff(x.shape[0])
            if between is not None:
                mixer_kwargs["handoff"] = between
        self.mixer.forward(h, batch, cache, state, self.position, x, reads_only, **mixer_kwargs)
        ffn_kwargs = {"outgoing": outgoing} if outgoing is not None and self.ffn.fills_handoff else {}
        if between is not None and between.groups:
            self.ffn.forward(None, batch, x, handoff=between, **ffn_kwargs)
        else:
            h = self.ffn_norm.forward(x)
            self.ffn.forward(h, batch, x, **ffn_kwargs)


register_block("prenorm", PreNormBlock)
