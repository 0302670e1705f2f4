"""Interfaces of the parts a layer is put together from, and the registries that name them.

A part is built from a :class:`~vipera_rs_amd.config.PartSpec` (its kind and parameters), a
tensor-name prefix and a :class:`~vipera_rs_amd.runtime.Runtime`.  It knows nothing about the model
it sits in.  Before any GPU work a part can *declare* the tensors it needs (names, shapes, how they
are kept), which is what the loader checks a model folder against and what random weights are made
from.

Kinds of parts and what each must provide:

``Norm``              ``forward(x, out=None, rows=None) -> h``: ``x`` is the 32-bit residual
                      ``[tokens, width]``; ``h`` has the run's dtype; ``rows`` (int32 indices)
                      selects rows.
``PositionEncoding``  ``apply(qkv, batch, heads, kv_heads, head_dim)`` rotates (or otherwise marks)
                      the q and k heads of the fused buffer in place; ``fused_rotary()`` may return
                      ``(inv_freq, rotary_dim)`` to let a mixer fold the rotation into its cache write.
``Mixer``             ``declare_cache(spec)`` says what it keeps per request (pages, state);
                      ``forward(h, batch, cache, state, position, residual, reads_only)`` adds its
                      output to ``residual`` (32-bit, in place).
``FeedForward``       ``forward(h, batch, residual)`` adds its output to ``residual``.
``Block``             ``forward(x, batch, cache, state, reads_only)`` runs its parts on the residual ``x``;
                      it has a ``mixer`` attribute (the part whose cache the model provides) and may
                      read further parts from ``LayerSpec.extras``.
embedding             ``embed(batch) -> x``: the 32-bit residual ``[tokens, width]`` a step starts from
                      (the batch brings tokens and positions); ``reads_device_tokens`` says whether it
                      takes token ids that the sampler left on the device (``batch.token_source``).
head                  ``forward(h) -> logits`` (32-bit) and ``vocab``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict, List, Optional, Tuple, Type

import torch

from ..config.base import LayerSpec, PartSpec
from ..errors import UnsupportedError
from ..weights.checkpoint import TensorSpec


@dataclass(frozen=True)
class KVCacheSpec:
    """Keys and values in pages: per position ``kv_heads * head_dim`` keys and ``kv_heads * value_dim``
    values (``value_dim`` 0: as wide as the keys); ``window`` 0 keeps all.  ``block_size``: positions per page if the
    mixer needs a page size of its own (0: the engine's).  Layers with the same window and page size share a
    *group*: one pool of pages and one block table per request."""

    kv_heads: int
    head_dim: int
    window: int = 0
    value_dim: int = 0
    block_size: int = 0

    @property
    def value_width(self) -> int:
        return self.value_dim or self.head_dim

    def bytes_per_position(self, element: int) -> int:
        return self.kv_heads * (self.head_dim + self.value_width) * element


@dataclass(frozen=True)
class StateSpec:
    """Per-request state of fixed size: one tensor of ``shape`` and ``dtype`` per slot."""

    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32

    def bytes_per_slot(self) -> int:
        count = 1
        for dim in self.shape:
            count *= int(dim)
        return count * torch.empty(0, dtype=self.dtype).element_size()


class Part:
    kind = ""

    def __init__(self, spec: PartSpec, prefix: str, runtime):
        self.spec = spec
        self.prefix = prefix
        self.runtime = runtime

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorSpec]:
        """Tensors this part needs, by full name. No GPU is touched."""
        return []

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        """Take the declared tensors (already on the device in their kept dtype)."""

    @classmethod
    def check_supported(cls, spec: PartSpec, dtype: torch.dtype) -> None:
        """Raise :class:`~vipera_rs_amd.errors.UnsupportedError` if no kernel takes a part of ``spec`` in a run of
        ``dtype``.  From the spec alone: it is asked when a model is opened, before any weight is read, as the
        reference refuses what its backend cannot run while it reads the header
        (crates/vipera-backend-cpu/src/model.rs:1323-1328, 1367-1383)."""


@dataclass
class NormHandoff:
    """A norm whose work is split between the products around it (few tokens, see
    ``kernels.gemm_bf16_follow``): the part before the norm, while it adds into the residual ``x``, fills
    ``scaled = x * gain`` and the workgroups' sums of squares and sets ``groups``; the part after the norm takes
    ``scaled`` as its input and divides by the root mean square itself.  ``groups`` 0: not filled (the part before
    could not), and the norm runs as a kernel of its own."""
    gain: torch.Tensor
    eps: float
    scaled: torch.Tensor
    sumsq: torch.Tensor
    groups: int = 0


class Norm(Part):
    def forward(self, x: torch.Tensor, out: Optional[torch.Tensor] = None,
                rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        raise NotImplementedError

    def handoff(self, tokens: int) -> Optional[NormHandoff]:
        """A :class:`NormHandoff` for ``tokens`` rows if this norm can be split between its neighbours, else None."""
        return None


class PositionEncoding(Part):
    def fused_rotary(self):
        return None

    def step_angles(self, batch):
        """With ``fused_rotary``: a table of the step's sines and cosines that the rotation kernel may read
        instead of computing them (shared by the layers of a step), or None."""
        return None

    def apply(self, qkv: torch.Tensor, batch, heads: int, kv_heads: int, head_dim: int) -> None:
        raise NotImplementedError


class Mixer(Part):
    @classmethod
    def declare_cache(cls, spec: PartSpec) -> Tuple[Optional[KVCacheSpec], Optional[StateSpec]]:
        """What a mixer of ``spec`` keeps per request: pages of keys and values, state of fixed size, both or
        neither.  From the spec alone, so that memory can be planned before anything is built."""
        return None, None

    def cache_spec(self) -> Optional[KVCacheSpec]:
        return type(self).declare_cache(self.spec)[0]

    def state_spec(self) -> Optional[StateSpec]:
        return type(self).declare_cache(self.spec)[1]

    #: a mixer that sets this takes ``handoff=`` in ``forward`` and may fill it (see :class:`NormHandoff`)
    fills_handoff = False

    def accepts_handoff(self, tokens: int, position, batch) -> bool:
        """Whether ``forward`` takes a filled :class:`NormHandoff` of the norm before it (``incoming=``, with ``h``
        None) for a step of ``tokens`` rows."""
        return False

    def forward(self, h, batch, cache, state, position, residual, reads_only: bool = False) -> None:
        raise NotImplementedError


class FeedForward(Part):
    #: a feed-forward that sets this takes ``outgoing=`` in ``forward`` and may fill it for the next layer's first norm
    fills_handoff = False

    def accepts_handoff(self, tokens: int) -> bool:
        """Whether ``forward`` takes a filled :class:`NormHandoff` (``handoff=``, with ``h`` None) for ``tokens`` rows."""
        return False

    def forward(self, h, batch, residual) -> None:
        raise NotImplementedError


class Block:
    """An arrangement of a layer's parts. Built from a LayerSpec and the part registries."""

    kind = ""

    def __init__(self, spec: LayerSpec, runtime):
        self.spec = spec
        self.runtime = runtime

    @classmethod
    def declare(cls, spec: LayerSpec) -> List[TensorSpec]:
        raise NotImplementedError

    def load(self, tensors) -> None:
        raise NotImplementedError

    @classmethod
    def check_supported(cls, spec: LayerSpec, dtype: torch.dtype) -> None:
        """Ask every part of the layer whether the kernels take it (see :meth:`Part.check_supported`)."""
        for family, part in (("norm", spec.mixer_norm), ("mixer", spec.mixer), ("norm", spec.ffn_norm),
                             ("ffn", spec.ffn), ("position", spec.position)):
            part_class(family, part.kind).check_supported(part, dtype)

    #: a block that sets this takes ``incoming=`` and ``outgoing=`` in ``forward`` and has ``accepts_incoming`` and
    #: ``fills_outgoing`` (see :class:`NormHandoff`: its first norm prepared by the layer before, the next layer's
    #: first norm prepared by this one)
    hands_off = False

    def forward(self, x, batch, cache, state, reads_only: bool = False) -> None:
        raise NotImplementedError


# --- registries ---------------------------------------------------------------------------------
_REGISTRIES: Dict[str, Dict[str, type]] = {
    "mixer": {}, "ffn": {}, "norm": {}, "position": {}, "block": {}, "embedding": {}, "head": {},
}


def _register(family: str, kind: str, cls: type) -> None:
    cls.kind = kind
    _REGISTRIES[family][kind] = cls


def _lookup(family: str, kind: str) -> type:
    registry = _REGISTRIES[family]
    if kind not in registry:
        known = ", ".join(registry) or "(none)"
        raise UnsupportedError(f"{family} kind \"{kind}\" is not registered; registered: {known}")
    return registry[kind]


def register_mixer(kind: str, cls: Type[Mixer]) -> None:
    _register("mixer", kind, cls)


def register_ffn(kind: str, cls: Type[FeedForward]) -> None:
    _register("ffn", kind, cls)


def register_norm(kind: str, cls: Type[Norm]) -> None:
    _register("norm", kind, cls)


def register_position(kind: str, cls: Type[PositionEncoding]) -> None:
    _register("position", kind, cls)


def register_block(kind: str, cls: Type[Block]) -> None:
    _register("block", kind, cls)


def register_embedding(kind: str, cls: Type[Part]) -> None:
    _register("embedding", kind, cls)


def register_head(kind: str, cls: Type[Part]) -> None:
    _register("head", kind, cls)


def part_class(family: str, kind: str) -> type:
    return _lookup(family, kind)


def registered(family: str) -> List[str]:
    return list(_REGISTRIES[family])


def unregister(family: str, kind: str) -> None:
    _REGISTRIES[family].pop(kind, None)
