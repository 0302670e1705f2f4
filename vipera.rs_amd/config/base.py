"""Typed model configuration and the layer-by-layer description built from it.

A configuration class reads the keys of its architecture's ``config.json`` and
turns them into data that the rest of the package consumes without knowing the
architecture: a list of :class:`LayerSpec` (which mixer, feed-forward, norm and
position encoding each layer has, with every size and constant as a parameter)
and a run order, a list of :class:`ScheduleEntry`.

The reference keeps nine numbers in ``ModelConfig`` and validates them while it
reads the model file (crates/vipera-backend-cpu/src/model.rs:34-53, 1315-1401);
the checks and error texts here follow that habit: an error names the key and
the value that is wrong.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from ..errors import InvalidArgumentError, IoError, ParseError


@dataclass(frozen=True)
class PartSpec:
    """One part of a layer: the registered kind and its parameters."""

    kind: str
    params: Dict[str, Any] = field(default_factory=dict)

    def get(self, key: str, default: Any = None) -> Any:
        return self.params.get(key, default)


@dataclass(frozen=True)
class LayerSpec:
    """What one layer is made of.

    ``block`` names the arrangement of the parts (for example ``"prenorm"``:
    ``x += mixer(norm(x)); x += ffn(norm(x))``).  ``prefix`` is the tensor-name
    prefix under which the layer's weights are stored.  ``extras`` holds further
    parts by a role name for arrangements that have more than these five (norms
    after the mixer and the feed-forward, say); a block kind defines which roles
    it reads and of which family (norm, mixer, ...) each is.
    """

    block: str
    mixer: PartSpec
    ffn: PartSpec
    mixer_norm: PartSpec
    ffn_norm: PartSpec
    position: PartSpec
    prefix: str
    extras: Dict[str, PartSpec] = field(default_factory=dict)


@dataclass(frozen=True)
class ScheduleEntry:
    """One step of the run order.

    ``layer`` indexes the list of layer specs; a layer may appear more than
    once.  ``cache_of`` is ``None`` when the entry owns a cache (or state) of
    its own, else the index of the earlier schedule entry whose cache it reads
    without writing.
    """

    layer: int
    cache_of: Optional[int] = None


class ModelConfig:
    """Base of every architecture's configuration.

    Subclasses define dataclass fields named like the ``config.json`` keys and
    implement :meth:`layer_specs`; everything the generic decoder needs comes
    from the methods below.
    """

    architecture: str = ""

    # --- what a subclass must provide -------------------------------------------------
    def layer_specs(self) -> List[LayerSpec]:
        raise NotImplementedError

    def schedule(self) -> List[ScheduleEntry]:
        return [ScheduleEntry(i) for i in range(len(self.layer_specs()))]

    def embedding_spec(self) -> PartSpec:
        raise NotImplementedError

    def final_norm_spec(self) -> PartSpec:
        raise NotImplementedError

    def head_spec(self) -> PartSpec:
        raise NotImplementedError

    def validate(self) -> None:
        raise NotImplementedError

    @classmethod
    def from_dict(cls, data: Dict[str, Any]) -> "ModelConfig":
        raise NotImplementedError

    def to_dict(self) -> Dict[str, Any]:
        raise NotImplementedError

    # --- shared helpers -----------------------------------------------------------------
    @property
    def context_limit(self) -> int:
        return int(getattr(self, "max_position_embeddings"))

    def save(self, folder: str) -> None:
        os.makedirs(folder, exist_ok=True)
        with open(os.path.join(folder, "config.json"), "w") as handle:
            json.dump(self.to_dict(), handle, indent=2)
            handle.write("\n")


def read_config_json(folder: str) -> Dict[str, Any]:
    """Parse ``<folder>/config.json`` into a dict, with typed errors."""
    path = os.path.join(folder, "config.json")
    try:
        with open(path, "r") as handle:
            text = handle.read()
    except OSError as err:
        raise IoError(f"cannot read {path}: {err.strerror or err}") from None
    try:
        data = json.loads(text)
    except json.JSONDecodeError as err:
        raise ParseError(f"{path} is not valid JSON: {err}") from None
    if not isinstance(data, dict):
        raise ParseError(f"{path} must hold a JSON object")
    return data


class KeyReader:
    """Reads typed values out of a ``config.json`` dict, naming key and value on error."""

    def __init__(self, data: Dict[str, Any], where: str = "config.json"):
        self.data = data
        self.where = where

    def _fail(self, key: str, value: Any, want: str) -> InvalidArgumentError:
        return InvalidArgumentError(f"{self.where}: key \"{key}\" is {value!r}, expected {want}")

    def has(self, key: str) -> bool:
        return key in self.data and self.data[key] is not None

    def integer(self, key: str, default: Optional[int] = None, minimum: int = 0) -> int:
        if not self.has(key):
            if default is None:
                raise InvalidArgumentError(f"{self.where}: required key \"{key}\" is missing")
            return default
        value = self.data[key]
        if isinstance(value, bool) or not isinstance(value, int):
            if isinstance(value, float) and value == int(value):
                value = int(value)
            else:
                raise self._fail(key, value, "an integer")
        if value < minimum:
            raise self._fail(key, value, f"an integer of at least {minimum}")
        return value

    def number(self, key: str, default: Optional[float] = None) -> float:
        if not self.has(key):
            if default is None:
                raise InvalidArgumentError(f"{self.where}: required key \"{key}\" is missing")
            return float(default)
        value = self.data[key]
        if isinstance(value, bool) or not isinstance(value, (int, float)):
            raise self._fail(key, value, "a number")
        value = float(value)
        if value != value or value in (float("inf"), float("-inf")):
            raise self._fail(key, value, "a finite number")
        return value

    def boolean(self, key: str, default: bool) -> bool:
        if not self.has(key):
            return default
        value = self.data[key]
        if not isinstance(value, bool):
            raise self._fail(key, value, "true or false")
        return value

    def string(self, key: str, default: Optional[str] = None) -> str:
        if not self.has(key):
            if default is None:
                raise InvalidArgumentError(f"{self.where}: required key \"{key}\" is missing")
            return default
        value = self.data[key]
        if not isinstance(value, str):
            raise self._fail(key, value, "a string")
        return value
