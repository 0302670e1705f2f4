"""One registry from an architecture's name to its configuration class and model builder.

The reference picks the block layout by a match on the architecture string and
refuses an unknown one by name (crates/vipera-backend-cpu/src/model.rs:1323-1328);
its samplers sit in a by-name registry that lists its names in registration order
(crates/vipera-traits/src/sampler.rs:98-132).  This registry works the same way
for model architectures.
"""
from __future__ import annotations

from typing import Any, Callable, Dict, List, Tuple, Type

from ..errors import InvalidArgumentError, UnsupportedError
from .base import ModelConfig, read_config_json

_ARCHITECTURES: Dict[str, Tuple[Type[ModelConfig], Callable[..., Any]]] = {}


def register_architecture(name: str, config_class: Type[ModelConfig], builder: Callable[..., Any]) -> None:
    """Register ``name`` (the string in ``config.json``'s ``architectures``).

    ``builder(config, runtime)`` returns the model; it is called by
    :func:`vipera_rs_amd.models.build_model`.
    """
    _ARCHITECTURES[name] = (config_class, builder)


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def architecture_names() -> List[str]:
    return list(_ARCHITECTURES)


def lookup_architecture(name: str) -> Tuple[Type[ModelConfig], Callable[..., Any]]:
    if name not in _ARCHITECTURES:
        known = ", ".join(architecture_names()) or "(none)"
        raise UnsupportedError(f"architecture \"{name}\" is not registered; registered: {known}")
    return _ARCHITECTURES[name]


def architecture_of(data: Dict[str, Any]) -> str:
    names = data.get("architectures")
    if not isinstance(names, list) or not names or not isinstance(names[0], str):
        raise InvalidArgumentError(
            f"config.json: key \"architectures\" is {names!r}, expected a list holding the model's class name"
        )
    return names[0]


def config_from_dict(data: Dict[str, Any]) -> ModelConfig:
    config_class, _ = lookup_architecture(architecture_of(data))
    return config_class.from_dict(data)


def load_config(folder: str) -> ModelConfig:
    """Read ``<folder>/config.json`` and return the typed configuration of its architecture."""
    return config_from_dict(read_config_json(folder))
