"""One registry from an architecture's name to its configuration and model.

The reference hard-codes ``model_type == "qwen3"`` in two places
(``src/model/config.cpp:11-13,40-42``); here an architecture registers a name
(config.json's ``architectures[0]``), optional ``model_type`` aliases, a typed
configuration reader and a spec builder, and everything else looks models up
by name.
"""

from __future__ import annotations

import dataclasses
from typing import Any, Callable, Dict, Mapping, Tuple

from ..errors import InvalidArgument, LoadError, UnsupportedError


@dataclasses.dataclass(frozen=True)
class Architecture:
    name: str
    model_types: Tuple[str, ...]
    read_config: Callable[[Mapping[str, Any]], Any]   # config.json values -> typed configuration
    build_spec: Callable[[Any], Any]                  # typed configuration -> ModelSpec


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(name: str, read_config, build_spec, model_types=()) -> Architecture:
    """Registers an architecture; registering a name twice replaces the earlier entry."""
    if not name:
        raise InvalidArgument("an architecture needs a name")
    arch = Architecture(name, tuple(model_types), read_config, build_spec)
    _ARCHITECTURES[name] = arch
    return arch


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def supported_architectures() -> Tuple[str, ...]:
    return tuple(sorted(_ARCHITECTURES))


def resolve_architecture(values: Mapping[str, Any]) -> Architecture:
    """Finds the architecture a config.json names.

    ``architectures[0]`` decides; a file without it falls back to ``model_type``
    (the only key the reference reads, ``config.cpp:39``). An unknown name is an
    UnsupportedError that lists what is registered.
    """
    names = values.get("architectures")
    if names is not None:
        if not isinstance(names, list) or not names or not all(isinstance(n, str) for n in names):
            raise LoadError(f"config.json: 'architectures' must be a non-empty list of strings, got {names!r}")
        if names[0] in _ARCHITECTURES:
            return _ARCHITECTURES[names[0]]
        wanted = names[0]
    else:
        wanted = None
    model_type = values.get("model_type")
    if model_type is not None and not isinstance(model_type, str):
        raise LoadError(f"config.json: 'model_type' must be a string, got {model_type!r}")
    if wanted is None:
        if model_type is None:
            raise LoadError("config.json has neither 'architectures' nor 'model_type'")
        for arch in _ARCHITECTURES.values():
            if model_type in arch.model_types:
                return arch
        wanted = model_type
    raise UnsupportedError(
        f"architecture '{wanted}' is not supported (supported: {', '.join(supported_architectures()) or 'none'})")
