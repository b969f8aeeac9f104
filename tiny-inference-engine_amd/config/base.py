"""Reading typed values out of a config.json dictionary.

A missing required key and a value of the wrong JSON type are both LoadErrors
that name the key, as in the reference's parser (``src/model/config.cpp:32-35,64-66``).
"""

from __future__ import annotations

import json
import math
import pathlib
from typing import Any, Mapping

from ..errors import LoadError

_MISSING = object()


class ConfigReader:
    """Typed access to the keys of one config.json."""

    def __init__(self, values: Mapping[str, Any], source: str = "config.json"):
        if not isinstance(values, Mapping):
            raise LoadError(f"{source}: the top level must be a JSON object, got {type(values).__name__}")
        self._values = values
        self._source = source

    def has(self, key: str) -> bool:
        return key in self._values and self._values[key] is not None

    def raw(self, key: str, default: Any = None) -> Any:
        return self._values.get(key, default)

    def _get(self, key: str, default: Any):
        if key not in self._values or self._values[key] is None:
            if default is _MISSING:
                raise LoadError(f"{self._source} has no '{key}'")
            return default, False
        return self._values[key], True

    def integer(self, key: str, default: Any = _MISSING) -> int:
        value, present = self._get(key, default)
        if not present:
            return value
        if isinstance(value, bool) or not isinstance(value, int):
            if isinstance(value, float) and value.is_integer():
                return int(value)
            raise LoadError(f"{self._source}: '{key}' must be an integer, got {value!r}")
        return value

    def number(self, key: str, default: Any = _MISSING) -> float:
        value, present = self._get(key, default)
        if not present:
            return value
        if isinstance(value, bool) or not isinstance(value, (int, float)):
            raise LoadError(f"{self._source}: '{key}' must be a number, got {value!r}")
        value = float(value)
        if not math.isfinite(value):
            raise LoadError(f"{self._source}: '{key}' must be finite, got {value!r}")
        return value

    def boolean(self, key: str, default: Any = _MISSING) -> bool:
        value, present = self._get(key, default)
        if not present:
            return value
        if not isinstance(value, bool):
            raise LoadError(f"{self._source}: '{key}' must be true or false, got {value!r}")
        return value

    def string(self, key: str, default: Any = _MISSING) -> str:
        value, present = self._get(key, default)
        if not present:
            return value
        if not isinstance(value, str):
            raise LoadError(f"{self._source}: '{key}' must be a string, got {value!r}")
        return value

    def string_list(self, key: str, default: Any = _MISSING) -> list:
        value, present = self._get(key, default)
        if not present:
            return value
        if not isinstance(value, list) or not all(isinstance(v, str) for v in value):
            raise LoadError(f"{self._source}: '{key}' must be a list of strings, got {value!r}")
        return list(value)


def read_config_json(path) -> dict:
    """Parses a config.json file into a dictionary; malformed JSON is a LoadError naming the file."""
    path = pathlib.Path(path)
    try:
        text = path.read_text()
    except OSError as e:
        raise LoadError(f"cannot read {path}: {e.strerror or e}") from None
    try:
        values = json.loads(text)
    except json.JSONDecodeError as e:
        raise LoadError(f"{path}: not valid JSON ({e})") from None
    if not isinstance(values, dict):
        raise LoadError(f"{path}: the top level must be a JSON object")
    return values
