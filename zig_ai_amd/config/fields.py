"""Typed access to the keys of a config.json dictionary."""

from __future__ import annotations

from typing import Any, Iterable, Mapping, Sequence

from .spec import ConfigError

_MISSING = object()


def _first_present(data: Mapping[str, Any], names: Sequence[str]) -> Any:
    for name in names:
        if name in data and data[name] is not None:
            return name, data[name]
    return None, _MISSING


def read_int(data: Mapping[str, Any], names: Sequence[str], default: Any = _MISSING,
             minimum: int | None = None) -> int:
    name, value = _first_present(data, names)
    if value is _MISSING:
        if default is _MISSING:
            raise ConfigError(f"config.json has no {' / '.join(names)}")
        return default
    if isinstance(value, bool) or not isinstance(value, int):
        if isinstance(value, float) and value == int(value):
            value = int(value)
        else:
            raise ConfigError(f"{name} must be an integer, got {value!r}")
    if minimum is not None and value < minimum:
        raise ConfigError(f"{name} must be at least {minimum}, got {value}")
    return value


def read_float(data: Mapping[str, Any], names: Sequence[str], default: Any = _MISSING,
               positive: bool = False) -> float:
    name, value = _first_present(data, names)
    if value is _MISSING:
        if default is _MISSING:
            raise ConfigError(f"config.json has no {' / '.join(names)}")
        return default
    if isinstance(value, bool) or not isinstance(value, (int, float)):
        raise ConfigError(f"{name} must be a number, got {value!r}")
    value = float(value)
    if positive and not value > 0.0:
        raise ConfigError(f"{name} must be positive, got {value}")
    return value


def read_bool(data: Mapping[str, Any], names: Sequence[str], default: Any = _MISSING) -> bool:
    name, value = _first_present(data, names)
    if value is _MISSING:
        if default is _MISSING:
            raise ConfigError(f"config.json has no {' / '.join(names)}")
        return default
    if not isinstance(value, bool):
        raise ConfigError(f"{name} must be true or false, got {value!r}")
    return value


def read_str_list(data: Mapping[str, Any], names: Sequence[str], default: Any = _MISSING) -> list:
    name, value = _first_present(data, names)
    if value is _MISSING:
        if default is _MISSING:
            raise ConfigError(f"config.json has no {' / '.join(names)}")
        return default
    if not isinstance(value, (list, tuple)) or not all(isinstance(v, str) for v in value):
        raise ConfigError(f"{name} must be a list of strings, got {value!r}")
    return list(value)


def read_int_list(data: Mapping[str, Any], names: Sequence[str], default: Any = _MISSING) -> list:
    name, value = _first_present(data, names)
    if value is _MISSING:
        if default is _MISSING:
            raise ConfigError(f"config.json has no {' / '.join(names)}")
        return default
    if not isinstance(value, (list, tuple)) or not all(
            isinstance(v, int) and not isinstance(v, bool) for v in value):
        raise ConfigError(f"{name} must be a list of integers, got {value!r}")
    return list(value)


def has_any(data: Mapping[str, Any], names: Iterable[str]) -> bool:
    return any(n in data and data[n] is not None for n in names)
