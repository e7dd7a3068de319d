"""Typed configuration: helpers that read config.json keys with clear errors.

The reference reads config.json as untyped JSON through `cfg_u64`, whose error names
the missing key (crates/denno-engine/src/model/mod.rs:79-83).  Here each architecture
has a frozen dataclass; these helpers keep that error style.
"""
from __future__ import annotations

import json
import os


class ConfigError(ValueError):
    """A config.json that cannot describe a model: names the key and the value."""


_MISSING = object()


def read_int(d: dict, key: str, default=_MISSING, aliases=(), minimum=None):
    for k in (key, *aliases):
        if k in d and d[k] is not None:
            v = d[k]
            if isinstance(v, bool) or not isinstance(v, int):
                raise ConfigError(f"config.json: key '{k}' must be an integer, got {v!r}")
            if minimum is not None and v < minimum:
                raise ConfigError(f"config.json: key '{k}' must be >= {minimum}, got {v}")
            return v
    if default is _MISSING:
        names = " (or " + ", ".join(repr(a) for a in aliases) + ")" if aliases else ""
        raise ConfigError(f"config.json: required key '{key}'{names} is missing")
    return default


def read_float(d: dict, key: str, default=_MISSING):
    if key in d and d[key] is not None:
        v = d[key]
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"config.json: key '{key}' must be a number, got {v!r}")
        return float(v)
    if default is _MISSING:
        raise ConfigError(f"config.json: required key '{key}' is missing")
    return default


def read_bool(d: dict, key: str, default):
    if key in d and d[key] is not None:
        v = d[key]
        if not isinstance(v, bool):
            raise ConfigError(f"config.json: key '{key}' must be true or false, got {v!r}")
        return v
    return default


def read_str(d: dict, key: str, default=_MISSING, choices=None):
    if key in d and d[key] is not None:
        v = d[key]
        if not isinstance(v, str):
            raise ConfigError(f"config.json: key '{key}' must be a string, got {v!r}")
        if choices is not None and v not in choices:
            raise ConfigError(
                f"config.json: key '{key}' = {v!r} is not supported; known: {sorted(choices)}")
        return v
    if default is _MISSING:
        raise ConfigError(f"config.json: required key '{key}' is missing")
    return default


def read_config_json(model_dir: str) -> dict:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"{model_dir}: no config.json")
    with open(path) as f:
        d = json.load(f)
    if not isinstance(d, dict):
        raise ConfigError(f"{path}: top level must be an object")
    return d
