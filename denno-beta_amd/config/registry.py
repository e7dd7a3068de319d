"""One registry from an architecture's name to its configuration class and model builder.

The reference dispatches on config.json's `model_type` and fails on an unknown one
(crates/denno-engine/src/model/mod.rs:88-104).  Here the key is `architectures[0]`
(what model folders name their class with), with `model_type` as the fallback.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict

from .base import ConfigError, read_config_json


@dataclass(frozen=True)
class Architecture:
    name: str
    config_cls: type          # has from_dict(dict) and to_dict()
    build: Callable           # build(config) -> parts.model.DecoderSpec


_BY_NAME: Dict[str, Architecture] = {}


def register_architecture(names, config_cls, build):
    """`names`: every string that config.json may name this architecture with
    (entries of `architectures`, or `model_type`)."""
    arch = Architecture(names[0], config_cls, build)
    for n in names:
        _BY_NAME[n] = arch
    return arch


def known_architectures():
    return sorted(_BY_NAME)


def resolve_architecture(config_json: dict) -> Architecture:
    _ensure_builtin()
    names = []
    archs = config_json.get("architectures")
    if isinstance(archs, list):
        names += [a for a in archs if isinstance(a, str)]
    if isinstance(config_json.get("model_type"), str):
        names.append(config_json["model_type"])
    for n in names:
        if n in _BY_NAME:
            return _BY_NAME[n]
    if not names:
        raise ConfigError("config.json names no architecture: neither 'architectures' nor "
                          f"'model_type' is set; known: {known_architectures()}")
    raise ConfigError(f"unsupported architecture {names}; known: {known_architectures()}")


def load_config(model_dir: str):
    """-> (Architecture, typed config) of a model folder."""
    d = read_config_json(model_dir)
    arch = resolve_architecture(d)
    return arch, arch.config_cls.from_dict(d)


def _ensure_builtin():
    # importing the models package registers what the framework ships
    from .. import models  # noqa: F401
