"""One registry from an architecture's name to its configuration class and model builder.

The reference detects the pipeline from config.json's `model_type` and lets every
unknown string fall through to Qwen3 (crates/synaptix/src/facade/arch.rs:73-83).  Here an
unknown name is an error that lists the known ones.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Callable

from .errors import ConfigError


@dataclass(frozen=True)
class Architecture:
    name: str                 # config.json: architectures[0]
    model_types: tuple        # config.json: model_type values that mean the same
    config_cls: type          # has from_dict(dict) and to_dict()
    build: Callable           # build(config) -> DecoderModel without weights


_BY_NAME: dict = {}


def register_architecture(name: str, config_cls: type, build: Callable, model_types=()) -> Architecture:
    arch = Architecture(name, tuple(model_types), config_cls, build)
    _BY_NAME[name] = arch
    return arch


def known_architectures() -> list:
    return sorted(_BY_NAME)


def resolve_architecture(config: dict) -> Architecture:
    """`architectures[0]` decides; `model_type` is the fallback when it is absent."""
    names = config.get("architectures") or []
    if isinstance(names, str):
        names = [names]
    for n in names:
        if n in _BY_NAME:
            return _BY_NAME[n]
    mt = config.get("model_type")
    if not names and mt is not None:
        for arch in _BY_NAME.values():
            if mt in arch.model_types:
                return arch
    asked = names[0] if names else mt
    raise ConfigError(f"unknown architecture {asked!r}; known: {', '.join(known_architectures())}")


def read_config_json(folder: str) -> dict:
    path = os.path.join(folder, "config.json")
    try:
        with open(path) as f:
            d = json.load(f)
    except OSError as e:
        raise ConfigError(f"read {path}: {e}") from None
    except json.JSONDecodeError as e:
        raise ConfigError(f"parse {path}: {e}") from None
    if not isinstance(d, dict):
        raise ConfigError(f"parse {path}: top level is not an object")
    return d


def load_config(folder: str):
    """(architecture, typed configuration) of a model folder."""
    d = read_config_json(folder)
    arch = resolve_architecture(d)
    return arch, arch.config_cls.from_dict(d)
