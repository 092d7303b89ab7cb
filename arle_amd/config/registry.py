"""One registry from the architecture's name in config.json to its configuration class and recipe.

`config.json["architectures"]` is searched in order and the first registered name wins
(infer/src/model_registry.rs:189-249).  An unknown name is an error that repeats it
(:234-236); a missing field is an error too (:251).
"""
from __future__ import annotations

import os
from dataclasses import dataclass
from typing import Callable

from .base import ConfigError, read_json_file, read_stop_token_ids


@dataclass(frozen=True)
class Architecture:
    name: str
    config_class: type        # has from_dict(raw) and to_dict()
    recipe: Callable          # (config, stop_token_ids) -> ModelSpec


_ARCHITECTURES: dict = {}


def register_architecture(name: str, config_class: type, recipe: Callable) -> None:
    _ARCHITECTURES[name] = Architecture(name, config_class, recipe)


def known_architectures() -> list:
    return sorted(_ARCHITECTURES)


def detect_architecture(raw: dict) -> Architecture:
    names = raw.get("architectures") if isinstance(raw, dict) else None
    if names is None:
        raise ConfigError("config.json has no `architectures` field")
    if not isinstance(names, list) or not all(isinstance(n, str) for n in names):
        raise ConfigError("config.json field `architectures` must be a list of strings")
    for n in names:
        if n in _ARCHITECTURES:
            return _ARCHITECTURES[n]
    raise ConfigError(f"unknown architectures: {names!r} (known: {known_architectures()})")


def load_model_config(model_dir: str):
    """Read `model_dir/config.json`; returns (Architecture, typed config, stop token ids)."""
    raw = read_json_file(os.path.join(model_dir, "config.json"))
    arch = detect_architecture(raw)
    config = arch.config_class.from_dict(raw)
    stops = read_stop_token_ids(model_dir, getattr(config, "eos_token_id", None))
    return arch, config, stops
