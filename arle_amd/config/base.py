"""Typed reading of config.json: required keys, aliases, and one error type.

A configuration class declares its keys once (`Key`), and `read_keys` turns a
config.json dictionary into constructor arguments or raises `ConfigError` naming
the key.  Unknown keys are ignored, as the reference's serde structs do
(crates/qwen3-spec/src/lib.rs:94-108).
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, Callable, Sequence


class ConfigError(ValueError):
    """A config.json that cannot be used; the message names the key or the rule."""


_MISSING = object()


@dataclass(frozen=True)
class Key:
    """One config.json key: its name, accepted aliases, type, and default (if optional)."""

    name: str
    kind: type
    aliases: Sequence[str] = ()
    default: Any = _MISSING

    @property
    def required(self) -> bool:
        return self.default is _MISSING


def _coerce(key: Key, value: Any) -> Any:
    if key.kind is bool:
        if isinstance(value, bool):
            return value
    elif key.kind is int:
        if isinstance(value, int) and not isinstance(value, bool):
            return value
        if isinstance(value, float) and value == int(value):
            return int(value)
    elif key.kind is float:
        if isinstance(value, (int, float)) and not isinstance(value, bool):
            return float(value)
    elif isinstance(value, key.kind):
        return value
    raise ConfigError(
        f"missing or invalid config field `{key.name}`: expected {key.kind.__name__}, "
        f"found {value!r}"
    )


def read_keys(raw: dict, keys: Sequence[Key]) -> dict:
    """Pick `keys` out of `raw`; a missing required key is an error that names it.

    Mirrors `missing or invalid config field` of infer/src/model/qwen3/config.rs:104-110.
    """
    if not isinstance(raw, dict):
        raise ConfigError("config.json must hold a JSON object")
    out = {}
    for key in keys:
        value = _MISSING
        for name in (key.name, *key.aliases):
            if name in raw and raw[name] is not None:
                value = raw[name]
                break
        if value is _MISSING:
            if key.required:
                raise ConfigError(f"missing or invalid config field `{key.name}`")
            out[key.name] = key.default
        else:
            out[key.name] = _coerce(key, value)
    return out


def read_json_file(path: str) -> dict:
    try:
        with open(path, "r", encoding="utf-8") as fh:
            return json.load(fh)
    except FileNotFoundError as exc:
        raise ConfigError(f"failed to load config from {path}: no such file") from exc
    except json.JSONDecodeError as exc:
        raise ConfigError(f"failed to load config from {path}: {exc}") from exc


def read_stop_token_ids(model_dir: str, eos_token_id: int | None) -> tuple:
    """Stop ids: generation_config.json `eos_token_id` (int or list), else the config's eos.

    infer/src/model/qwen3/config.rs:87-101.
    """
    path = os.path.join(model_dir, "generation_config.json")
    if os.path.exists(path):
        try:
            raw = read_json_file(path)
        except ConfigError:
            raw = {}
        eos = raw.get("eos_token_id") if isinstance(raw, dict) else None
        if isinstance(eos, int) and not isinstance(eos, bool):
            return (eos,)
        if isinstance(eos, list):
            ids = tuple(int(t) for t in eos if isinstance(t, int) and not isinstance(t, bool))
            if ids:
                return ids
    return (eos_token_id,) if eos_token_id is not None else ()


Validator = Callable[[Any], None]
