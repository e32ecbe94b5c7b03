"""Helpers for typed configurations read from a model folder's config.json.

Every architecture's configuration class reads its own keys with these
helpers, so that a missing or ill-typed key is reported by name, in the manner
of the reference's ``"missing/invalid metadata: <key>"``
(/root/reference/core/src/model/loader.cpp:641-654).
"""
from __future__ import annotations

import json
import os
from typing import Any, Mapping


class ConfigError(ValueError):
    """A config.json that cannot be turned into a typed configuration."""


_MISSING = object()


def read_key(d: Mapping[str, Any], key: str, kind, default=_MISSING):
    """``d[key]`` converted to ``kind`` (int, float, bool, str).

    A key that is absent (or null) takes ``default``; without a default it is
    an error.  Booleans are not accepted as numbers and numbers not as
    booleans; an integer key refuses a fractional value.
    """
    v = d.get(key, None)
    if v is None:
        if default is _MISSING:
            raise ConfigError(f"missing/invalid config key: {key}")
        return default
    if kind is bool:
        if isinstance(v, bool):
            return v
    elif kind is int:
        if isinstance(v, int) and not isinstance(v, bool):
            return int(v)
        if isinstance(v, float) and float(v).is_integer():
            return int(v)
    elif kind is float:
        if isinstance(v, (int, float)) and not isinstance(v, bool):
            return float(v)
    elif kind is str:
        if isinstance(v, str):
            return v
    raise ConfigError(f"missing/invalid config key: {key} (found {v!r}, want {kind.__name__})")


def read_config_json(folder: str) -> dict:
    path = os.path.join(folder, "config.json")
    try:
        with open(path) as f:
            d = json.load(f)
    except FileNotFoundError:
        raise ConfigError(f"no config.json in {folder}") from None
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path}: not valid JSON ({e})") from None
    if not isinstance(d, dict):
        raise ConfigError(f"{path}: the top level must be an object")
    return d


def merge_generation_config(folder: str, d: dict) -> dict:
    """config.json's dict with the stop ids of the folder's generation_config.json (when there is
    one) added to ``eos_token_id``: model folders keep the ids that end a turn there, often more
    than config.json names.  Ids of config.json come first; nothing else is taken from the file."""
    path = os.path.join(folder, "generation_config.json")
    if not os.path.isfile(path):
        return d
    try:
        with open(path) as f:
            g = json.load(f)
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path}: not valid JSON ({e})") from None
    if not isinstance(g, dict):
        raise ConfigError(f"{path}: the top level must be an object")
    more = token_id_list(g.get("eos_token_id"), "eos_token_id (generation_config.json)")
    if not more:
        return d
    have = token_id_list(d.get("eos_token_id"), "eos_token_id")
    merged = list(have) + [t for t in more if t not in have]
    out = dict(d)
    out["eos_token_id"] = merged[0] if len(merged) == 1 else merged
    return out


def token_id_list(v, key: str) -> tuple:
    """``eos_token_id`` style values: null, one id, or a list of ids."""
    if v is None:
        return ()
    if isinstance(v, int) and not isinstance(v, bool):
        return (int(v),)
    if isinstance(v, (list, tuple)) and all(isinstance(t, int) and not isinstance(t, bool) for t in v):
        return tuple(int(t) for t in v)
    raise ConfigError(f"missing/invalid config key: {key} (found {v!r}, want an id or a list of ids)")
