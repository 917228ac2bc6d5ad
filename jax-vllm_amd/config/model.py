"""What every architecture's typed configuration is made with: reading ``config.json`` and
taking one key of it with a type check.  The configuration classes themselves live beside
their architectures under ``models/``.  Reference: ``jllm/model/weights.py:59-65`` reads the
file; the per-key checks are added here (the reference indexes the dictionary directly).
"""
from __future__ import annotations

import json
from pathlib import Path
from typing import Any, Mapping

from .errors import ConfigError


def read_config_json(path) -> dict:
    """``config.json`` of a model folder (or the file itself) as a dict."""
    p = Path(path)
    if p.is_dir():
        p = p / "config.json"
    if not p.exists():
        raise ConfigError(f"no config.json at {p}")
    try:
        data = json.loads(p.read_text())
    except json.JSONDecodeError as e:
        raise ConfigError(f"{p} is not valid JSON: {e}") from e
    if not isinstance(data, dict):
        raise ConfigError(f"{p} must hold a JSON object")
    return data


def config_value(c: Mapping[str, Any], key: str, typ, default=None, required=True):
    """``c[key]`` as ``typ`` (an int is accepted for a float); ``default`` if it is absent or null and
    not ``required``; a ``ConfigError`` that names the key otherwise."""
    if key not in c or c[key] is None:
        if required:
            raise ConfigError(f"config.json lacks the required key {key!r}")
        return default
    v = c[key]
    if typ is float and isinstance(v, int) and not isinstance(v, bool):
        v = float(v)
    if typ is int and isinstance(v, bool) or not isinstance(v, typ):
        raise ConfigError(f"config.json key {key!r} must be {typ.__name__}, got {v!r}")
    return v
