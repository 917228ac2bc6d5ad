"""One registry from the architecture's name (``config.json["architectures"][0]``) to its model.

Reference: ``jllm/model/weights.py:59-65`` (reading the name, error when absent) and
``:161-170`` (dispatch, error for an unknown name).  An entry holds the typed
configuration class and the function that turns a configuration into a ``ModelSpec``
(the list of layers, their parts and the order they run in).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Mapping

from .errors import ConfigError
from .model import read_config_json


@dataclass(frozen=True)
class Architecture:
    name: str
    config_from_dict: Callable[[Mapping[str, Any]], Any]
    build_spec: Callable[[Any], Any]


_ARCHITECTURES: dict[str, Architecture] = {}


def register_architecture(name: str, config_from_dict, build_spec) -> None:
    _ARCHITECTURES[name] = Architecture(name, config_from_dict, build_spec)


def architecture_name(config: Mapping[str, Any], where: str = "config.json") -> str:
    archs = config.get("architectures") or []
    if not archs:
        raise ConfigError(f"no 'architectures' field in {where}")
    return archs[0]


def get_architecture(name: str) -> Architecture:
    _ensure_builtin()
    if name not in _ARCHITECTURES:
        raise ConfigError(f"unsupported architecture: {name!r}. Supported: {', '.join(sorted(_ARCHITECTURES))}")
    return _ARCHITECTURES[name]


def supported_architectures() -> list[str]:
    _ensure_builtin()
    return sorted(_ARCHITECTURES)


def resolve(path_or_dict):
    """(architecture, typed config, raw dict) of a model folder, config file or dict."""
    raw = dict(path_or_dict) if isinstance(path_or_dict, Mapping) else read_config_json(path_or_dict)
    arch = get_architecture(architecture_name(raw, str(path_or_dict) if not isinstance(path_or_dict, Mapping) else "config"))
    return arch, arch.config_from_dict(raw), raw


def _ensure_builtin() -> None:
    from .. import models  # noqa: F401  (registers the built-in architectures)
