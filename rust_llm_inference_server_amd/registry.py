"""One registry from an architecture's name (``architectures[0]`` of config.json) to its typed
configuration and its model specification.  The reference dispatches on the file kind only
(crates/model/src/lib.rs:21-32) and matches names just for GGUF (gguf.rs:64-76); here the name
in config.json chooses the model everywhere: loader, engine, replay.

The registry names no architecture itself.  Each architecture registers from its own module
(``models/llama.py`` does for ``LlamaForCausalLM``); the modules that ship with the package are
imported, once, at the first lookup."""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import TYPE_CHECKING, Any, Callable, Dict

from .config.errors import ConfigError

if TYPE_CHECKING:
    from .models.spec import ModelSpec


@dataclass
class Architecture:
    name: str
    parse_config: Callable[[Dict[str, Any]], Any]      # config.json dict -> typed config
    build_spec: Callable[[Any], "ModelSpec"]           # typed config -> model specification
    config_to_dict: Callable[[Any], Dict[str, Any]]    # typed config -> config.json dict


_ARCHITECTURES: Dict[str, Architecture] = {}
_shipped_loaded = False


def register_architecture(arch: Architecture) -> None:
    _ARCHITECTURES[arch.name] = arch


def _load_shipped() -> None:
    """Import the package's own model modules, which register their architectures."""
    global _shipped_loaded
    if not _shipped_loaded:
        _shipped_loaded = True
        from . import models  # noqa: F401


def architecture(name: str) -> Architecture:
    _load_shipped()
    if name not in _ARCHITECTURES:
        raise ConfigError(f"architecture '{name}' is not supported "
                          f"(known: {', '.join(sorted(_ARCHITECTURES))})")
    return _ARCHITECTURES[name]


def architecture_names():
    _load_shipped()
    return sorted(_ARCHITECTURES)


def architecture_of(config_dict: Dict[str, Any]) -> Architecture:
    archs = config_dict.get("architectures")
    if not isinstance(archs, list) or not archs or not isinstance(archs[0], str):
        raise ConfigError("config.json: 'architectures' must be a non-empty list of names")
    return architecture(archs[0])


def read_config_dict(path: str) -> Dict[str, Any]:
    if os.path.isdir(path):
        path = os.path.join(path, "config.json")
    try:
        with open(path, "r", encoding="utf-8") as f:
            d = json.load(f)
    except FileNotFoundError:
        raise ConfigError(f"{path}: no such file") from None
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path}: not valid JSON ({e})") from None
    if not isinstance(d, dict):
        raise ConfigError(f"{path}: top level must be an object")
    return d
