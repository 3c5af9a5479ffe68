"""One registry from an architecture's name (``architectures[0]`` of config.json) to its typed
configuration and its model specification.  The reference dispatches on the file kind only
(crates/model/src/lib.rs:21-32) and matches names just for GGUF (gguf.rs:64-76); here the name
in config.json chooses the model everywhere: loader, engine, replay."""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, Callable, Dict

from .config.llama import ConfigError, LlamaConfig
from .models.llama import llama_spec
from .models.spec import ModelSpec


@dataclass
class Architecture:
    name: str
    parse_config: Callable[[Dict[str, Any]], Any]      # config.json dict -> typed config
    build_spec: Callable[[Any], ModelSpec]             # typed config -> model specification
    config_to_dict: Callable[[Any], Dict[str, Any]]    # typed config -> config.json dict


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(arch: Architecture) -> None:
    _ARCHITECTURES[arch.name] = arch


def architecture(name: str) -> Architecture:
    if name not in _ARCHITECTURES:
        raise ConfigError(f"architecture '{name}' is not supported "
                          f"(known: {', '.join(sorted(_ARCHITECTURES))})")
    return _ARCHITECTURES[name]


def architecture_names():
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


register_architecture(Architecture(
    name="LlamaForCausalLM",
    parse_config=LlamaConfig.from_dict,
    build_spec=llama_spec,
    config_to_dict=lambda cfg: cfg.to_dict(),
))
