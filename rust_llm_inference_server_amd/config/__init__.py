"""Typed configurations: the model's (from config.json) and the engine's."""
import json
import os
from typing import List

from .engine import EngineConfig
from .errors import ConfigError
from .generation import read_eos_token_ids
from .llama import LlamaConfig, RopeScaling

_PRESET_DIR = os.path.join(os.path.dirname(__file__), "presets")


def preset_names() -> List[str]:
    return sorted(f[:-5] for f in os.listdir(_PRESET_DIR) if f.endswith(".json"))


def preset_dict(name: str) -> dict:
    """A named config.json that ships with the package (the shapes the benchmarks use)."""
    path = os.path.join(_PRESET_DIR, name + ".json")
    if not os.path.exists(path):
        raise ConfigError(f"unknown preset '{name}' (known: {', '.join(preset_names())})")
    with open(path, "r", encoding="utf-8") as f:
        return json.load(f)


__all__ = ["ConfigError", "EngineConfig", "LlamaConfig", "RopeScaling", "preset_dict",
           "read_eos_token_ids",
           "preset_names"]
