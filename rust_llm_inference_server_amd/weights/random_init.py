"""Random weights from a specification and a seed, in memory or as a model folder
(``config.json`` + ``model.safetensors``) that the ordinary loader reads back.

Distributions: ``normal`` tensors (linear and embedding weights) are N(0, std) with the
spec's std (0.02), ``ones_normal`` tensors (norm weights) 1 + N(0, std).  Each tensor has a
generator of its own, seeded from the seed and the tensor's name, so a tensor's values do not
depend on which other tensors exist.  (The reference's tests draw from an empty ``VarMap``,
whose distribution its text does not state: crates/engine/src/testing.rs:68-77.)"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Dict, Sequence

import torch

from ..parts.base import TensorSpec
from .safetensors_io import save_file


def _tensor_seed(seed: int, name: str) -> int:
    h = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(h[:8], "little") & 0x7FFFFFFFFFFFFFFF


def random_tensor(spec: TensorSpec, seed: int, dtype: torch.dtype,
                  device: torch.device = torch.device("cpu")) -> torch.Tensor:
    """Values are drawn in float32 on the CPU (so they are the same everywhere), then rounded
    to ``dtype`` and moved."""
    gen = torch.Generator(device="cpu")
    gen.manual_seed(_tensor_seed(seed, spec.name))
    t = torch.randn(spec.shape, generator=gen, dtype=torch.float32) * spec.std
    if spec.init == "ones_normal":
        t += 1.0
    elif spec.init == "zeros":
        t.zero_()
    elif spec.init != "normal":
        raise ValueError(f"tensor '{spec.name}': unknown init '{spec.init}'")
    return t.to(dtype).to(device)


def random_weights(specs: Sequence[TensorSpec], seed: int, dtype: torch.dtype,
                   device: torch.device = torch.device("cpu")) -> Dict[str, torch.Tensor]:
    return {s.name: random_tensor(s, seed, dtype, device) for s in specs}


def write_model_folder(folder: str, config_dict: dict, specs: Sequence[TensorSpec], seed: int,
                       dtype: torch.dtype = torch.float32) -> None:
    """Create ``folder`` with ``config.json`` and ``model.safetensors`` of random weights."""
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as f:
        json.dump(config_dict, f, indent=1)
    save_file(random_weights(specs, seed, dtype), os.path.join(folder, "model.safetensors"),
              metadata={"format": "pt", "seed": str(seed)})
