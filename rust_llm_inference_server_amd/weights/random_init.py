"""Random weights from a specification and a seed, in memory or as a model folder
(``config.json`` + ``model.safetensors``) that the ordinary loader reads back.

Distributions: ``normal`` tensors (linear and embedding weights) are N(0, std) with the
spec's std (0.02), ``ones_normal`` tensors (norm weights) 1 + N(0, std).  Every value is a
function of (seed, index of the tensor in the specification's list, index of the element)
alone: a counter-based hash (splitmix64) gives two uniforms per pair of elements and Box-Muller
turns them into two normals, in double precision, rounded once to float32 (the formula is
written out in ``csrc/runtime/random_fill.cpp``, which computes it on as many threads as the
machine has).  So a tensor's values depend neither on which other tensors follow it, nor on the
number of threads, nor on a library's generator, and any other implementation of those few lines
reproduces them.  (The reference's tests draw from an empty ``VarMap``, whose distribution its
text does not state: crates/engine/src/testing.rs:68-77.)"""
from __future__ import annotations

import json
import os
from typing import Dict, Sequence

import torch

from ..parts.base import TensorSpec
from .safetensors_io import save_file


def normal_fill(numel: int, seed: int, tensor_index: int, mean: float, std: float,
                threads: int = 0) -> torch.Tensor:
    """``numel`` float32 values ``mean + std * N(0, 1)`` keyed by (seed, tensor index, element
    index); ``threads`` 0 uses all the machine has (the values do not depend on it)."""
    from ..cache.manager import runtime
    out = torch.empty(numel, dtype=torch.float32)
    mask = (1 << 64) - 1
    if runtime().rlis_fill_normal(out.data_ptr(), numel, int(seed) & mask, int(tensor_index) & mask,
                                  float(mean), float(std), int(threads)) != 0:
        raise RuntimeError("rlis_fill_normal refused its arguments")
    return out


def random_tensor(spec: TensorSpec, seed: int, dtype: torch.dtype,
                  device: torch.device = torch.device("cpu"), index: int = 0) -> torch.Tensor:
    """The tensor ``spec`` describes, ``index`` being its place in the specification's list.
    Values are made in float32 on the host, then rounded to ``dtype`` and moved; for a tensor
    that is to live on the GPU they are made there, by the same formula (a model of billions of
    weights is then ready in a moment)."""
    if device.type == "cuda" and spec.init in ("normal", "ones_normal"):
        from .. import ops
        with torch.cuda.device(device):
            t = torch.empty(tuple(spec.shape), dtype=dtype, device=device)
            ops.fill_normal(t, seed, index, 1.0 if spec.init == "ones_normal" else 0.0, spec.std)
        return t
    numel = 1
    for n in spec.shape:
        numel *= int(n)
    if spec.init == "normal":
        t = normal_fill(numel, seed, index, 0.0, spec.std)
    elif spec.init == "ones_normal":
        t = normal_fill(numel, seed, index, 1.0, spec.std)
    elif spec.init == "zeros":
        t = torch.zeros(numel, dtype=torch.float32)
    else:
        raise ValueError(f"tensor '{spec.name}': unknown init '{spec.init}'")
    return t.reshape(tuple(spec.shape)).to(dtype).to(device)


def random_weights(specs: Sequence[TensorSpec], seed: int, dtype: torch.dtype,
                   device: torch.device = torch.device("cpu")) -> Dict[str, torch.Tensor]:
    return {s.name: random_tensor(s, seed, dtype, device, index=i) for i, s in enumerate(specs)}


def write_model_folder(folder: str, config_dict: dict, specs: Sequence[TensorSpec], seed: int,
                       dtype: torch.dtype = torch.float32) -> None:
    """Create ``folder`` with ``config.json`` and ``model.safetensors`` of random weights."""
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as f:
        json.dump(config_dict, f, indent=1)
    save_file(random_weights(specs, seed, dtype), os.path.join(folder, "model.safetensors"),
              metadata={"format": "pt", "seed": str(seed)})
