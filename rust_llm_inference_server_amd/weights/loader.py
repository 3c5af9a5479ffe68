"""Loads a model's tensors from safetensors by name and checks them against what the model's
parts declare (``TensorSpec`` lists), with one error that lists everything wrong at once:
missing tensors, unexpected tensors and wrong shapes.

Dtype policy: floating tensors stored in 16 bits are kept (or made) bfloat16; a tensor stored
in 32 bits stays float32 (the parts take either); integer tables become int32.  In a float32
run every floating tensor is float32.  The reference casts on the CPU and uploads the final
dtype only (crates/model/src/llama.rs:33-64); so does this loader, tensor by tensor."""
from __future__ import annotations

import fnmatch
from typing import Dict, Iterable, List, Sequence

import torch

from ..parts.base import TensorSpec
from .safetensors_io import open_folder

# Buffers some exporters write beside the weights; they carry nothing the model reads.
IGNORED_PATTERNS = ("*.rotary_emb.inv_freq", "*.attn.bias", "*.attn.masked_bias")


class WeightError(ValueError):
    """The checkpoint does not hold what the model needs; the message lists every fault."""

    def __init__(self, folder: str, missing: List[str], unexpected: List[str],
                 wrong_shape: List[str]):
        self.missing, self.unexpected, self.wrong_shape = missing, unexpected, wrong_shape
        lines = [f"{folder}: the checkpoint does not match the model"]
        if missing:
            lines.append(f"  missing tensors ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong_shape:
            lines.append(f"  wrong shapes ({len(wrong_shape)}): " + "; ".join(wrong_shape))
        super().__init__("\n".join(lines))


def target_dtype(stored: torch.dtype, run_dtype: torch.dtype) -> torch.dtype:
    if stored in (torch.int64, torch.int32, torch.int16, torch.int8, torch.uint8, torch.bool):
        return torch.int32
    if run_dtype == torch.float32:
        return torch.float32
    if stored in (torch.float32, torch.float64):
        return torch.float32          # stored in 32 bits (or more): stays 32-bit
    return torch.bfloat16


def load_weights(folder: str, specs: Sequence[TensorSpec], run_dtype: torch.dtype,
                 device: torch.device, optional: Iterable[str] = ()) -> Dict[str, torch.Tensor]:
    """Tensors named by ``specs`` from the safetensors files of ``folder``, on ``device``.

    ``optional`` names tensors that may be present without being read (a stored ``lm_head``
    beside tied embeddings)."""
    files = open_folder(folder)
    where = {}
    for f in files:
        for name in f.names():
            where[name] = f
    wanted = {s.name: s for s in specs}
    optional = set(optional)
    missing = [n for n in wanted if n not in where]
    unexpected = [n for n in where
                  if n not in wanted and n not in optional
                  and not any(fnmatch.fnmatch(n, p) for p in IGNORED_PATTERNS)]
    wrong = []
    for name, spec in wanted.items():
        if name in where:
            _, shape = where[name].info(name)
            if tuple(shape) != tuple(spec.shape):
                wrong.append(f"{name}: expected shape {list(spec.shape)}, checkpoint has "
                             f"{list(shape)}")
    if missing or unexpected or wrong:
        raise WeightError(folder, sorted(missing), sorted(unexpected), wrong)
    out: Dict[str, torch.Tensor] = {}
    for name in wanted:
        t = where[name].tensor(name)
        out[name] = t.to(target_dtype(t.dtype, run_dtype)).to(device).contiguous()
        if out[name].data_ptr() == t.data_ptr():
            out[name] = out[name].clone()     # never hand out a view of the file map
    return out
