"""Rotary position encoding with optional llama3 frequency scaling.

Inverse frequencies are computed in float32 exactly as the reference does
(crates/model/src/rope.rs:19-49): ``1 / theta^(2j/d)``; under ``llama3`` scaling a frequency
whose wavelength is below ``original / high_freq_factor`` is kept, one above
``original / low_freq_factor`` is divided by ``factor``, and those between are blended.
Angles ``position * inv_freq``, cosines and sines are float32 (rope.rs:61-78) and stay so:
the table is never rounded to the activation dtype.  The rotation pairs dim ``j`` with
``j + rot/2`` (rotate-half, rope.rs:111-117) and is applied by the cache-write kernel."""
from __future__ import annotations

import math
from typing import Any, Dict, Optional

import torch

from .base import BuildContext, PositionEncoding, register


def inverse_frequencies(rot_dim: int, theta: float, scaling: Optional[Dict[str, Any]]
                        ) -> torch.Tensor:
    f32 = torch.float32
    exponent = torch.arange(0, rot_dim, 2, dtype=f32) / torch.tensor(float(rot_dim), dtype=f32)
    inv = 1.0 / torch.pow(torch.tensor(float(theta), dtype=f32), exponent)
    if not scaling:
        return inv
    kind = scaling.get("rope_type")
    if kind != "llama3":
        raise ValueError(f"position encoding 'rope': unknown scaling '{kind}' (known: 'llama3')")
    factor = torch.tensor(float(scaling["factor"]), dtype=f32)
    low = torch.tensor(float(scaling["low_freq_factor"]), dtype=f32)
    high = torch.tensor(float(scaling["high_freq_factor"]), dtype=f32)
    old_ctx = torch.tensor(float(scaling["original_max_position_embeddings"]), dtype=f32)
    low_wavelen, high_wavelen = old_ctx / low, old_ctx / high
    wavelen = torch.tensor(2.0 * math.pi, dtype=f32) / inv
    smooth = (old_ctx / wavelen - low) / (high - low)
    blended = (1.0 - smooth) * inv / factor + smooth * inv
    return torch.where(wavelen < high_wavelen, inv,
                       torch.where(wavelen > low_wavelen, inv / factor, blended))


@register("position", "rope")
class RotaryEmbedding(PositionEncoding):
    """Parameters: ``rot_dim`` (rotated width, at most the head size), ``theta``, ``scaling``
    (None or the llama3 fields).  Holds ``cos``/``sin`` float32 ``(max_positions, rot/2)``."""

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        rot = int(params["rot_dim"])
        if rot % 2:
            raise ValueError(f"position encoding 'rope': rot_dim {rot} must be even")
        inv = inverse_frequencies(rot, params["theta"], params.get("scaling"))
        pos = torch.arange(ctx.max_positions, dtype=torch.float32).reshape(-1, 1)
        angles = pos * inv.reshape(1, -1)
        self.rot_dim = rot
        self.inv_freq = inv
        self.cos = torch.cos(angles).to(ctx.device).contiguous()
        self.sin = torch.sin(angles).to(ctx.device).contiguous()
        self.max_positions = ctx.max_positions


@register("position", "none")
class NoPosition(PositionEncoding):
    """No position encoding: queries and keys go to the cache as they are."""

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        self.rot_dim, self.cos, self.sin = 0, None, None
        self.max_positions = ctx.max_positions


def shared_position(spec, ctx: BuildContext) -> PositionEncoding:
    """One table per distinct parameter set, shared by all mixers that name it."""
    from .base import create
    key = ("position", spec.kind, repr(sorted(spec.params.items(), key=lambda kv: kv[0])))
    if key not in ctx.shared:
        ctx.shared[key] = create("position", spec, "", ctx)
    return ctx.shared[key]
