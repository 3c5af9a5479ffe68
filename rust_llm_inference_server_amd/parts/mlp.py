"""SwiGLU feed-forward: ``down(silu(gate(x)) * up(x))`` with three bias-free projections
(crates/model/src/layers.rs:156-187).  Gate and up run as one product over the row-concatenated
weights; ``silu`` and the product are 32-bit with one rounding."""
from __future__ import annotations

from typing import Any, Dict, List

import torch

from .. import ops
from .base import BuildContext, FeedForward, TensorSpec, join, project, register


@register("feed_forward", "swiglu")
class SwiGLU(FeedForward):
    """Parameters: ``hidden_size``, ``intermediate_size``."""

    graph_safe = True

    takes_normed_input = True

    @classmethod
    def tensor_specs(cls, params: Dict[str, Any], prefix: str) -> List[TensorSpec]:
        H, I = params["hidden_size"], params["intermediate_size"]
        return [TensorSpec(join(prefix, "gate_proj.weight"), (I, H)),
                TensorSpec(join(prefix, "up_proj.weight"), (I, H)),
                TensorSpec(join(prefix, "down_proj.weight"), (H, I))]

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        gate = ctx.weights.pop(join(prefix, "gate_proj.weight"))
        up = ctx.weights.pop(join(prefix, "up_proj.weight"))
        if gate.dtype != up.dtype:
            gate, up = gate.to(torch.float32), up.to(torch.float32)
        self.w_gate_up = torch.cat([gate, up], dim=0).contiguous()
        del gate, up
        self.w_down = ctx.take(join(prefix, "down_proj.weight"))
        self.act_dtype = ctx.act_dtype

    def forward(self, x: Any, step: Any) -> torch.Tensor:
        hidden = project(x, self.w_gate_up, self.act_dtype, gated=True)
        return ops.pending_linear(hidden, self.w_down, self.act_dtype)
