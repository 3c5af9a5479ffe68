"""RMSNorm: ``y = x * rsqrt(mean(x^2) + eps) * w`` over the hidden axis; the weight multiplies
directly, not as ``1 + w`` (crates/model/src/layers.rs:103-122, 141-146).  The input is the
32-bit residual stream; statistics and both multiplies are 32-bit, one rounding at the store."""
from __future__ import annotations

from typing import Any, Dict, List, Optional

import torch

from .. import ops
from .base import BuildContext, Norm, ResidualStream, TensorSpec, join, register


@register("norm", "rmsnorm")
class RMSNorm(Norm):
    """Parameters: ``size`` (hidden width), ``eps``."""

    graph_safe = True

    @classmethod
    def tensor_specs(cls, params: Dict[str, Any], prefix: str) -> List[TensorSpec]:
        return [TensorSpec(join(prefix, "weight"), (params["size"],), init="ones_normal")]

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        self.eps = float(params["eps"])
        self.weight = ctx.take(join(prefix, "weight"))
        self.out_dtype = ctx.act_dtype

    def forward(self, stream: ResidualStream) -> torch.Tensor:
        delta, stream.pending = stream.delta(), None
        return ops.add_rmsnorm(stream.x, delta, self.weight, self.eps, self.out_dtype,
                               round_parts=stream.round_parts)

    def forward_rows(self, stream: ResidualStream, rows: torch.Tensor) -> torch.Tensor:
        return ops.add_rmsnorm(stream.x, stream.delta(), self.weight, self.eps, self.out_dtype,
                               rows=rows, round_parts=stream.round_parts)

    def fused_linear(self, stream: ResidualStream, w: torch.Tensor, out_dtype: torch.dtype,
                     gated: bool, rows: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
        if self.out_dtype != torch.bfloat16:
            return None
        product = stream.pending
        if isinstance(product, ops.PendingProduct) and rows is None \
                and ops.can_join_norm_linear(product, stream.x, w):
            # The product in front adds itself to the residual and leaves the rows times this
            # norm's weight and their sums of squares; the product behind scales by them.
            xw, ss = ops.linear_join_norm(product, stream.x, self.weight, stream.round_parts)
            stream.pending = None
            return ops.linear_scaled(xw, ss, self.eps, w, out_dtype, gated=gated)
        count = stream.x.shape[0] if rows is None else rows.numel()
        if not ops.can_fuse_norm_linear(stream.x, w, count):
            return None
        y, total = ops.norm_linear(stream.x, stream.delta(), self.weight, self.eps, w, out_dtype,
                                   gated=gated, rows=rows, round_parts=stream.round_parts)
        if rows is None:
            stream.x, stream.pending = total, None
        return y
