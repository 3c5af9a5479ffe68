"""Token embedding and output head.

Embedding: ``x[t] = E[ids[t]]`` with no scaling and no position term
(crates/model/src/llama.rs:256-262), written straight into the 32-bit residual stream.
Head: ``logits = h * W^T`` on the selected rows, ``W`` being the embedding table when the
embeddings are tied (llama.rs:152-156); logits are float32 (llama.rs:285)."""
from __future__ import annotations

from typing import Any, Dict, List

import torch

from .. import ops
from .base import BuildContext, Embedding, Head, TensorSpec, join, project, register


@register("embedding", "token")
class TokenEmbedding(Embedding):
    """Parameters: ``vocab_size``, ``hidden_size``."""

    graph_safe = True

    @classmethod
    def tensor_specs(cls, params: Dict[str, Any], prefix: str) -> List[TensorSpec]:
        return [TensorSpec(join(prefix, "weight"), (params["vocab_size"], params["hidden_size"]))]

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        self.weight = ctx.take(join(prefix, "weight"))
        self.vocab_size = int(params["vocab_size"])

    def forward(self, ids: torch.Tensor) -> torch.Tensor:
        return ops.embed(ids, self.weight)


@register("head", "linear")
class LinearHead(Head):
    """Parameters: ``vocab_size``, ``hidden_size``, ``tied_to`` (name of the tensor to share,
    or None for a weight of its own at ``prefix.weight``)."""

    graph_safe = True

    takes_normed_input = True

    @classmethod
    def tensor_specs(cls, params: Dict[str, Any], prefix: str) -> List[TensorSpec]:
        if params.get("tied_to"):
            return []
        return [TensorSpec(join(prefix, "weight"), (params["vocab_size"], params["hidden_size"]))]

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        self.weight = ctx.take(params.get("tied_to") or join(prefix, "weight"))

    def forward(self, x: Any) -> torch.Tensor:
        return project(x, self.weight, torch.float32)
