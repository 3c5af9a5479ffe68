"""The pre-norm decoder block: ``x += mixer(norm(x)); x += feed_forward(norm(x))``
(crates/model/src/llama.rs:264-271).  Which mixer, feed-forward and norms it holds, and under
which weight names, is given by its parameters, layer by layer."""
from __future__ import annotations

from typing import Any, Dict, List

from .base import (Block, BuildContext, CacheBinding, ResidualStream, TensorSpec,
                   create, join, normed, register, tensor_specs)


@register("block", "prenorm")
class PreNormBlock(Block):
    """Parameters: ``mixer``, ``feed_forward``, ``mixer_norm``, ``ffn_norm`` (PartSpecs) and
    ``names``: the weight-name suffix of each of the four under the block's prefix."""

    _SLOTS = (("mixer_norm", "norm"), ("mixer", "mixer"), ("ffn_norm", "norm"),
              ("feed_forward", "feed_forward"))

    @classmethod
    def tensor_specs(cls, params: Dict[str, Any], prefix: str) -> List[TensorSpec]:
        out: List[TensorSpec] = []
        for slot, category in cls._SLOTS:
            out += tensor_specs(category, params[slot], join(prefix, params["names"][slot]))
        return out

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        built = {slot: create(category, params[slot], join(prefix, params["names"][slot]), ctx)
                 for slot, category in self._SLOTS}
        self.mixer_norm, self.mixer = built["mixer_norm"], built["mixer"]
        self.ffn_norm, self.feed_forward = built["ffn_norm"], built["feed_forward"]

    @property
    def graph_safe(self) -> bool:
        return all(p.graph_safe for p in (self.mixer_norm, self.mixer, self.ffn_norm,
                                          self.feed_forward))

    def forward(self, stream: ResidualStream, step: Any, binding: CacheBinding) -> None:
        stream.add(self.mixer.forward(normed(self.mixer_norm, stream, self.mixer), step, binding))
        stream.add(self.feed_forward.forward(normed(self.ffn_norm, stream, self.feed_forward),
                                             step))
