"""Grouped-query attention over the paged cache.

As the reference's ``Attention::forward`` (crates/model/src/attention.rs:61-103): three
bias-free projections (here fused into one product over the row-concatenated weights), heads
split column-wise (column ``h * d + j`` is head ``h``, dim ``j``), rotation of q and k by
absolute position, K and V of the new tokens written to the cache before attention reads them
(crates/model/src/paged.rs:324-337), query head ``h`` using KV head ``h / group``
(attention.rs:166-171), scores scaled by ``scale``, float32 softmax, heads merged head-major,
output projection."""
from __future__ import annotations

from typing import Any, Dict, List, Optional

import torch

from .. import ops
from .base import (BuildContext, CacheBinding, CacheRequest, Mixer, PartSpec, TensorSpec, join,
                   project, register)
from .rope import shared_position


@register("mixer", "attention")
class PagedAttention(Mixer):
    """Parameters: ``hidden_size``, ``num_heads``, ``num_kv_heads``, ``head_dim``, ``scale``,
    ``window`` (None: all earlier positions), ``position`` (a PartSpec).

    What the position part may carry: ``rot_dim``, ``cos``, ``sin`` (float32 tables, a rotation
    of the first ``rot_dim`` dims of every q and k head; rot_dim 0: none), ``interleaved``
    (the rotation pairs dim 2j with 2j + 1 instead of j with j + rot/2), ``bias_slopes``
    (float32, one per query head: slope * (key position - query position) is added to the
    scores).  The reference's Llama uses the first three (crates/model/src/rope.rs:61-117)."""

    graph_safe = True
    takes_normed_input = True

    @classmethod
    def tensor_specs(cls, params: Dict[str, Any], prefix: str) -> List[TensorSpec]:
        H, nh, nkv, d = (params[k] for k in ("hidden_size", "num_heads", "num_kv_heads",
                                             "head_dim"))
        return [TensorSpec(join(prefix, "q_proj.weight"), (nh * d, H)),
                TensorSpec(join(prefix, "k_proj.weight"), (nkv * d, H)),
                TensorSpec(join(prefix, "v_proj.weight"), (nkv * d, H)),
                TensorSpec(join(prefix, "o_proj.weight"), (H, nh * d))]

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        self.num_heads = int(params["num_heads"])
        self.num_kv_heads = int(params["num_kv_heads"])
        self.head_dim = int(params["head_dim"])
        self.scale = float(params["scale"])
        self.window: Optional[int] = params.get("window")
        if self.num_heads % self.num_kv_heads:
            raise ValueError(f"attention: {self.num_heads} heads are not a multiple of "
                             f"{self.num_kv_heads} KV heads")
        q, k, v = (ctx.weights.pop(join(prefix, f"{n}_proj.weight")) for n in "qkv")
        if not (q.dtype == k.dtype == v.dtype):
            q, k, v = (t.to(torch.float32) for t in (q, k, v))
        # One product for q, k and v: the rows of the three weights, concatenated.
        self.w_qkv = torch.cat([q, k, v], dim=0).contiguous()
        del q, k, v
        self.w_o = ctx.take(join(prefix, "o_proj.weight"))
        self.act_dtype = ctx.act_dtype
        self.position = shared_position(params.get("position") or PartSpec("none"), ctx)
        if self.position.rot_dim > self.head_dim:
            raise ValueError("attention: the rotated width exceeds the head size")

        self.planner = ops.attention_planner(
            self.num_heads, self.num_kv_heads, self.head_dim, self.act_dtype,
            biased=getattr(self.position, "bias_slopes", None) is not None)

    def cache_request(self) -> CacheRequest:
        return CacheRequest.kv(self.num_kv_heads, self.head_dim, self.window)

    def step_planner(self):
        return self.planner

    def forward(self, x: Any, step: Any, binding: CacheBinding) -> torch.Tensor:
        group = step.groups[binding.group]
        qkv = project(x, self.w_qkv, self.act_dtype)
        if step.max_context > self.position.max_positions:
            raise ValueError(f"sequence of {step.max_context} positions exceeds max_seq_len "
                             f"{self.position.max_positions}")
        out = ops.rope_attention(qkv, self.num_heads, self.num_kv_heads, self.head_dim,
                                 self.position.cos, self.position.sin, step.positions,
                                 group.slots, binding.k_pages, binding.v_pages, group.page_size,
                                 group.block_tables, step, self.scale, self.window,
                                 write_kv=binding.writes, plan=step.plans.get(self.planner.key()),
                                 interleaved=bool(getattr(self.position, "interleaved", False)),
                                 bias_slopes=getattr(self.position, "bias_slopes", None),
                                 counters=binding.counters)
        return ops.pending_linear(out, self.w_o, self.act_dtype)
