"""A model as data, and the class that builds and runs it.

``ModelSpec`` lists the layers (each a block specification with its weight-name prefix) and
the *run order*: a list of ``RunEntry`` that names which layer runs when.  A layer may be
named more than once (each run then has a cache of its own), and a run may read the cache
another run writes (``cache_of``) instead of writing its own.  ``Model`` builds the parts
through the registries, groups the cache requests of the runs into page groups, and runs a
step: embedding, the run order, final norm on the wanted rows, head."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple

import torch

from ..parts.base import (Block, BuildContext, CacheRequest, PartSpec,
                          ResidualStream, TensorSpec, create, normed, tensor_specs)


@dataclass
class LayerSpec:
    block: PartSpec
    prefix: str


@dataclass
class RunEntry:
    layer: int
    # Index into the run order of the run whose cache this run reads; None: a cache of its own.
    cache_of: Optional[int] = None


@dataclass
class ModelSpec:
    hidden_size: int
    vocab_size: int
    embedding: PartSpec
    embedding_prefix: str
    layers: List[LayerSpec]
    final_norm: PartSpec
    final_norm_prefix: str
    head: PartSpec
    head_prefix: str
    run_order: Optional[List[RunEntry]] = None     # None: every layer once, in order
    # Checkpoint tensors that may be present without being read.
    optional_tensors: Tuple[str, ...] = ()

    def runs(self) -> List[RunEntry]:
        if self.run_order is not None:
            return self.run_order
        return [RunEntry(i) for i in range(len(self.layers))]

    def tensor_specs(self) -> List[TensorSpec]:
        out = tensor_specs("embedding", self.embedding, self.embedding_prefix)
        for layer in self.layers:
            out += tensor_specs("block", layer.block, layer.prefix)
        out += tensor_specs("norm", self.final_norm, self.final_norm_prefix)
        out += tensor_specs("head", self.head, self.head_prefix)
        seen, unique = set(), []
        for s in out:
            if s.name not in seen:
                seen.add(s.name)
                unique.append(s)
        return unique

    def validate(self) -> None:
        runs = self.runs()
        for i, r in enumerate(runs):
            if not 0 <= r.layer < len(self.layers):
                raise ValueError(f"run {i} names layer {r.layer}, the model has {len(self.layers)}")
            if r.cache_of is not None:
                if not 0 <= r.cache_of < i:
                    raise ValueError(f"run {i} reads the cache of run {r.cache_of}, which does "
                                     "not run before it")
                if runs[r.cache_of].cache_of is not None:
                    raise ValueError(f"run {i} reads the cache of run {r.cache_of}, which has "
                                     "none of its own")


@dataclass
class CacheGroupLayout:
    """One page group of a built model: the request its runs share and which runs write
    into which layer slot of the group's pool."""
    request: CacheRequest
    writer_runs: List[int] = field(default_factory=list)   # run index of each layer slot


@dataclass
class RunBinding:
    group: int = -1          # page group, -1: the run keeps nothing in pages
    slot: int = -1           # layer slot inside the group's pool
    writes: bool = True
    state_offset: int = -1   # byte offset of the run's state inside a request's state slot
    state_bytes: int = 0


class Model:
    """The parts of a ``ModelSpec`` on a device, and the forward pass of one step."""

    def __init__(self, spec: ModelSpec, weights: Dict[str, torch.Tensor], act_dtype: torch.dtype,
                 device: torch.device, max_positions: int):
        spec.validate()
        self.spec = spec
        self.act_dtype = act_dtype
        self.device = device
        self.max_positions = max_positions
        ctx = BuildContext(device=device, act_dtype=act_dtype, weights=dict(weights),
                           max_positions=max_positions)
        self.embedding = create("embedding", spec.embedding, spec.embedding_prefix, ctx)
        self.layers: List[Block] = [create("block", l.block, l.prefix, ctx) for l in spec.layers]
        self.final_norm = create("norm", spec.final_norm, spec.final_norm_prefix, ctx)
        self.head = create("head", spec.head, spec.head_prefix, ctx)
        self.runs = spec.runs()
        self.graph_safe = all(getattr(p, "graph_safe", False)
                              for p in (self.embedding, *self.layers, self.final_norm, self.head))
        self._plan_cache()
        if device.type == "cuda":
            # the library's products are tried out over the weights of one shape in turn
            from .. import ops
            ops.note_weights(self._tensors())
        # The per-step planners of the mixers, one per distinct key.
        self.step_planners: List[Any] = []
        seen = set()
        for layer in self.layers:
            planner = layer.mixer.step_planner()
            if planner is not None and planner.key() not in seen:
                seen.add(planner.key())
                self.step_planners.append(planner)

    def _tensors(self):
        """Every tensor that a part of the model holds as an attribute (parts within parts
        included)."""
        from ..parts.base import Part
        todo, seen = [self.embedding, *self.layers, self.final_norm, self.head], set()
        while todo:
            part = todo.pop()
            if id(part) in seen:
                continue
            seen.add(id(part))
            for value in vars(part).values():
                if isinstance(value, torch.Tensor):
                    yield value
                elif isinstance(value, Part):
                    todo.append(value)

    # ---------------------------------------------------------------- cache plan
    def _plan_cache(self) -> None:
        self.cache_groups: List[CacheGroupLayout] = []
        self.bindings: List[RunBinding] = []
        by_key: Dict[Any, int] = {}
        state_total = 0
        for i, run in enumerate(self.runs):
            mixer = self.layers[run.layer].mixer
            b = RunBinding()
            req = mixer.cache_request()
            if req is not None:
                if run.cache_of is None:
                    g = by_key.setdefault(req.group_key(), len(self.cache_groups))
                    if g == len(self.cache_groups):
                        self.cache_groups.append(CacheGroupLayout(req))
                    b.group, b.slot = g, len(self.cache_groups[g].writer_runs)
                    self.cache_groups[g].writer_runs.append(i)
                else:
                    src = self.bindings[run.cache_of]
                    theirs = self.layers[self.runs[run.cache_of].layer].mixer.cache_request()
                    if theirs is None or theirs.group_key() != req.group_key():
                        raise ValueError(f"run {i} cannot read the cache of run {run.cache_of}: "
                                         "their cache requests differ")
                    b.group, b.slot, b.writes = src.group, src.slot, False
            nbytes = int(mixer.state_bytes())
            if nbytes:
                b.state_offset, b.state_bytes = state_total, nbytes
                state_total += -(-nbytes // 16) * 16
            self.bindings.append(b)
        self.state_bytes = state_total

    # ------------------------------------------------------------------- forward
    def forward(self, step: Any, pools: Any) -> torch.Tensor:
        """Logits float32 ``(R, V)`` at ``step.logit_rows``; K, V and state of the step's
        tokens are left in ``pools``."""
        stream = ResidualStream(self.embedding.forward(step.ids), self.act_dtype)
        for i, run in enumerate(self.runs):
            self.layers[run.layer].forward(stream, step, pools.binding(self.bindings[i]))
        if step.num_logit_rows == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=self.device)
        return self.head.forward(normed(self.final_norm, stream, self.head, step.logit_rows))
