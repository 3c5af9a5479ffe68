"""The interfaces of the parts a model is put together from, and one registry per kind.

A model is a list of blocks; a block arranges a *mixer* (the part through which a token sees
earlier tokens), a *feed-forward* and *norms*; a mixer may use a *position encoding*.  Each
part is built from a ``PartSpec`` (a kind name plus a dict of parameters that carries every
size and constant), a weight-name prefix and a ``BuildContext``.  No part knows which model
it is in: what it needs arrives as parameters, per-step data arrives in the ``StepContext``.

The reference builds its layers the same way, with constants passed in:
``RmsNorm::new(weight, eps)`` (crates/model/src/layers.rs:112-118), ``Attention::new(q, k, v,
bias, o, cfg)`` (attention.rs:23-41), ``Mlp::new(gate, up, down)`` (layers.rs:165-167),
``Rope::from_inv_freqs`` (rope.rs:61-78).

Adding a part: subclass the base class of its kind, decorate it with ``@register(kind_name)``
and name it in a model's specification.  The registries are open; a test may register a part
of its own without touching this package.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Dict, List, Optional, Tuple, Type

import torch

from ..stepplan import HostPlan, StepLengths, StepPlan, StepPlanner  # noqa: F401 (re-exported)


# --------------------------------------------------------------------------- specs
@dataclass(frozen=True)
class TensorSpec:
    """One checkpoint tensor a part reads: its full name, its shape and how random weights
    for it are drawn (``normal``: N(0, std); ``ones_normal``: 1 + N(0, std))."""

    name: str
    shape: Tuple[int, ...]
    init: str = "normal"
    std: float = 0.02


@dataclass
class PartSpec:
    kind: str
    params: Dict[str, Any] = field(default_factory=dict)


PAGE = -1     # in a PageArray's shape: the axis that is as long as a page has positions


@dataclass(frozen=True)
class PageArray:
    """One array a mixer keeps per page: its name and the shape of one page, in which ``PAGE``
    marks the axis of positions.  Keys of 8 heads of 64 are ``("k", (8, PAGE, 64))``; one latent
    vector of 96 numbers per position is ``("latent", (PAGE, 96))``.  ``dtype`` None: the
    model's activation dtype; a mixer that caches something in a precision of its own (float32
    sums in a bfloat16 model, 8-bit codes) names the torch dtype here, and the pools allocate
    and size that array by it."""

    name: str
    shape: Tuple[int, ...]
    dtype: Optional[torch.dtype] = None

    def __post_init__(self):
        if self.shape.count(PAGE) != 1 or any(n <= 0 for n in self.shape if n != PAGE):
            raise ValueError(f"page array '{self.name}': shape {self.shape} needs positive sizes "
                             "and the position axis exactly once")
        if self.dtype is not None and not isinstance(self.dtype, torch.dtype):
            raise ValueError(f"page array '{self.name}': dtype must be a torch dtype or None, "
                             f"got {self.dtype!r}")

    def element_size(self, act_dtype: torch.dtype) -> int:
        """Bytes of one element, in a model whose activations are ``act_dtype``."""
        return torch.empty((), dtype=self.dtype or act_dtype).element_size()

    def bytes_per_token(self, act_dtype: torch.dtype) -> int:
        return self.elements_per_token() * self.element_size(act_dtype)

    def page_shape(self, page_size: int) -> Tuple[int, ...]:
        return tuple(page_size if n == PAGE else n for n in self.shape)

    def elements_per_token(self) -> int:
        n = 1
        for x in self.shape:
            n *= 1 if x == PAGE else x
        return n


@dataclass(frozen=True)
class CacheRequest:
    """What a mixer keeps in pages for every cached position: a kind of its own, given as the
    arrays of one page (each in the activation dtype unless it names its own), for every earlier position (``window``
    None) or for the last ``window`` positions only.  Mixers with equal requests share a page
    group; the pools are allocated from the request, so a mixer that caches something else than
    keys and values names its own arrays.  ``CacheRequest.kv`` is the kind attention uses."""

    arrays: Tuple[PageArray, ...]
    window: Optional[int] = None

    def __post_init__(self):
        names = [a.name for a in self.arrays]
        if not names or len(set(names)) != len(names):
            raise ValueError(f"a cache request needs arrays with distinct names, got {names}")

    @classmethod
    def kv(cls, num_kv_heads: int, head_dim: int, window: Optional[int] = None) -> "CacheRequest":
        """Keys ``[kv head][position][d]`` and values ``[kv head][d][position]`` (values
        transposed inside a page, so that both attention kernels read each as it lies)."""
        return cls((PageArray("k", (num_kv_heads, PAGE, head_dim)),
                    PageArray("v", (num_kv_heads, head_dim, PAGE))), window)

    def group_key(self) -> Tuple[Any, ...]:
        return (self.arrays, self.window)

    def elements_per_token(self) -> int:
        return sum(a.elements_per_token() for a in self.arrays)

    def bytes_per_token(self, act_dtype: torch.dtype) -> int:
        """Bytes that one cached position takes in one layer slot of the group."""
        return sum(a.bytes_per_token(act_dtype) for a in self.arrays)


@dataclass
class CacheBinding:
    """Where one run of a mixer keeps its memory of the past.

    ``pages`` maps each array name of the mixer's cache request to this run's slice of its
    group's pool, ``(num_pages, *page shape)``; ``group`` indexes ``StepContext.groups`` (block
    tables and slots of that group).  ``writes`` is false when the run reads the cache another
    run has written in the same step.  ``state`` is the run's slice of the fixed-size
    per-request state buffer, ``(num_slots, state_bytes)`` uint8, or None when the mixer asked
    for none.  ``counters`` is a run of int32 zeros on the device that belongs to the runner
    (and so to its stream): a mixer's kernels may count in it within one launch, the
    workgroups of the decode attention do when they merge partitions, if they leave zeros."""

    group: int = -1
    pages: Dict[str, torch.Tensor] = field(default_factory=dict)
    writes: bool = True
    state: Optional[torch.Tensor] = None
    counters: Optional[torch.Tensor] = None

    @property
    def k_pages(self) -> Optional[torch.Tensor]:
        return self.pages.get("k")

    @property
    def v_pages(self) -> Optional[torch.Tensor]:
        return self.pages.get("v")


@dataclass
class BuildContext:
    """What a part may look at while it is built."""

    device: torch.device
    act_dtype: torch.dtype                      # torch.float32 or torch.bfloat16
    weights: Dict[str, torch.Tensor]            # checkpoint name -> device tensor
    max_positions: int                          # longest sequence the engine will run
    shared: Dict[Any, Any] = field(default_factory=dict)   # e.g. position tables by parameters

    def take(self, name: str) -> torch.Tensor:
        try:
            return self.weights[name]
        except KeyError:
            raise KeyError(f"weight '{name}' was not loaded") from None


# ---------------------------------------------------------------------- registries
_REGISTRIES: Dict[str, Dict[str, Type["Part"]]] = {
    "mixer": {}, "feed_forward": {}, "norm": {}, "position": {}, "block": {},
    "embedding": {}, "head": {},
}


def register(category: str, kind: str) -> Callable[[Type["Part"]], Type["Part"]]:
    """Class decorator: make ``kind`` buildable as a part of ``category``."""
    if category not in _REGISTRIES:
        raise KeyError(f"unknown part category '{category}' (known: {sorted(_REGISTRIES)})")

    def deco(cls: Type["Part"]) -> Type["Part"]:
        _REGISTRIES[category][kind] = cls
        cls.category = category
        cls.kind = kind
        return cls

    return deco


def lookup(category: str, kind: str) -> Type["Part"]:
    reg = _REGISTRIES[category]
    if kind not in reg:
        raise KeyError(f"no {category} of kind '{kind}' is registered (known: {sorted(reg)})")
    return reg[kind]


def create(category: str, spec: PartSpec, prefix: str, ctx: BuildContext) -> "Part":
    return lookup(category, spec.kind)(spec.params, prefix, ctx)


def tensor_specs(category: str, spec: PartSpec, prefix: str) -> List[TensorSpec]:
    return lookup(category, spec.kind).tensor_specs(spec.params, prefix)


def join(prefix: str, name: str) -> str:
    return f"{prefix}.{name}" if prefix else name


# ---------------------------------------------------------------------- base classes
class Part:
    category = ""
    kind = ""
    # True when the part's forward launches only device work that reads the step's device
    # tensors (no host decision on device data, no synchronisation), so that a decode step may
    # be captured into a HIP graph and replayed with new metadata.  A model's decode steps are
    # captured only when every part of it says so; a new part starts out on the safe side.
    graph_safe = False

    @classmethod
    def tensor_specs(cls, params: Dict[str, Any], prefix: str) -> List[TensorSpec]:
        """The checkpoint tensors this part reads, by full name."""
        return []

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        self.params = params
        self.prefix = prefix


class Norm(Part):
    """``forward(stream)`` returns the normalised activations ``(T, H)`` in the activation
    dtype; it first adds the stream's pending delta into the 32-bit residual (one fused pass).
    ``forward_rows(stream, rows)`` does the same for the selected rows only and leaves the
    residual untouched."""

    def forward(self, stream: "ResidualStream") -> torch.Tensor:
        raise NotImplementedError

    def forward_rows(self, stream: "ResidualStream", rows: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError

    def fused_linear(self, stream: "ResidualStream", w: torch.Tensor, out_dtype: torch.dtype,
                     gated: bool, rows: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
        """The norm and the projection behind it in one kernel: ``norm(stream) @ w.T`` (gated:
        ``silu(. @ Wg.T) * (. @ Wu.T)`` for ``w = [Wg; Wu]``), with the effects of ``forward``
        (or ``forward_rows``) on the stream.  None when this norm has no such kernel for these
        operands; the caller then applies the norm and the projection one after the other."""
        return None


class NormedInput:
    """A norm that has not been applied yet, handed to a part that sets ``takes_normed_input``
    in place of the normalised activations, so that the part's first projection can take the
    norm into its kernel.  ``tensor()`` applies the norm now; ``linear(w, ...)`` is the
    projection of the normalised activations."""

    __slots__ = ("norm", "stream", "rows")

    def __init__(self, norm: Norm, stream: "ResidualStream", rows: Optional[torch.Tensor] = None):
        self.norm, self.stream, self.rows = norm, stream, rows

    def tensor(self) -> torch.Tensor:
        if self.rows is None:
            return self.norm.forward(self.stream)
        return self.norm.forward_rows(self.stream, self.rows)

    def linear(self, w: torch.Tensor, out_dtype: torch.dtype, gated: bool = False) -> torch.Tensor:
        y = self.norm.fused_linear(self.stream, w, out_dtype, gated, self.rows)
        if y is None:
            from .. import ops
            x = self.tensor()
            y = ops.linear_swiglu(x, w) if gated else ops.linear(x, w, out_dtype)
        return y


def project(x: Any, w: torch.Tensor, out_dtype: torch.dtype, gated: bool = False) -> torch.Tensor:
    """``x @ w.T`` (or the gated form) for activations ``x`` or a ``NormedInput``."""
    if isinstance(x, NormedInput):
        return x.linear(w, out_dtype, gated)
    from .. import ops
    return ops.linear_swiglu(x, w) if gated else ops.linear(x, w, out_dtype)


def normed(norm: Norm, stream: "ResidualStream", consumer: Part,
           rows: Optional[torch.Tensor] = None) -> Any:
    """What ``consumer`` gets from ``norm``: the norm itself, unapplied, when it asks for that."""
    if getattr(consumer, "takes_normed_input", False):
        return NormedInput(norm, stream, rows)
    return norm.forward(stream) if rows is None else norm.forward_rows(stream, rows)


class PositionEncoding(Part):
    """Built once per distinct parameter set and shared by the mixers that name it."""


class Mixer(Part):
    """``forward(x, step, binding)`` maps activations ``(T, H)`` to ``(T, H)``.  The result goes
    to the residual stream, so it may also be a stack ``(S, T, H)`` of float32 partial sums
    (what ``ops.linear(..., partials=True)`` returns), which the stream adds in order, or the
    last projection not run yet (what ``ops.pending_linear`` returns), which the norm behind
    it may run with the add inside; ``as_tensor`` gives the tensor either way.

    ``cache_request()`` says what the mixer keeps in pages (None: nothing);
    ``state_bytes()`` how many bytes of fixed-size state it keeps per request (0: none).  A
    mixer with state must leave, after a step, the state as it is after the last token the
    step brought for that request.  ``step_planner()`` names the host-side planning its kernels
    need per step (None: the common metadata is enough)."""

    # True when forward takes ``x`` as a NormedInput (and projects it with ``project``).
    takes_normed_input = False

    def cache_request(self) -> Optional[CacheRequest]:
        return None

    def step_planner(self) -> Optional[StepPlanner]:
        return None

    def state_bytes(self) -> int:
        return 0

    def forward(self, x: torch.Tensor, step: Any, binding: CacheBinding) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    """``forward(x, step)`` maps activations ``(T, H)`` to ``(T, H)``, row by row (or to a
    stack of float32 partial sums of that, or to a projection that has not run yet, as a mixer
    may)."""

    takes_normed_input = False       # as for a mixer

    def forward(self, x: torch.Tensor, step: Any) -> torch.Tensor:
        raise NotImplementedError


class Block(Part):
    """Arranges a mixer, a feed-forward and their norms around the residual stream."""

    mixer: Mixer

    def forward(self, stream: "ResidualStream", step: Any, binding: CacheBinding) -> None:
        raise NotImplementedError


class Embedding(Part):
    def forward(self, ids: torch.Tensor) -> torch.Tensor:
        """Token ids ``(T)`` int32 -> residual stream ``(T, H)`` float32."""
        raise NotImplementedError


class Head(Part):
    takes_normed_input = False       # as for a mixer

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """Normalised rows ``(R, H)`` -> logits ``(R, V)`` float32."""
        raise NotImplementedError


def as_tensor(delta: Any) -> torch.Tensor:
    """What a mixer or a feed-forward returned, as one ``(T, H)`` tensor: a projection that has
    not run yet runs now, a stack of partial sums is added up."""
    if not isinstance(delta, torch.Tensor):
        delta = delta.run()
    return delta.sum(0) if delta.dim() == 3 else delta


class ResidualStream:
    """The residual sum, kept in 32-bit, plus a delta that has not been added yet.

    A block's output is left *pending* so that the next norm can add it and normalise in one
    pass over the row; the sum itself is always formed and stored in float32.  A block's output
    joins the sum rounded once to the activation dtype: a delta that arrives as a stack of
    float32 partial sums is added up and, in a bfloat16 model, rounded to bfloat16 first
    (``round_parts``), as a delta that arrives whole in bfloat16 was by its kernel, so that the
    rounding does not depend on which kernel a batch's size chose."""

    __slots__ = ("x", "pending", "round_parts")

    def __init__(self, x: torch.Tensor, act_dtype: torch.dtype = torch.float32):
        assert x.dtype == torch.float32
        self.x = x
        # a tensor, or a product that has not run yet (``ops.pending_linear``), which a norm
        # may run with the add and its own multiplies inside
        self.pending: Any = None
        self.round_parts = act_dtype == torch.bfloat16

    def add(self, delta: Any) -> None:
        if self.pending is not None:
            self.flush()
        self.pending = delta

    def delta(self) -> Optional[torch.Tensor]:
        """The pending delta as a tensor (a product that has not run yet runs now)."""
        if self.pending is not None and not isinstance(self.pending, torch.Tensor):
            self.pending = self.pending.run()
        return self.pending

    def flush(self) -> torch.Tensor:
        """Fold a pending delta into the residual and return the residual."""
        if self.pending is not None:
            from .. import ops
            ops.add_residual(self.x, self.delta(), round_parts=self.round_parts)
            self.pending = None
        return self.x
