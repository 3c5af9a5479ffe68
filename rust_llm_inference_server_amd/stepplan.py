"""Per-step plans: what a mixer's kernels need laid out on the host for one step beyond the
metadata every step has (work lists, partition counts), and how the step builder carries it.

A mixer names a ``StepPlanner`` (``Mixer.step_planner()``); the step builder calls its ``plan``
once per step with the step's host-side lengths, sends the int32 arrays it returns to the
device together with the common metadata, and hands the result to the mixer as
``step.plans[planner.key()]``.  The builder never looks inside a plan."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict

import torch


@dataclass
class StepLengths:
    """What the host knows of a step before anything runs, in the step's own order of
    sequences (those that bring a single token come first): positions cached before the step,
    new tokens, and the page size."""

    start: Any                 # (S) int64 numpy array
    new: Any                   # (S) int64 numpy array
    num_single: int
    page_size: int

    @property
    def num_seqs(self) -> int:
        return len(self.new)


@dataclass
class HostPlan:
    """What a ``StepPlanner`` hands back: int32 arrays that go to the device with the step's
    other metadata (one copy), and host values (launch sizes and the like)."""

    arrays: Dict[str, Any] = field(default_factory=dict)      # name -> numpy int32 array
    values: Dict[str, Any] = field(default_factory=dict)


class StepPlan:
    """A ``HostPlan`` whose arrays are on the device: ``plan["name"]`` is a device tensor,
    ``plan.value("name")`` a host value."""

    def __init__(self, arrays: Dict[str, torch.Tensor], values: Dict[str, Any]):
        self.arrays, self.values = arrays, values

    def __getitem__(self, name: str) -> torch.Tensor:
        return self.arrays[name]

    def value(self, name: str, default: Any = None) -> Any:
        return self.values.get(name, default)


class StepPlanner:
    """Host-side planning that a mixer's kernels need per step beyond the common metadata
    (work lists, partition counts).  The step builder calls ``plan`` once per step for every
    distinct ``key`` among the model's mixers and carries the result opaquely; the mixer finds
    it as ``step.plans[key]``.  A plan must follow from each sequence's own lengths and from
    constants, so that a row's arithmetic does not depend on what else is in the batch."""

    def key(self) -> Any:
        raise NotImplementedError

    def plan(self, lengths: StepLengths) -> HostPlan:
        raise NotImplementedError

    def plan_captured(self, num_seqs: int, max_context: int, page_size: int) -> HostPlan:
        """The plan of a captured step of one token per sequence: it may hold values only, and
        must be valid for any contexts up to ``max_context``."""
        raise NotImplementedError
