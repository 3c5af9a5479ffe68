"""Host-side planning of the attention kernels' work for one step.

The step builder knows nothing of these kernels: a mixer that uses them names an
``AttentionPlanner`` as its ``step_planner()``, and the builder carries what ``plan`` returns
(int32 arrays and a few launch sizes) to the device with the rest of the step's metadata.

Every choice here follows from a sequence's *own* lengths and from the constants below, never
from how many other sequences or tiles the batch holds, so that the order of a row's sums (and
with it the rounding of its result) is the same alone and among neighbours:

* a sequence that brings one token is cut into partitions of ``DECODE_PART_KEYS`` keys (a
  multiple of that beyond ``DECODE_MAX_PARTS`` partitions) by the decode kernels themselves;
  the plan only says how deep the grid must be for the longest of them;
* a sequence that brings a portion of a prompt takes tiles of 128 queries when its own context
  is long or its own tiles are plenty, else tiles of 64;
* the keys of its tiles are cut into runs (one workgroup each, merged afterwards) when its own
  tiles are too few to fill the chip and its context is long.

The reference cuts decode contexts by a rule of the same kind
(crates/model/src/paged_attention.rs:21-36), though from the batch's longest context."""
from __future__ import annotations

from typing import Any, List, Tuple

import numpy as np

from ..stepplan import HostPlan, StepLengths, StepPlanner

# Keys per partition of a decode context and the most partitions a context is cut into.
DECODE_PART_KEYS = 1024
DECODE_MAX_PARTS = 16
PREFILL_TILE = 64     # new tokens per workgroup of the matrix-core prefill attention
WIDE_TILE = 128       # ... of its form with two query blocks per wave
# A sequence takes tiles of 128 queries when they make this many workgroups (tiles x heads; 5/3
# as many up to head size 64), or when its context is long (4096 positions after the step, or
# 2048 cached ones); 1 << 30: never.
PREFILL_WIDE_MIN_GROUPS = 768
# A sequence whose tiles make at most this many workgroups has the keys of its tiles cut into
# runs: as many as keep the compute units' resident workgroups busy, with at least
# PREFILL_SPLIT_MIN_KEYS keys a run and at most PREFILL_MAX_RUNS runs (0 units: never).
PREFILL_SPLIT_UNITS = 256
PREFILL_SPLIT_MIN_KEYS = 1024
PREFILL_MAX_RUNS = 16


def decode_parts(context: int, window: int = 0) -> int:
    """Live partitions of a decode context of ``context`` positions (what the kernels'
    ``decode_part_len`` gives); with a window only its keys count (rounded as the matrix-core
    kernel rounds their start, down to a multiple of 32)."""
    lo = max(0, context - window) if window else 0
    n = context - (lo & ~31)
    span = DECODE_PART_KEYS * DECODE_MAX_PARTS
    part = DECODE_PART_KEYS * max(1, -(-n // span))
    return max(1, -(-n // part))


def decode_depth(max_context: int) -> int:
    """Grid depth (and stride of the partial results) that covers every context up to
    ``max_context``."""
    return max(1, min(DECODE_MAX_PARTS, -(-max_context // DECODE_PART_KEYS)))


def decode_walk_room(group: int, head_dim: int) -> int:
    """Partitions whose parked sums (eight waves, ``group`` heads, ``head_dim`` + 2 floats) a
    decode workgroup has LDS for: 64 KB up to head size 64, where two workgroups share a compute
    unit's 160 KB, 159 KB beyond, where a compute unit holds one."""
    lds = 64 * 1024 if head_dim <= 64 else 159 * 1024
    return lds // (8 * group * (head_dim + 2) * 4)


def decode_shares(num_seqs: int, num_kv_heads: int, depth: int, group: int, head_dim: int,
                  compute_units: int) -> Tuple[int, int]:
    """(groups, cap) for the matrix-core decode kernel under a grid ``depth`` partitions deep:
    a sequence's partitions are dealt out evenly to ``groups`` workgroups, none of which takes
    more than ``cap`` (a sequence with more partitions than that gets more workgroups); cap 1:
    a workgroup per partition.  This is the one choice here that looks at the batch, and it
    may: the partitions and the order of their sums stay what a sequence's own length makes
    them, only the workgroups that share them change, and the kernel gives the same floats
    however they are dealt out.  Sequences times KV heads that fill the compute units by
    themselves take one workgroup each; fewer take as many each as bring them to about what the
    compute units hold at once (two workgroups each up to head size 64, one beyond).  The
    eight waves' sums of every partition in a share must fit the LDS (``decode_walk_room``),
    and the kernel takes shares of whole pairs of chunks only (partitions of a multiple of 512
    keys)."""
    if depth <= 1 or DECODE_PART_KEYS % 512 != 0:
        return depth, 1
    resident = 2 if head_dim <= 64 else 1
    each = max(1, compute_units * resident // max(1, num_seqs * num_kv_heads))
    groups = min(depth, each)
    cap = min(decode_walk_room(group, head_dim), -(-depth // groups))
    return (groups, cap) if cap > 1 else (depth, 1)


class AttentionPlanner(StepPlanner):
    """Plans for ``ops.paged_attention`` with ``num_heads`` query heads of ``head_dim``.

    ``matrix``: the batch can take the matrix-core kernels (bfloat16, head size in steps of 16
    up to 256); without it only the depth of the decode grid is planned.  ``singles_apart``:
    sequences that bring one token beside portions of prompts take the decode kernel (they
    lead the step); otherwise they get tiles like everyone else."""

    def __init__(self, num_heads: int, num_kv_heads: int, head_dim: int, matrix: bool = True,
                 singles_apart: bool = True):
        self.nh, self.nkv, self.d = int(num_heads), int(num_kv_heads), int(head_dim)
        self.matrix = bool(matrix) and self.d % 16 == 0 and self.d <= 256
        g = self.nh // max(1, self.nkv)
        # what the matrix-core decode kernel takes: at most 16 query heads per KV head, whose
        # merge buffer fits the LDS
        self.singles_apart = (bool(singles_apart) and self.matrix and g <= 16
                              and g * (self.d + 2) * 32 <= 65536)

    def key(self) -> Any:
        return ("attention", self.nh, self.nkv, self.d, self.matrix, self.singles_apart)

    @staticmethod
    def pages_fit(page_size: int) -> bool:
        """Page sizes the matrix-core kernels take: powers of two from 8 on."""
        return page_size >= 8 and page_size & (page_size - 1) == 0

    # ------------------------------------------------------------------ per sequence
    def tile_queries(self, cached: int, new: int) -> int:
        """64 or 128: the tile form of a sequence with ``cached`` positions and ``new`` tokens."""
        if self.d > 128 or PREFILL_WIDE_MIN_GROUPS >= (1 << 30):
            return PREFILL_TILE
        groups = -(-new // WIDE_TILE) * self.nh
        enough = PREFILL_WIDE_MIN_GROUPS if self.d > 64 else PREFILL_WIDE_MIN_GROUPS * 5 // 3
        if groups >= enough or cached + new >= 4096 or cached >= 2048:
            return WIDE_TILE
        return PREFILL_TILE

    def key_runs(self, cached: int, new: int, tile: int) -> int:
        """Runs the keys of this sequence's tiles are cut into (1: none)."""
        groups = -(-new // tile) * self.nh
        if PREFILL_SPLIT_UNITS <= 0 or groups > PREFILL_SPLIT_UNITS:
            return 1
        # resident workgroups per compute unit: 4 up to head size 64, 3 with tiles of 128
        # queries, 2 beyond
        resident = 2 if self.d > 64 else (3 if tile == WIDE_TILE else 4)
        return max(1, min(PREFILL_SPLIT_UNITS * resident // groups,
                          (cached + new) // PREFILL_SPLIT_MIN_KEYS, PREFILL_MAX_RUNS))

    # ----------------------------------------------------------------------- a step
    def plan(self, lengths: StepLengths) -> HostPlan:
        start = np.asarray(lengths.start, dtype=np.int64)
        new = np.asarray(lengths.new, dtype=np.int64)
        S = len(new)
        matrix = self.matrix and self.pages_fit(lengths.page_size)
        all_single = lengths.num_single == S
        singles = lengths.num_single if (self.singles_apart and matrix) or all_single else 0
        runs = np.ones(S, dtype=np.int32)
        units: dict = {PREFILL_TILE: [], WIDE_TILE: []}
        for s in range(singles if matrix else S, S):
            c, n = int(start[s]), int(new[s])
            tile = self.tile_queries(c, n)
            r = self.key_runs(c, n, tile)
            runs[s] = r
            qb = np.arange(0, n, tile, dtype=np.int64)
            keys = c + np.minimum(n, qb + tile)                # keys a tile walks
            u = np.empty((len(qb), r, 5), dtype=np.int64)
            u[:, :, 0] = s
            u[:, :, 1] = qb[:, None]
            u[:, :, 2] = np.arange(r)[None, :]
            u[:, :, 3] = r
            u[:, :, 4] = (keys[:, None] + r - 1) // r          # work of a unit
            units[tile].append(u.reshape(-1, 5))
        arrays, values = {"seq_runs": runs}, {}
        for tile, name in ((PREFILL_TILE, "units64"), (WIDE_TILE, "units128")):
            if units[tile]:
                u = np.concatenate(units[tile])
                u = u[np.argsort(-u[:, 4], kind="stable")]     # longest first
                arrays[name] = u[:, :4].astype(np.int32).reshape(-1)
                values["num_" + name] = len(u)
            else:
                arrays[name] = np.zeros(0, dtype=np.int32)
                values["num_" + name] = 0
        values["max_runs"] = int(runs.max()) if S else 1
        values["tile_row0"] = int(new[:singles].sum())         # rows before the tiles' rows
        values["num_decode"] = singles
        ctx = start + new
        values["decode_depth"] = decode_depth(int(ctx[:singles].max()) if singles else 1)
        return HostPlan(arrays, values)

    def plan_captured(self, num_seqs: int, max_context: int, page_size: int) -> HostPlan:
        return HostPlan({}, {"decode_depth": decode_depth(max_context), "num_decode": num_seqs,
                             "max_runs": 1, "tile_row0": num_seqs, "num_units64": 0,
                             "num_units128": 0})


def plan_for(lens_cached: List[int], lens_new: List[int], planner: AttentionPlanner,
             page_size: int) -> Tuple[HostPlan, StepLengths]:
    """The plan of a batch given as plain lists, single tokens first (for tests and probes)."""
    num_single = 0
    for n in lens_new:
        if n != 1:
            break
        num_single += 1
    lengths = StepLengths(np.asarray(lens_cached, dtype=np.int64),
                          np.asarray(lens_new, dtype=np.int64), num_single, page_size)
    return planner.plan(lengths), lengths
