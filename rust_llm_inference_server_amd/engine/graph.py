"""Decode steps as HIP graphs.

A step in which every request brings one token launches well over a hundred small kernels;
at batch 1 their launch cost exceeds their run time.  Such steps are therefore captured once
per batch-size bucket into a HIP graph and replayed: the step's metadata lives in one static
int32 buffer (filled on the host by the native page manager; the graph begins with its copy to
the device), the kernels read it through fixed views, and the logits land in a static tensor.
A second kind of graph goes on where the first ends: the sampling kernel on those logits (keys
and temperatures travel with the metadata), which leaves the tokens where the next step's ids
are.  Its launch copies the metadata to the device in front of it and the tokens to pinned
host memory behind it, so that between two decode steps the host waits for one event; and a
step of the same requests can be launched while the one before it still runs, on the tokens
as they lie on the device: it brings everything but the ids from the host.  The host side of
the metadata exists twice for that, the two taking turns.

Unused rows of a bucket are padding requests of context 1 that read and write a scratch page
beyond the manager's pages and a scratch state slot beyond its slots, so they touch nothing a
live request owns.  Nothing in the graph depends on the host: what a mixer's planner sizes by
the longest context is fixed per context bucket, and how a sequence's own work is cut follows
from its own lengths on the device, so a replay computes bit for bit what the eager step does
(to rounding where the library's products compute, bfloat16 at 33 to 64 rows: a captured step
runs its bucket's rows, for which the library may take another algorithm than for the step's
own count).
Graphs hold no memset nodes (the kernels clear nothing) and are checked against the eager step
in the tests, replay after replay with eager work in between."""
from __future__ import annotations

import collections
import contextlib
import ctypes
import gc
import warnings
import weakref
from typing import Dict, Optional, Sequence, Tuple

import numpy as np
import torch

from ..stepplan import StepPlan
from .batch import GroupStep, MetadataBuffer, StepContext, common_layout


def bucket_for(n: int, limit: int) -> int:
    """The smallest power of two that holds ``n`` requests, capped at ``limit``."""
    b = 1
    while b < n:
        b *= 2
    return min(b, max(limit, n))


@contextlib.contextmanager
def no_collection():
    """Keeps Python's cyclic collector from running inside the block.  Under stream capture it
    must not: what it finds (an earlier engine's graphs, pinned buffers, events: they sit in
    reference cycles) is destroyed through HIP calls that a capturing stream refuses, and an
    error inside a destructor ends the process.  Garbage is collected before the block and
    waits until after it."""
    gc.collect()
    enabled = gc.isenabled()
    gc.disable()
    try:
        yield
    finally:
        if enabled:
            gc.enable()


def context_bucket(context: int, limit: int) -> int:
    """The smallest of 1024, 2048, 4096, ... that holds ``context`` positions, capped at
    ``limit``: captured steps are kept per bucket, so that what a planner sizes by the longest
    context (the depth of a grid) need not be sized for the longest context there could be."""
    b = 1024
    while b < context:
        b *= 2
    return min(b, limit)


LOGITS, SAMPLED = "logits", "sampled"


class _HostSide:
    """One host copy of a bucket's metadata, pinned, with its views and the addresses that the
    native page manager fills; where a sampling step leaves its tokens for the host, and the
    event after the last step that was prepared here."""

    def __init__(self, meta: MetadataBuffer, B: int, num_groups: int):
        self.host = torch.zeros(meta.size, dtype=torch.int32).pin_memory()
        self.np = self.host.numpy()
        self.h = {name: meta.view(self.np, name) for name in meta.offsets}
        self.h["seq_of_token"][:] = np.arange(B)
        self.h["cu"][:] = np.arange(B + 1)
        self.h["logit_rows"][:] = np.arange(B)
        base = self.host.data_ptr()
        ptr = lambda name: base + 4 * meta.offsets[name][0]
        self.ptr_positions, self.ptr_slots = ptr("positions"), ptr("state_slots")
        self.ptr_tables = (ctypes.c_void_p * num_groups)(
            *[ptr(f"tables{g}") for g in range(num_groups)])
        self.ptr_wslots = (ctypes.c_void_p * num_groups)(
            *[ptr(f"slots{g}") for g in range(num_groups)])
        self.tokens_host = torch.zeros(B, dtype=torch.int32).pin_memory()
        self.done: Optional[torch.cuda.Event] = None


class DecodeGraph:
    """The captured decode steps of one batch-size bucket: one static metadata buffer, and one
    HIP graph per context bucket."""

    def __init__(self, runner, bucket: int):
        self.runner = weakref.proxy(runner)     # the runner owns its graphs: no cycle
        self.bucket = B = bucket
        model, cache = runner.model, runner.cache
        dev = runner.device
        ps = cache.page_size
        self.width = W = max(8, -(-(-(-model.max_positions // ps)) // 8) * 8)
        ng = cache.num_groups
        # ---- static layout: the step builder's arrays for B single tokens, all wanted, with
        # block tables at their widest --------------------------------------------------------
        self.meta = meta = MetadataBuffer()
        for name, count in common_layout(B, B, B, [W] * ng):
            meta.reserve(name, count)
        # what the sampling kernel needs per row (bit patterns; 1/T = 0: greedy), for the steps
        # that sample inside the graph
        meta.reserve("sample_keys", B)
        meta.reserve("sample_inv_t", B)
        # Two host sides take turns: a step is prepared in one while the step before it, which
        # was prepared in the other, may not have read its metadata yet.
        self.sides = [_HostSide(meta, B, ng), _HostSide(meta, B, ng)]
        self.h = self.sides[0].h
        self.dev = torch.zeros(meta.size, dtype=torch.int32, device=dev)
        self.seq_ids = np.zeros(B, dtype=np.int64)
        self.scratch_pages = list(runner.pools.scratch_pages) or [0] * ng
        self.scratch_state_slot = runner.pools.scratch_state_slot
        dview = lambda name: meta.view(self.dev, name)
        self.groups = [GroupStep(page_size=ps, window=cache.groups[g].window,
                                 block_tables=dview(f"tables{g}").reshape(B, W),
                                 slots=dview(f"slots{g}")) for g in range(ng)]
        self.views = {name: dview(name) for name in meta.offsets}
        # (context bucket, LOGITS or SAMPLED) -> (graph, its static logits or sampled tokens)
        self.graphs: Dict[Tuple[int, str], Tuple[torch.cuda.CUDAGraph, torch.Tensor]] = {}
        # what of the metadata a chained step brings from the host: everything behind the ids
        self.behind_ids = meta.offsets["positions"][0]
        # the requests of the step prepared last, and those whose sampled tokens are where the
        # ids are (None: something else is there)
        self._prepared: Optional[Tuple[int, ...]] = None
        self._sampled_for: Optional[Tuple[int, ...]] = None

    def step_for(self, context_limit: int) -> StepContext:
        """The step as the kernels of a captured run see it: static views, and each planner's
        plan for any contexts up to ``context_limit``."""
        B, v = self.bucket, self.views
        runner = self.runner
        plans = {}
        for planner in runner.model.step_planners:
            host = planner.plan_captured(B, context_limit, runner.cache.page_size)
            if host.arrays:
                raise ValueError(f"the plan of a captured step may hold values only, "
                                 f"{type(planner).__name__} returned arrays")
            plans[planner.key()] = StepPlan({}, host.values)
        return StepContext(
            num_tokens=B, num_seqs=B, ids=v["ids"], positions=v["positions"],
            seq_of_token=v["seq_of_token"], cu_seqlens=v["cu"], start_pos=v["start_pos"],
            ctx_lens=v["ctx_lens"], logit_rows=v["logit_rows"], num_logit_rows=B,
            state_slots=v["state_slots"], groups=self.groups, max_context=context_limit,
            max_new=1, all_decode=True, num_single=B, plans=plans)

    # ------------------------------------------------------------------------------------
    def _pad_from(self, S: int, h: Optional[dict] = None) -> None:
        """Rows S.. of the bucket: padding requests of context 1 on the scratch page, with the
        scratch state slot (in the host views ``h``, the live ones by default)."""
        B, W = self.bucket, self.width
        h = self.h if h is None else h
        if S < B:
            h["ids"][S:] = 0
            h["positions"][S:] = 0
            h["state_slots"][S:] = self.scratch_state_slot
            for g in range(len(self.groups)):
                h[f"tables{g}"].reshape(B, W)[S:, 0] = self.scratch_pages[g]
                h[f"slots{g}"][S:] = self.scratch_pages[g] * self.runner.cache.page_size
        h["start_pos"][:] = h["positions"]
        h["ctx_lens"][:] = h["positions"] + 1

    def prepare(self, seq_ids: Sequence[int], tokens: Optional[Sequence[int]],
                modes: Optional[Sequence[Tuple[int, float]]] = None, side: int = 0) -> np.ndarray:
        """Fill host side ``side`` of the metadata for one token per request (``modes``: each
        row's (key, 1/T) for a step that samples inside the graph; ``tokens`` None: a chained
        step, whose ids are on the device already); returns the new tokens' positions.  Nothing
        is launched yet."""
        hs = self.sides[side]
        if hs.done is not None:
            hs.done.synchronize()            # the last step prepared here has read this side
        h = hs.h
        S = len(seq_ids)
        self.seq_ids[:S] = seq_ids
        self._prepared = tuple(seq_ids)
        if tokens is not None:
            h["ids"][:S] = tokens
        if modes is not None:
            h["sample_keys"][:S] = np.asarray([k for k, _ in modes], dtype=np.uint32).view(np.int32)
            h["sample_inv_t"][:S] = np.asarray([t for _, t in modes],
                                               dtype=np.float32).view(np.int32)
            h["sample_keys"][S:] = 0
            h["sample_inv_t"][S:] = 0
        self.runner.cache.decode_batch(self.seq_ids.ctypes.data, S, self.width,
                                       hs.ptr_positions, hs.ptr_slots, hs.ptr_tables,
                                       hs.ptr_wslots)
        self._pad_from(S, h)
        return h["positions"][:S]

    def launch(self, num_seqs: int, context_limit: int) -> torch.Tensor:
        """Run the step prepared in side 0.  Logits ``(num_seqs, vocab)``: a view of a static
        tensor that the next call for the same context bucket overwrites."""
        graph, result = self._graph(context_limit, LOGITS)
        self._sampled_for = None
        graph.replay()          # begins with the copy of side 0 of the metadata to the device
        hs = self.sides[0]
        if hs.done is None:
            hs.done = torch.cuda.Event()
        hs.done.record()
        return result[:num_seqs]

    def launch_sampled(self, num_seqs: int, context_limit: int, side: int = 0,
                       chained: bool = False):
        """Run the step prepared in ``side`` with the sampling inside; returns a function that
        waits for the step and returns the requests' tokens.  ``chained``: the step's ids are
        the tokens that the sampling of the step before it (the same requests in the same
        rows) left on the device; that step may still be running."""
        if chained and self._sampled_for != self._prepared:
            raise ValueError("a chained step follows a sampling step of the same requests in "
                             "the same order")
        graph, _ = self._graph(context_limit, SAMPLED)        # (a capture runs a step of padding)
        self._sampled_for = self._prepared
        hs = self.sides[side]
        lo = self.behind_ids if chained else 0
        self.dev[lo:].copy_(hs.host[lo:], non_blocking=True)
        graph.replay()
        hs.tokens_host.copy_(self.views["ids"], non_blocking=True)
        if hs.done is None:
            hs.done = torch.cuda.Event()
        hs.done.record()
        done, tokens = hs.done, hs.tokens_host

        def wait() -> list:
            done.synchronize()
            return tokens[:num_seqs].tolist()
        return wait

    def _graph(self, context_limit: int, kind: str):
        key = (context_limit, kind)
        if key not in self.graphs:
            self._capture(context_limit, kind)
        return self.graphs[key]

    def _capture(self, context_limit: int, kind: str) -> None:
        """Capture the step.  LOGITS: the copy of side 0 of the host's metadata to the device
        and the model.  SAMPLED: the model and the sampling kernel, which leaves its tokens
        where the next step's ids are; its launch copies the metadata to the device and the
        tokens to the host, from and to whichever side it names.  The warm-up run works on
        metadata that is all padding: what it computes lands on the scratch page and the
        scratch state slot, so that no request's cache or state moves before the first replay
        (the capture itself runs nothing); the ids on the device, which a chained step is
        about to read, are put back after it."""
        from .. import ops
        runner = self.runner
        host = self.sides[0].host
        padding = host.clone()
        flat = padding.numpy()
        self._pad_from(0, {name: self.meta.view(flat, name) for name in self.meta.offsets})
        ids = self.views["ids"]
        kept = ids.clone()
        self.dev.copy_(padding)
        step = self.step_for(context_limit)
        keys = self.views["sample_keys"]
        inv_t = self.views["sample_inv_t"].view(torch.float32)

        def run():
            logits = runner.model.forward(step, runner.pools)
            return logits if kind == LOGITS else ops.sample_rows(logits, keys, inv_t, out=ids)

        # One eager run first: it settles lazy initialisation (library loading, workspace
        # allocations) that must not happen under capture.  The graph will be replayed on the
        # stream that is current now, so its library products take that stream's workspace.
        from ..ops import lib
        with lib.workspace_owner(torch.cuda.current_stream()):
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                run()
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with no_collection(), torch.cuda.graph(graph):
                if kind == LOGITS:
                    self.dev.copy_(host, non_blocking=True)
                result = run()
        ids.copy_(kept)
        self.graphs[(context_limit, kind)] = (graph, result)


class RepeatedSteps:
    """Steps that are not pure decode steps, captured when their shape comes back.

    A step's launches (which kernels, their grids, what every planner made of the step) follow
    from its host side: every sequence's cached and new positions, its state slot, and how many
    rows are wanted.  Two steps that agree in all of that differ in data alone (token ids, page
    tables, write slots, wanted rows, work lists of the same sizes), and all of that lies in
    the one metadata buffer.  So when such a shape has come back often enough the step is
    captured over a buffer that stays where it is, and from then on it is replayed: the new
    step's metadata is copied into that buffer on the device, and one graph launch takes the
    place of some 150 kernel launches.  Shapes that come back are the windows of a perplexity
    run, whole prompts of one length, and the portions of long prompts under a token budget
    on an otherwise idle engine; a step that mixes decoding requests with a portion hardly
    ever meets its shape again and stays eager.  What a replay saves is the host's time for
    the launches where that exceeds the kernels' time (1B shape, 16 layers: a step of 128
    tokens 2.6 -> 1.7 ms, of 512 tokens 2.6 -> 2.4, of 2,048 tokens 5.6 -> 5.4), and a
    capture costs 30 to 60 ms, which is why a shape is not captured the first time it comes
    back.  A capture runs nothing, so the step it captures is run once, by its first replay.
    The least recently used of more than ``limit`` captured shapes is dropped with its memory;
    steps of more than ``max_tokens`` tokens stay eager."""

    CAPTURE_AT = 4          # a shape is captured when it is seen for the fourth time

    def __init__(self, runner, limit: int = 4, max_tokens: int = 8192):
        self.runner = weakref.proxy(runner)
        self.limit, self.max_tokens = limit, max_tokens
        self.seen: Dict[tuple, int] = {}
        # shape -> (graph, its metadata buffer, its static logits), least recently used first
        self.graphs: "collections.OrderedDict[tuple, tuple]" = collections.OrderedDict()
        self.replays = 0

    @staticmethod
    def shape_of(step: StepContext) -> tuple:
        return (tuple(step.host_start_pos), tuple(step.host_new), tuple(step.host_state_slots),
                step.num_logit_rows, step.buffer.numel())

    def run(self, step: StepContext) -> Optional[torch.Tensor]:
        """The step's logits from a captured run (a static tensor that the next replay of the
        shape overwrites), or None: the caller then runs the step eagerly."""
        if step.buffer is None or step.over is None or step.num_tokens > self.max_tokens:
            return None
        shape = self.shape_of(step)
        held = self.graphs.get(shape)
        if held is None:
            count = self.seen.get(shape, 0) + 1
            if count < self.CAPTURE_AT:
                if len(self.seen) >= 4096:
                    self.seen.clear()
                self.seen[shape] = count
                return None
            self.seen.pop(shape, None)
            try:
                held = self._capture(shape, step)
            except RuntimeError as e:
                # (a part that waits for the device in such a step, say: nothing has run, the
                # step is the caller's to run eagerly, and the shape is left alone from now on)
                warnings.warn(f"a step of {step.num_tokens} tokens could not be captured and "
                              f"stays eager: {e}")
                self.seen[shape] = -(1 << 60)
                return None
        else:
            self.graphs.move_to_end(shape)
        graph, buffer, logits = held
        buffer.copy_(step.buffer, non_blocking=True)
        graph.replay()
        self.replays += 1
        return logits

    def _capture(self, shape: tuple, step: StepContext) -> tuple:
        runner = self.runner
        while len(self.graphs) >= self.limit:
            self.graphs.popitem(last=False)
        buffer = torch.empty_like(step.buffer)
        buffer.copy_(step.buffer)
        static = step.over(buffer)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        from ..ops import lib
        with lib.workspace_owner(torch.cuda.current_stream()), no_collection(), \
                torch.cuda.graph(graph):
            logits = runner.model.forward(static, runner.pools)
        held = self.graphs[shape] = (graph, buffer, logits)
        return held
