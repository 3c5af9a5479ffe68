"""Decode steps as HIP graphs.

A step in which every request brings one token launches well over a hundred small kernels;
at batch 1 their launch cost exceeds their run time.  Such steps are therefore captured once
per batch-size bucket into a HIP graph and replayed: the step's metadata lives in one static
int32 buffer (filled on the host by the native page manager, one copy to the device), the
kernels read it through fixed views, and the logits land in a static tensor.

Unused rows of a bucket are padding requests of context 1 that read and write a scratch page
beyond the manager's pages, so they touch nothing a live request owns.  Nothing in the graph
depends on the host: partition counts of the decode attention are fixed per bucket and each
sequence cuts its own context into that many partitions.  Graphs hold no memset nodes (the
kernels clear nothing) and are checked against the eager step in the tests, replay after
replay with eager work in between."""
from __future__ import annotations

import contextlib
import ctypes
import gc
import weakref
from typing import Optional, Sequence

import numpy as np
import torch

from .batch import GroupStep, StepContext


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


class DecodeGraph:
    """The captured decode step of one batch-size bucket."""

    def __init__(self, runner, bucket: int):
        self.runner = weakref.proxy(runner)     # the runner owns its graphs: no cycle
        self.bucket = B = bucket
        model, cache = runner.model, runner.cache
        dev = runner.device
        ps = cache.page_size
        self.width = W = max(8, -(-(-(-model.max_positions // ps)) // 8) * 8)
        ng = cache.num_groups
        # ---- static layout ---------------------------------------------------------------
        names = ["ids", "positions", "seq_of_token", "cu", "start_pos", "ctx_lens", "logit_rows",
                 "state_slots"]
        sizes = {n: B for n in names}
        sizes["cu"] = B + 1
        for g in range(ng):
            sizes[f"slots{g}"] = B
            sizes[f"tables{g}"] = B * W
        self.offsets, total = {}, 0
        for name, n in sizes.items():
            self.offsets[name] = (total, n)
            total += -(-n // 4) * 4
        self.host = torch.zeros(total, dtype=torch.int32).pin_memory()
        self.np = self.host.numpy()
        self.dev = torch.zeros(total, dtype=torch.int32, device=dev)
        self.seq_ids = np.zeros(B, dtype=np.int64)

        def hview(name):
            o, n = self.offsets[name]
            return self.np[o:o + n]

        def dview(name):
            o, n = self.offsets[name]
            return self.dev[o:o + n]

        self.h = {name: hview(name) for name in sizes}
        self.h["seq_of_token"][:] = np.arange(B)
        self.h["cu"][:] = np.arange(B + 1)
        self.h["logit_rows"][:] = np.arange(B)
        base = self.host.data_ptr()
        ptr = lambda name: base + 4 * self.offsets[name][0]
        self.ptr_positions, self.ptr_slots = ptr("positions"), ptr("state_slots")
        self.ptr_tables = (ctypes.c_void_p * ng)(*[ptr(f"tables{g}") for g in range(ng)])
        self.ptr_wslots = (ctypes.c_void_p * ng)(*[ptr(f"slots{g}") for g in range(ng)])
        self.scratch_page = runner.pools.scratch_page
        groups = [GroupStep(page_size=ps, window=cache.groups[g].window,
                            block_tables=dview(f"tables{g}").reshape(B, W),
                            slots=dview(f"slots{g}")) for g in range(ng)]
        self.step = StepContext(
            num_tokens=B, num_seqs=B, ids=dview("ids"), positions=dview("positions"),
            seq_of_token=dview("seq_of_token"), cu_seqlens=dview("cu"),
            start_pos=dview("start_pos"), ctx_lens=dview("ctx_lens"),
            logit_rows=dview("logit_rows"), num_logit_rows=B, state_slots=dview("state_slots"),
            tile_map=dview("ids")[:0], num_tiles=0, groups=groups,
            max_context=model.max_positions, max_new=1, all_decode=True, decode_splits=None)
        self.graph: Optional[torch.cuda.CUDAGraph] = None
        self.logits: Optional[torch.Tensor] = None
        self._copied: Optional[torch.cuda.Event] = None

    # ------------------------------------------------------------------------------------
    def _fill(self, seq_ids: Sequence[int], tokens: Sequence[int]) -> None:
        S, B, W = len(seq_ids), self.bucket, self.width
        h = self.h
        self.seq_ids[:S] = seq_ids
        h["ids"][:S] = tokens
        self.runner.cache.decode_batch(self.seq_ids.ctypes.data, S, W, self.ptr_positions,
                                       self.ptr_slots, self.ptr_tables, self.ptr_wslots)
        if S < B:                        # padding requests: context 1 on the scratch page
            h["ids"][S:] = 0
            h["positions"][S:] = 0
            h["state_slots"][S:] = 0
            for g in range(len(self.ptr_tables)):
                h[f"tables{g}"].reshape(B, W)[S:, 0] = self.scratch_page
                h[f"slots{g}"][S:] = self.scratch_page * self.runner.cache.page_size
        h["start_pos"][:] = h["positions"]
        h["ctx_lens"][:] = h["positions"] + 1

    def run(self, seq_ids: Sequence[int], tokens: Sequence[int]) -> torch.Tensor:
        """Logits ``(len(seq_ids), vocab)`` of one decode token per request.  The result
        views a static tensor: it is overwritten by the next call."""
        if self._copied is not None:
            self._copied.synchronize()       # the host buffer is free to be written again
        self._fill(seq_ids, tokens)
        self.dev.copy_(self.host, non_blocking=True)
        if self._copied is None:
            self._copied = torch.cuda.Event()
        self._copied.record()
        if self.graph is None:
            self._capture()
        else:
            self.graph.replay()
        return self.logits[:len(seq_ids)]

    def _capture(self) -> None:
        runner = self.runner
        # One eager run first: it settles lazy initialisation (library loading, workspace
        # allocations) that must not happen under capture.  The step is idempotent: it writes
        # the same keys and values to the same slots.
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            runner.model.forward(self.step, runner.pools)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with no_collection(), torch.cuda.graph(graph):
            self.logits = runner.model.forward(self.step, runner.pools)
        self.graph = graph
        graph.replay()
