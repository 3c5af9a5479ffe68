"""Python face of the native scheduler (``csrc/runtime/scheduler.cpp``), which decides what
each step computes: continuous batching, chunked prefill under a token budget, preemption by
recompute when pages run out (crates/engine/src/scheduler.rs of the reference)."""
from __future__ import annotations

import ctypes
from ctypes import c_int, c_longlong
from dataclasses import dataclass, field
from typing import List, Sequence, Tuple

import numpy as np

from ..cache.manager import CacheManager, PageCopy, rt_error, runtime


@dataclass
class Schedule:
    """One step's work: portions ``(id, start, end)`` in batch order, page copies to perform
    before the forward pass, and the requests preempted while making room."""
    seqs: List[Tuple[int, int, int]] = field(default_factory=list)
    copies: List[PageCopy] = field(default_factory=list)
    preempted: List[int] = field(default_factory=list)

    def num_tokens(self) -> int:
        return sum(e - s for _, s, e in self.seqs)


class Scheduler:
    def __init__(self, cache: CacheManager, max_num_seqs: int, max_batched_tokens: int,
                 watermark_pages: int = 0, policy: str = "continuous"):
        if policy not in ("continuous", "static"):
            raise ValueError(f"unknown scheduling policy {policy!r}")
        self.cache = cache
        self.max_num_seqs = max_num_seqs
        self.max_batched_tokens = max_batched_tokens
        rt = runtime()
        self._h = rt.rlis_sched_create(cache._h, max_num_seqs, max_batched_tokens,
                                       watermark_pages, 1 if policy == "static" else 0)
        if not self._h:
            raise ValueError(rt_error())
        cap = max_num_seqs + 1
        self._seqs = (c_longlong * (3 * cap))()
        self._pre = (c_longlong * (cap + 1))()
        self._copies = (c_int * (3 * 4 * cap * max(1, cache.num_groups)))()
        self._n = (c_int(0), c_int(0), c_int(0))

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            try:
                runtime().rlis_sched_destroy(h)
            except Exception:
                pass

    def add(self, seq_id: int, prompt_len: int) -> None:
        if runtime().rlis_sched_add(self._h, seq_id, prompt_len) != 0:
            raise ValueError(rt_error())

    def schedule(self) -> Schedule:
        n_s, n_p, n_c = self._n
        rc = runtime().rlis_sched_schedule(
            self._h, self._seqs, len(self._seqs) // 3, n_s, self._pre, len(self._pre), n_p,
            self._copies, len(self._copies) // 3, n_c)
        if rc != 0:
            raise RuntimeError(rt_error())
        c = self._copies
        # (read through a numpy view: element by element a ctypes array costs more than the
        # scheduling itself at 64 requests)
        triples = np.frombuffer(self._seqs, dtype=np.int64, count=3 * n_s.value)
        return Schedule(
            seqs=[tuple(t) for t in triples.reshape(-1, 3).tolist()],
            copies=[PageCopy(c[3 * i], c[3 * i + 1], c[3 * i + 2]) for i in range(n_c.value)],
            preempted=list(self._pre[:n_p.value]),
        )

    def advance(self, seq_id: int, end: int) -> None:
        if runtime().rlis_sched_advance(self._h, seq_id, end) != 0:
            raise ValueError(rt_error())

    def append_token(self, seq_id: int) -> None:
        runtime().rlis_sched_append_token(self._h, seq_id)

    def append_tokens(self, seq_ids: Sequence[int]) -> None:
        """One more token each for ``seq_ids``, in one call."""
        n = len(seq_ids)
        if n and runtime().rlis_sched_append_tokens(self._h, (c_longlong * n)(*seq_ids), n) != 0:
            raise ValueError(rt_error())

    def is_caught_up(self, seq_id: int) -> bool:
        return bool(runtime().rlis_sched_is_caught_up(self._h, seq_id))

    def remove(self, seq_id: int) -> None:
        if runtime().rlis_sched_remove(self._h, seq_id) != 0:
            raise RuntimeError(rt_error())

    def has_work(self) -> bool:
        return bool(runtime().rlis_sched_has_work(self._h))

    @property
    def num_running(self) -> int:
        return runtime().rlis_sched_num_running(self._h)

    @property
    def num_waiting(self) -> int:
        return runtime().rlis_sched_num_waiting(self._h)

    @property
    def num_preemptions(self) -> int:
        return runtime().rlis_sched_num_preemptions(self._h)

    @property
    def max_seq_tokens(self) -> int:
        return runtime().rlis_sched_max_seq_tokens(self._h)

    def num_tokens(self, seq_id: int) -> int:
        return runtime().rlis_sched_num_tokens(self._h, seq_id)

    def num_computed(self, seq_id: int) -> int:
        return runtime().rlis_sched_num_computed(self._h, seq_id)

    def check(self) -> None:
        buf = ctypes.create_string_buffer(512)
        if runtime().rlis_sched_check(self._h, buf, 512) != 0:
            raise AssertionError(buf.value.decode())
