"""The device side of the cache: one pool of pages per group and one buffer of fixed-size
per-request state.

A group's pool holds, for every layer slot of the group and for every array its cache request
names, ``num_pages`` pages of that array's page shape.  The attention kind keeps keys
``[page][kv head][offset][d]`` and values ``[page][kv head][d][offset]`` (values transposed
inside a page, so that both attention kernels read each as it lies); another mixer names its
own arrays and gets them the same way.  One page id addresses the same page in every layer
slot of its group, as one block id addresses every layer in the reference
(crates/model/src/paged.rs:1-7, 41-60).  Pools are allocated once, zeroed.

One page beyond the manager's is scratch in every group, and one state slot beyond the
manager's: padding rows of a captured decode step read and write them, so they touch nothing a
request owns.

``pool_pages`` is the sizing rule: how many pages each group gets out of one budget of bytes,
from each group's own bytes per page and window."""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import torch

from ..parts.base import CacheBinding


def pool_pages(cache_groups: Sequence, act_dtype: torch.dtype, page_size: int, budget_bytes: int,
               max_num_seqs: int, max_batched_tokens: int, max_seq_len: int) -> List[int]:
    """Pages for every group's pool out of ``budget_bytes``.

    A model whose groups all keep every position gets the reference's rule (crates/engine/src/
    engine.rs:252-262): budget / bytes of one page across all groups, the same count for each.
    A group that keeps a window only never holds more per request than the window plus the
    positions of one step that are reserved before the window has moved on (and one page for
    where in a page the window begins), except at admission, when a request's whole known
    length is reserved in every group: so its pool is capped at what ``max_num_seqs`` requests
    hold that way, but never below one request of ``max_seq_len`` (what admission needs), and
    what the cap leaves of the budget goes to the groups that keep everything."""
    per_page = [max(1, len(g.writer_runs)) * g.request.bytes_per_token(act_dtype) * page_size
                for g in cache_groups]
    if not per_page:
        return []
    even = budget_bytes // sum(per_page)
    pages = [even] * len(per_page)
    for_one = -(-max_seq_len // page_size) + 1
    left = budget_bytes
    full = []
    for i, g in enumerate(cache_groups):
        w = g.request.window
        if w:
            held = -(-(w + max_batched_tokens) // page_size) + 1
            pages[i] = min(even, max(for_one, max_num_seqs * held))
            left -= pages[i] * per_page[i]
        else:
            full.append(i)
    if full and len(full) < len(per_page):
        share = left // sum(per_page[i] for i in full)
        for i in full:
            pages[i] = max(even, share)
    return pages


COUNTERS = 1 << 16


class CachePools:
    def __init__(self, cache_groups: Sequence, num_pages: Sequence[int], page_size: int,
                 dtype: torch.dtype, device: torch.device, num_state_slots: int = 0,
                 state_bytes: int = 0):
        self.page_size = page_size
        self.dtype = dtype
        self.device = device
        # Per group: array name -> (layer slots, pages + 1, *page shape).
        self.arrays: List[Dict[str, torch.Tensor]] = []
        # Per group: the page beyond the manager's, which padding rows read and write.
        self.scratch_pages: List[int] = [int(n) for n in num_pages]
        for layout, pages in zip(cache_groups, num_pages):
            n = max(1, len(layout.writer_runs))
            self.arrays.append({
                a.name: torch.zeros((n, int(pages) + 1) + a.page_shape(page_size),
                                    dtype=a.dtype or dtype, device=device)
                for a in layout.request.arrays})
        # Zeros that the kernels of one launch may count in and leave zero again (CacheBinding).
        self.counters = torch.zeros(COUNTERS, dtype=torch.int32, device=device)
        self.state: Optional[torch.Tensor] = None
        self.scratch_state_slot = num_state_slots
        if state_bytes > 0 and num_state_slots > 0:
            self.state = torch.zeros((num_state_slots + 1, state_bytes), dtype=torch.uint8,
                                     device=device)

    def binding(self, rb) -> CacheBinding:
        b = CacheBinding(group=rb.group, writes=rb.writes, counters=self.counters)
        if rb.group >= 0:
            b.pages = {name: t[rb.slot] for name, t in self.arrays[rb.group].items()}
        if rb.state_bytes and self.state is not None:
            b.state = self.state[:, rb.state_offset:rb.state_offset + rb.state_bytes]
        return b

    def copy_pages(self, group: int, src: Sequence[int], dst: Sequence[int]) -> None:
        """Copy-on-write copies, in every layer slot and array of the group."""
        from .. import ops
        s = torch.tensor(list(src), dtype=torch.int32, device=self.device)
        d = torch.tensor(list(dst), dtype=torch.int32, device=self.device)
        for t in self.arrays[group].values():
            ops.copy_pages(t, s, d)

    def zero_state(self, slot: int) -> None:
        if self.state is not None:
            self.state[slot].zero_()

    def zero_states(self, slots: Sequence[int]) -> None:
        """Clear the state of several requests at once (those that start at position 0)."""
        if self.state is not None and len(slots):
            self.state[torch.tensor(list(slots), dtype=torch.long, device=self.device)] = 0

    def copy_state(self, src: int, dst: int) -> None:
        if self.state is not None:
            self.state[dst].copy_(self.state[src])

    def bytes_per_page(self, group: int) -> int:
        return sum(t.shape[0] * t[0, 0].numel() * t.element_size()
                   for t in self.arrays[group].values())
