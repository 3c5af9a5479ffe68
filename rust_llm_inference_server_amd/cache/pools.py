"""The device side of the cache: one pool of pages per group and one buffer of fixed-size
per-request state.

A group's pool holds, for every layer slot of the group, ``num_pages`` pages of keys
``[page][kv head][offset][d]`` and of values ``[page][kv head][d][offset]`` (values transposed
inside a page, so that both attention kernels read each as it lies).  One page id addresses
the same page in every layer slot of its group, as one block id addresses every layer in the
reference (crates/model/src/paged.rs:1-7, 41-60).  Pools are allocated once, zeroed."""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch

from ..parts.base import CacheBinding


class CachePools:
    def __init__(self, cache_groups: Sequence, num_pages: Sequence[int], page_size: int,
                 dtype: torch.dtype, device: torch.device, num_state_slots: int = 0,
                 state_bytes: int = 0):
        self.page_size = page_size
        self.dtype = dtype
        self.k: List[torch.Tensor] = []
        self.v: List[torch.Tensor] = []
        # One page beyond the manager's is scratch: padding rows of a captured decode step
        # read and write it, so they touch nothing a request owns.
        self.scratch_page = max(num_pages) if len(num_pages) else 0
        for layout, pages in zip(cache_groups, num_pages):
            r, n = layout.request, max(1, len(layout.writer_runs))
            total = self.scratch_page + 1
            self.k.append(torch.zeros((n, total, r.num_kv_heads, page_size, r.head_dim),
                                      dtype=dtype, device=device))
            self.v.append(torch.zeros((n, total, r.num_kv_heads, r.head_dim, page_size),
                                      dtype=dtype, device=device))
        self.state: Optional[torch.Tensor] = None
        if state_bytes > 0 and num_state_slots > 0:
            self.state = torch.zeros((num_state_slots, state_bytes), dtype=torch.uint8,
                                     device=device)

    def binding(self, rb) -> CacheBinding:
        b = CacheBinding(group=rb.group, writes=rb.writes)
        if rb.group >= 0:
            b.k_pages = self.k[rb.group][rb.slot]
            b.v_pages = self.v[rb.group][rb.slot]
        if rb.state_bytes and self.state is not None:
            b.state = self.state[:, rb.state_offset:rb.state_offset + rb.state_bytes]
        return b

    def copy_pages(self, group: int, src: Sequence[int], dst: Sequence[int]) -> None:
        """Copy-on-write copies, in every layer slot of the group."""
        from .. import ops
        dev = self.k[group].device
        s = torch.tensor(list(src), dtype=torch.int32, device=dev)
        d = torch.tensor(list(dst), dtype=torch.int32, device=dev)
        ops.copy_pages(self.k[group], s, d)
        ops.copy_pages(self.v[group], s, d)

    def zero_state(self, slot: int) -> None:
        if self.state is not None:
            self.state[slot].zero_()

    def bytes_per_page(self, group: int) -> int:
        k = self.k[group]
        return 2 * k.shape[0] * k[0, 0].numel() * k.element_size()
