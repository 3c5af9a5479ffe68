"""Python face of the native page manager (``csrc/runtime/cache_manager.cpp``).

``CacheManager`` decides which physical pages hold which request's positions, per page group,
and which state slot a request owns; it holds no GPU memory (``pools.py`` does).  Its
behaviour follows the reference's ``BlockManager`` (crates/kvcache/src/lib.rs:177-438):
``reserve`` is all-or-nothing and returns the copy-on-write copies to perform, ``free``
returns everything, ``check_invariants`` verifies that no page is lost, held twice or freed
twice.  A reservation makes positions addressable and the pages from the computed length on
the request's own, so a request that shares pages after a ``fork`` gets its copies before it
writes, however far ahead it had reserved."""
from __future__ import annotations

import ctypes
from ctypes import POINTER, c_char_p, c_int, c_longlong, c_void_p
from dataclasses import dataclass
from typing import List, Optional, Sequence, Tuple

_RT: Optional[ctypes.CDLL] = None


def runtime() -> ctypes.CDLL:
    """The host runtime library, built on first use (g++ only, no GPU needed)."""
    global _RT
    if _RT is None:
        from ..csrc import build
        lib = ctypes.CDLL(build.ensure("runtime"))
        PI, PL = POINTER(c_int), POINTER(c_longlong)
        sig = {
            "rlis_rt_last_error": (c_char_p, []),
            "rlis_cache_create": (c_void_p, [c_int, c_int, PI, PI, c_int]),
            "rlis_cache_destroy": (None, [c_void_p]),
            "rlis_cache_reserve": (c_int, [c_void_p, c_longlong, c_int, PI, c_int, PI]),
            "rlis_cache_advance": (c_int, [c_void_p, c_longlong, c_int]),
            "rlis_cache_fork": (c_int, [c_void_p, c_longlong, c_longlong, PI]),
            "rlis_cache_free": (c_int, [c_void_p, c_longlong]),
            "rlis_cache_num_free": (c_int, [c_void_p, c_int]),
            "rlis_cache_num_pages": (c_int, [c_void_p, c_int]),
            "rlis_cache_refcount": (c_int, [c_void_p, c_int, c_int]),
            "rlis_cache_num_free_slots": (c_int, [c_void_p]),
            "rlis_cache_contains": (c_int, [c_void_p, c_longlong]),
            "rlis_cache_pages_needed": (c_int, [c_void_p, c_longlong, c_int, c_int]),
            "rlis_cache_table": (c_int, [c_void_p, c_longlong, c_int, PI, c_int]),
            "rlis_cache_info": (c_int, [c_void_p, c_longlong, PI]),
            "rlis_cache_check": (c_int, [c_void_p, c_char_p, c_int]),
            "rlis_cache_decode_batch": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p,
                                                c_void_p, c_void_p, c_void_p]),
            "rlis_cache_step_layout": (c_longlong, [c_void_p, c_int, c_void_p, c_void_p, c_void_p,
                                                    c_void_p, c_void_p, c_void_p, c_void_p,
                                                    c_void_p]),
            "rlis_cache_step_fill": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p,
                                             c_void_p, c_void_p, c_int, c_void_p, c_longlong]),
            "rlis_fill_normal": (c_int, [c_void_p, c_longlong, ctypes.c_ulonglong,
                                         ctypes.c_ulonglong, ctypes.c_double, ctypes.c_double,
                                         c_int]),
            "rlis_sched_create": (c_void_p, [c_void_p, c_int, c_int, c_int, c_int]),
            "rlis_sched_destroy": (None, [c_void_p]),
            "rlis_sched_add": (c_int, [c_void_p, c_longlong, c_int]),
            "rlis_sched_schedule": (c_int, [c_void_p, PL, c_int, PI, PL, c_int, PI, PI, c_int, PI]),
            "rlis_sched_advance": (c_int, [c_void_p, c_longlong, c_int]),
            "rlis_sched_append_token": (c_int, [c_void_p, c_longlong]),
            "rlis_sched_append_tokens": (c_int, [c_void_p, PL, c_int]),
            "rlis_sched_is_caught_up": (c_int, [c_void_p, c_longlong]),
            "rlis_sched_remove": (c_int, [c_void_p, c_longlong]),
            "rlis_sched_has_work": (c_int, [c_void_p]),
            "rlis_sched_num_running": (c_int, [c_void_p]),
            "rlis_sched_num_waiting": (c_int, [c_void_p]),
            "rlis_sched_num_preemptions": (c_longlong, [c_void_p]),
            "rlis_sched_max_seq_tokens": (c_int, [c_void_p]),
            "rlis_sched_num_tokens": (c_int, [c_void_p, c_longlong]),
            "rlis_sched_num_computed": (c_int, [c_void_p, c_longlong]),
            "rlis_sched_check": (c_int, [c_void_p, c_char_p, c_int]),
        }
        for name, (res, args) in sig.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _RT = lib
    return _RT


def rt_error() -> str:
    return runtime().rlis_rt_last_error().decode("utf-8", "replace")


class OutOfPages(Exception):
    """No group has the pages (or no state slot is free) for a reservation; nothing changed."""


@dataclass(frozen=True)
class GroupSpec:
    """A page group: ``window`` None keeps every position, an integer only the latest ones."""
    num_pages: int
    window: Optional[int] = None


@dataclass(frozen=True)
class PageCopy:
    group: int
    src: int
    dst: int


class CacheManager:
    def __init__(self, page_size: int, groups: Sequence[GroupSpec], num_state_slots: int = 0):
        self.page_size = int(page_size)
        self.groups = list(groups)
        self.num_state_slots = int(num_state_slots)
        rt = runtime()
        n = len(self.groups)
        windows = (c_int * n)(*[int(g.window or 0) for g in self.groups])
        pages = (c_int * n)(*[int(g.num_pages) for g in self.groups])
        self._h = rt.rlis_cache_create(self.page_size, n, windows, pages, self.num_state_slots)
        if not self._h:
            raise ValueError(rt_error())
        self._copies = (c_int * (3 * 4 * max(1, n)))()
        self._n = c_int(0)
        self._info = (c_int * 3)()

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h and _RT is not None:
            _RT.rlis_cache_destroy(h)

    # ------------------------------------------------------------------ queries
    @property
    def num_groups(self) -> int:
        return len(self.groups)

    def num_free_pages(self, group: int = 0) -> int:
        return runtime().rlis_cache_num_free(self._h, group)

    def num_pages(self, group: int = 0) -> int:
        return runtime().rlis_cache_num_pages(self._h, group)

    def refcount(self, group: int, page: int) -> int:
        return runtime().rlis_cache_refcount(self._h, group, page)

    def num_free_slots(self) -> int:
        return runtime().rlis_cache_num_free_slots(self._h)

    def contains(self, seq: int) -> bool:
        return bool(runtime().rlis_cache_contains(self._h, seq))

    def pages_for(self, tokens: int) -> int:
        return -(-tokens // self.page_size)

    def pages_needed(self, seq: int, total_tokens: int, group: int = 0) -> int:
        return runtime().rlis_cache_pages_needed(self._h, seq, total_tokens, group)

    def table(self, seq: int, group: int = 0) -> List[int]:
        """Physical page of every logical page of ``seq`` (-1 once a window has passed it)."""
        rt = runtime()
        cap = 64
        while True:
            buf = (c_int * cap)()
            n = rt.rlis_cache_table(self._h, seq, group, buf, cap)
            if n < 0:
                raise KeyError(f"request {seq} holds no pages")
            if n <= cap:
                return list(buf[:n])
            cap = n

    def _get_info(self, seq: int) -> Tuple[int, int, int]:
        if runtime().rlis_cache_info(self._h, seq, self._info) != 0:
            raise KeyError(f"request {seq} holds no pages")
        return self._info[0], self._info[1], self._info[2]

    def num_tokens(self, seq: int) -> int:
        """Positions of ``seq`` with a slot reserved."""
        return self._get_info(seq)[0]

    def num_computed(self, seq: int) -> int:
        return self._get_info(seq)[1] if self.contains(seq) else 0

    def state_slot(self, seq: int) -> int:
        return self._get_info(seq)[2]

    # ---------------------------------------------------------------- mutations
    def reserve(self, seq: int, total_tokens: int) -> List[PageCopy]:
        """Make positions ``[0, total_tokens)`` of ``seq`` addressable (all or nothing)."""
        rc = runtime().rlis_cache_reserve(self._h, seq, total_tokens, self._copies,
                                          len(self._copies) // 3, self._n)
        if rc < 0:
            raise RuntimeError(rt_error())
        if rc != 0:
            raise OutOfPages("out of cache pages" if rc == 1 else "out of state slots")
        c = self._copies
        return [PageCopy(c[3 * i], c[3 * i + 1], c[3 * i + 2]) for i in range(self._n.value)]

    def advance(self, seq: int, computed: int) -> None:
        """Positions ``[0, computed)`` are written; pages behind a window go back."""
        if runtime().rlis_cache_advance(self._h, seq, computed) != 0:
            raise ValueError(rt_error())

    def fork(self, parent: int, child: int) -> Tuple[int, int]:
        """``child`` shares the pages of ``parent``'s computed positions (what ``parent`` has
        reserved beyond them stays its own).  Returns the state slots ``(parent's, child's)``
        whose contents the device must copy, ``(-1, -1)`` without state slots."""
        seats = (c_int * 2)()
        if runtime().rlis_cache_fork(self._h, parent, child, seats) != 0:
            raise ValueError(rt_error())
        return seats[0], seats[1]

    def free(self, seq: int) -> None:
        if runtime().rlis_cache_free(self._h, seq) != 0:
            raise RuntimeError(rt_error())

    def decode_batch(self, seqs_ptr: int, n: int, width: int, positions_ptr: int,
                     state_slots_ptr: int, tables_ptrs, slots_ptrs) -> None:
        """Fill the metadata of a step of one token per request straight into caller-owned
        int32 buffers (see ``rlis_cache_decode_batch``); ``tables_ptrs`` and ``slots_ptrs``
        are ctypes arrays of one pointer per group."""
        if runtime().rlis_cache_decode_batch(self._h, seqs_ptr, n, width, positions_ptr,
                                             state_slots_ptr, tables_ptrs, slots_ptrs) != 0:
            raise ValueError(rt_error())

    def step_layout(self, n: int, seqs_ptr: int, counts_ptr: int, tokens_ptr: int,
                    want_counts_ptr: int, wants_ptr: int, info_ptr: int, offsets_ptr: int,
                    order_ptr: int) -> int:
        """Sizes, array offsets and sequence order of a step's common metadata (see
        ``rlis_cache_step_layout``); returns the buffer's size in int32 elements."""
        total = runtime().rlis_cache_step_layout(self._h, n, seqs_ptr, counts_ptr, tokens_ptr,
                                                 want_counts_ptr, wants_ptr, info_ptr, offsets_ptr,
                                                 order_ptr)
        if total < 0:
            raise ValueError(rt_error())
        return total

    def step_fill(self, n: int, seqs_ptr: int, counts_ptr: int, tokens_ptr: int,
                  want_counts_ptr: int, wants_ptr: int, vocab_size: int, buf_ptr: int,
                  capacity: int) -> None:
        """Fill a step's common metadata into a caller-owned int32 buffer."""
        if runtime().rlis_cache_step_fill(self._h, n, seqs_ptr, counts_ptr, tokens_ptr,
                                          want_counts_ptr, wants_ptr, vocab_size, buf_ptr,
                                          capacity) != 0:
            raise ValueError(rt_error())

    def check_invariants(self) -> None:
        buf = ctypes.create_string_buffer(512)
        if runtime().rlis_cache_check(self._h, buf, 512) != 0:
            raise AssertionError(buf.value.decode())
