"""Per-step metadata: what one batch of (request, its next tokens) looks like to the kernels.

The reference builds the same per step in ``PagedBatch::new`` (crates/model/src/paged.rs:
256-296): positions ``P_i .. P_i + n_i`` of every sequence concatenated in batch order
(llama.rs:252), the write slot ``table[pos / page] * page + pos % page`` of every new token
(paged.rs:258-263), zero-padded block tables and context lengths (paged.rs:199-213).  Here one
slot id per token is enough (the write kernel spreads it over heads and dims), and all of it
goes to the device in one copy.

What is laid out here is common to every mixer, and the host runtime does it (one pass in C++
over the requests' leases, ``csrc/runtime/step_builder.cpp``; ``build_step_in_python`` is its
twin).  What only one kind of mixer needs (the work lists of its kernels) comes from that
mixer's ``StepPlanner`` and is carried along unseen: ``build_step`` calls each planner with the
step's host-side lengths and packs the arrays it returns into the same buffer
(``step.plans[key]``)."""
from __future__ import annotations

import itertools
from dataclasses import dataclass, field
from typing import Any, Callable, Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..stepplan import HostPlan, StepLengths, StepPlan, StepPlanner


@dataclass
class StepEntry:
    """One request's part of a step: its next ``tokens`` (continuing exactly at its cached
    length) and ``want``, the indices among them whose logits are asked for."""
    seq_id: int
    tokens: Sequence[int]
    want: Sequence[int] = ()


@dataclass
class GroupStep:
    page_size: int
    window: Optional[int]
    block_tables: torch.Tensor        # (S, max_pages) int32
    slots: torch.Tensor               # (T) int32


@dataclass
class StepContext:
    num_tokens: int
    num_seqs: int
    ids: torch.Tensor                 # (T) int32
    positions: torch.Tensor           # (T) int32, absolute
    seq_of_token: torch.Tensor        # (T) int32, index into the step's sequences
    cu_seqlens: torch.Tensor          # (S + 1) int32
    start_pos: torch.Tensor           # (S) int32: positions cached before the step
    ctx_lens: torch.Tensor            # (S) int32: positions cached after the step
    logit_rows: torch.Tensor          # (R) int32: token rows whose logits are wanted
    num_logit_rows: int
    state_slots: torch.Tensor         # (S) int32
    groups: List[GroupStep]
    max_context: int
    max_new: int
    all_decode: bool
    # Sequences that bring a single token come first in the step: sequences (and token rows)
    # [0, num_single) are theirs, so that a decode kernel can take them beside the portions.
    num_single: int = 0
    # What the mixers' planners made of this step, by planner key.
    plans: Dict[Any, StepPlan] = field(default_factory=dict)
    # Host copies, for parts that plan on the host.
    lengths: Optional[StepLengths] = None
    host_start_pos: List[int] = field(default_factory=list)
    host_new: List[int] = field(default_factory=list)
    host_state_slots: List[int] = field(default_factory=list)
    host_order: List[int] = field(default_factory=list)   # entry index of every sequence
    # The one device buffer that all the arrays above are views of, and the same step over
    # another buffer of that layout (for a captured step, whose kernels read a buffer that
    # stays where it is).
    buffer: Optional[torch.Tensor] = None
    over: Optional[Callable[[torch.Tensor], "StepContext"]] = None


class MetadataBuffer:
    """Named int32 arrays packed into one buffer, each starting on a 16-byte boundary, so that
    a step's metadata reaches the device in one copy.  The eager step builder fills one per
    step; a captured decode step keeps one of fixed sizes and rewrites it in place."""

    def __init__(self) -> None:
        self.offsets: Dict[str, Tuple[int, int]] = {}
        self.size = 0
        self._chunks: List[np.ndarray] = []

    def put(self, name: str, values) -> None:
        arr = np.asarray(values, dtype=np.int32).reshape(-1)
        self.reserve(name, arr.size)
        self._chunks.append(arr)
        pad = -arr.size % 4
        if pad:
            self._chunks.append(np.zeros(pad, dtype=np.int32))

    def reserve(self, name: str, count: int) -> None:
        if name in self.offsets:
            raise KeyError(f"metadata array '{name}' is laid out twice")
        self.offsets[name] = (self.size, int(count))
        self.size += -(-int(count) // 4) * 4

    def packed(self) -> torch.Tensor:
        if not self._chunks:
            return torch.zeros(0, dtype=torch.int32)
        return torch.from_numpy(np.concatenate(self._chunks))

    def view(self, buf, name: str):
        o, n = self.offsets[name]
        return buf[o:o + n]


def plan_name(index: int, array: str) -> str:
    return f"plan{index}.{array}"


# The arrays that every step carries and how long each is (T tokens, S sequences, R wanted rows),
# in the order of the host runtime's layout (csrc/runtime/step_builder.h); each page group adds
# its write slots and its block tables, W pages wide.  This one table lays out the eager step
# (the runtime's and its Python twin's) and the static buffer of a captured step: an array is
# declared here once, and filled by the runtime's builder and by the twin.
COMMON_ARRAYS = (("ids", "T"), ("positions", "T"), ("seq_of_token", "T"), ("cu", "S+1"),
                 ("start_pos", "S"), ("ctx_lens", "S"), ("logit_rows", "R"), ("state_slots", "S"))
GROUP_ARRAYS = (("slots{g}", "T"), ("tables{g}", "S*W"))


def common_layout(T: int, S: int, R: int, widths: Sequence[int]) -> List[Tuple[str, int]]:
    """(name, length) of every common array of a step with ``T`` tokens, ``S`` sequences and
    ``R`` wanted rows whose page groups have block tables ``widths`` pages wide, in order."""
    def length(kind: str, W: int = 0) -> int:
        return {"T": T, "S": S, "S+1": S + 1, "R": R, "S*W": S * W}[kind]
    out = [(name, length(kind)) for name, kind in COMMON_ARRAYS]
    for g, W in enumerate(widths):
        out += [(name.format(g=g), length(kind, W)) for name, kind in GROUP_ARRAYS]
    return out


def _common_native(entries: Sequence[StepEntry], cache, vocab_size: int, spare: int):
    """The common arrays laid out by the host runtime (one pass in C++ over the requests'
    leases).  Returns (pinned buffer with ``spare`` ints of room behind the layout, offsets by
    name as (offset, count), info) with info = (T, S, R, single-token sequences, longest
    context, most new tokens, widths per group, order)."""
    n = len(entries)
    ng = cache.num_groups
    counts = np.fromiter((len(e.tokens) for e in entries), dtype=np.int32, count=n)
    want_counts = np.fromiter((len(e.want) for e in entries), dtype=np.int32, count=n)
    seqs = np.fromiter((e.seq_id for e in entries), dtype=np.int64, count=n)
    try:
        tokens = np.fromiter(itertools.chain.from_iterable(e.tokens for e in entries),
                             dtype=np.int64, count=int(counts.sum()))
        wants = np.fromiter(itertools.chain.from_iterable(e.want for e in entries),
                            dtype=np.int32, count=int(want_counts.sum()))
    except (TypeError, ValueError):
        raise ValueError("a request's tokens and wanted indices must be flat lists of integers") \
            from None
    info = np.zeros(6 + ng, dtype=np.int32)
    offsets = np.zeros(len(COMMON_ARRAYS) + len(GROUP_ARRAYS) * ng, dtype=np.int64)
    order = np.zeros(n, dtype=np.int32)
    args = (n, seqs.ctypes.data, counts.ctypes.data, tokens.ctypes.data, want_counts.ctypes.data,
            wants.ctypes.data)
    total = cache.step_layout(*args, info.ctypes.data, offsets.ctypes.data, order.ctypes.data)
    host = torch.empty(total + spare, dtype=torch.int32, pin_memory=torch.cuda.is_available())
    cache.step_fill(*args, vocab_size, host.data_ptr(), total)
    T, S, R = int(info[0]), int(info[1]), int(info[2])
    widths = [int(w) for w in info[6:]]
    layout = {name: (int(o), int(c))
              for (name, c), o in zip(common_layout(T, S, R, widths), offsets)}
    return host, total, layout, (T, S, R, int(info[3]), int(info[4]), int(info[5]), widths,
                                 order.tolist())


def build_step(entries: Sequence[StepEntry], cache, device: torch.device,
               vocab_size: int, planners: Sequence[StepPlanner] = (),
               native: Optional[bool] = None) -> StepContext:
    """Lay out a step.  Every entry's request must hold reserved positions for its tokens.

    Inside the step the sequences are ordered single tokens first (``host_order`` maps them back
    to the entries); ``logit_rows`` keeps the order of the entries and of their ``want``.

    The common arrays are laid out by the host runtime where the cache manager is the runtime's
    (``native``; None: if it is); ``build_step_in_python`` does the same here, for caches of
    another kind and as the twin that tests hold the runtime's layout against."""
    if native is None:
        native = hasattr(cache, "step_fill")
    if not native:
        return build_step_in_python(entries, cache, device, vocab_size, planners)
    if not entries:
        raise ValueError("a step needs at least one request")
    # what the planners add is not known before the lengths are; their arrays go behind the
    # common ones, into room asked for up front (a second buffer when a plan outgrows it)
    spare = 256 + (16 * len(entries) + sum(len(e.tokens) for e in entries) // 4) \
        * max(1, len(planners))
    host, used, layout, info = _common_native(entries, cache, vocab_size, spare)
    T, S, R, num_single, max_context, max_new, widths, order = info
    ps = cache.page_size
    view_host = host.numpy()

    def host_view(name):
        o, c = layout[name]
        return view_host[o:o + c]

    start_pos = host_view("start_pos")
    new = np.diff(host_view("cu"))
    lengths = StepLengths(start_pos.astype(np.int64), new.astype(np.int64), num_single, ps)
    host_plans: List[Tuple[Any, HostPlan]] = []
    extra: List[Tuple[str, np.ndarray]] = []
    at = used
    for k, planner in enumerate(planners):
        plan = planner.plan(lengths)
        for name, arr in plan.arrays.items():
            arr = np.asarray(arr, dtype=np.int32).reshape(-1)
            layout[plan_name(k, name)] = (at, arr.size)
            extra.append((plan_name(k, name), arr))
            at += -(-arr.size // 4) * 4
        host_plans.append((planner.key(), plan))
    if at > host.numel():
        grown = torch.empty(at, dtype=torch.int32, pin_memory=host.is_pinned())
        grown[:used] = host[:used]
        host, view_host = grown, grown.numpy()
    for name, arr in extra:
        o, c = layout[name]
        view_host[o:o + c] = arr
    dev = host[:at].to(device, non_blocking=True)
    fixed = dict(num_tokens=T, num_seqs=S, num_logit_rows=R, max_context=max_context,
                 max_new=max_new, all_decode=num_single == S, num_single=num_single,
                 lengths=lengths, host_start_pos=start_pos.tolist(), host_new=new.tolist(),
                 host_state_slots=host_view("state_slots").tolist(), host_order=order)
    return _context_over(dev, layout, cache, widths, host_plans, fixed)


def _context_over(dev: torch.Tensor, layout: Dict[str, Tuple[int, int]], cache,
                  widths: Sequence[int], host_plans: Sequence[Tuple[Any, HostPlan]],
                  fixed: Dict[str, Any]) -> StepContext:
    """The step whose arrays are views of ``dev`` by ``layout`` (name -> (offset, count))."""
    def view(name):
        o, c = layout[name]
        return dev[o:o + c]

    S, ps = fixed["num_seqs"], cache.page_size
    groups = [GroupStep(page_size=ps, window=cache.groups[g].window,
                        block_tables=view(f"tables{g}").reshape(S, widths[g]),
                        slots=view(f"slots{g}")) for g in range(cache.num_groups)]
    plans = {key: StepPlan({name: view(plan_name(k, name)) for name in plan.arrays}, plan.values)
             for k, (key, plan) in enumerate(host_plans)}
    return StepContext(
        ids=view("ids"), positions=view("positions"), seq_of_token=view("seq_of_token"),
        cu_seqlens=view("cu"), start_pos=view("start_pos"), ctx_lens=view("ctx_lens"),
        logit_rows=view("logit_rows"), state_slots=view("state_slots"), groups=groups,
        plans=plans, buffer=dev,
        over=lambda other: _context_over(other, layout, cache, widths, host_plans, fixed),
        **fixed)


def build_step_in_python(entries: Sequence[StepEntry], cache, device: torch.device,
                         vocab_size: int, planners: Sequence[StepPlanner] = ()) -> StepContext:
    """``build_step`` with the common arrays laid out here, through the cache's ``table`` and
    ``_get_info`` alone."""
    if not entries:
        raise ValueError("a step needs at least one request")
    order = sorted(range(len(entries)), key=lambda i: len(entries[i].tokens) != 1)
    ps = cache.page_size
    S = len(entries)
    ids: List[np.ndarray] = []
    positions: List[np.ndarray] = []
    cu = [0]
    start_pos: List[int] = []
    ctx_lens: List[int] = []
    state_slots: List[int] = []
    new: List[int] = []
    ng = cache.num_groups
    tables: List[List[List[int]]] = [[] for _ in range(ng)]
    slots: List[List[np.ndarray]] = [[] for _ in range(ng)]
    seen = set()
    base_of = [0] * S
    for i in order:
        e = entries[i]
        n = len(e.tokens)
        if n == 0:
            raise ValueError("empty sequence in batch")          # llama.rs:231-233
        if e.seq_id in seen:
            raise ValueError(f"request {e.seq_id} appears twice in one step")
        seen.add(e.seq_id)
        if not cache.contains(e.seq_id):
            raise ValueError(f"request {e.seq_id}: position 0 has no page reserved")
        reserved, computed, slot = cache._get_info(e.seq_id)
        if computed + n > reserved:
            # paged.rs:258-263 "position {pos} has no block reserved"
            raise ValueError(f"request {e.seq_id}: position {reserved} has no page reserved")
        toks = np.asarray(e.tokens, dtype=np.int64)
        if toks.ndim != 1:
            raise ValueError(f"request {e.seq_id}: its tokens must be a flat list")
        if int(toks.min()) < 0 or int(toks.max()) >= vocab_size:
            bad = int(toks[(toks < 0) | (toks >= vocab_size)][0])
            raise ValueError(f"request {e.seq_id}: token id {bad} is outside the vocabulary "
                             f"of {vocab_size}")
        base_of[i] = cu[-1]
        ids.append(toks)
        pos = np.arange(computed, computed + n, dtype=np.int64)
        positions.append(pos)
        cu.append(cu[-1] + n)
        new.append(n)
        start_pos.append(computed)
        ctx_lens.append(computed + n)
        state_slots.append(max(slot, 0))
        for w in e.want:
            if not 0 <= int(w) < n:
                raise ValueError(f"request {e.seq_id}: wanted index {w} is outside its {n} tokens")
        for g in range(ng):
            table = cache.table(e.seq_id, g)
            tables[g].append(table)
            pages = np.asarray(table, dtype=np.int64)[pos // ps]
            if int(pages.min()) < 0:
                p = int(pos[pages < 0][0])
                raise ValueError(f"request {e.seq_id}: position {p} has no page reserved")
            slots[g].append(pages * ps + pos % ps)
    logit_rows = [base_of[i] + int(w) for i, e in enumerate(entries) for w in e.want]
    T = cu[-1]
    num_single = sum(1 for n in new if n == 1)
    widths = [max(8, -(-max(len(t) for t in tables[g]) // 8) * 8) for g in range(ng)]
    lengths = StepLengths(np.asarray(start_pos, dtype=np.int64), np.asarray(new, dtype=np.int64),
                          num_single, ps)

    made = {"ids": np.concatenate(ids), "positions": np.concatenate(positions),
            "seq_of_token": np.repeat(np.arange(S, dtype=np.int32), new), "cu": cu,
            "start_pos": start_pos, "ctx_lens": ctx_lens, "logit_rows": logit_rows,
            "state_slots": state_slots}
    for g in range(ng):
        made[f"slots{g}"] = np.concatenate(slots[g])
        rows = np.zeros((S, widths[g]), dtype=np.int32)
        for r, t in enumerate(tables[g]):
            rows[r, :len(t)] = np.maximum(np.asarray(t, dtype=np.int32), 0)
        made[f"tables{g}"] = rows
    meta = MetadataBuffer()
    for name, count in common_layout(T, S, len(logit_rows), widths):
        meta.put(name, made[name])
        if meta.offsets[name][1] != count:
            raise AssertionError(f"step array '{name}' has {meta.offsets[name][1]} entries, "
                                 f"the layout says {count}")
    host_plans: List[Tuple[Any, HostPlan]] = []
    for k, planner in enumerate(planners):
        plan = planner.plan(lengths)
        for name, arr in plan.arrays.items():
            meta.put(plan_name(k, name), arr)
        host_plans.append((planner.key(), plan))
    host = meta.packed()

    if device.type == "cuda":
        host = host.pin_memory()
    dev = host.to(device, non_blocking=True)
    fixed = dict(num_tokens=T, num_seqs=S, num_logit_rows=len(logit_rows),
                 max_context=max(ctx_lens), max_new=max(new), all_decode=num_single == S,
                 num_single=num_single, lengths=lengths, host_start_pos=start_pos, host_new=new,
                 host_state_slots=state_slots, host_order=order)
    return _context_over(dev, dict(meta.offsets), cache, widths, host_plans, fixed)
