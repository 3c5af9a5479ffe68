"""The step function and what it owns: the model's parts, the page manager and the pools.

``ModelRunner.step(entries)`` runs one batch of (request, its next tokens): portions of
prompts beside single decoded tokens, cut anywhere.  It computes only the tokens it is given,
reads everything earlier from the cache, writes the new keys and values there, and returns
float32 logits at the wanted rows.  It is the one forward path: the engine, the replay
program, the perplexity tool and the benchmark all call it.  Its contract is the reference's
``Llama::forward_batch`` over a ``PagedBatch`` (crates/model/src/llama.rs:216-286;
crates/model/src/paged.rs:154-161, 255-296)."""
from __future__ import annotations

import os
from typing import Callable, Dict, List, Optional, Sequence, Tuple, Union

import torch

from ..cache.manager import CacheManager, GroupSpec
from ..cache.pools import CachePools
from ..config.generation import read_eos_token_ids
from ..models.spec import Model
from ..registry import architecture_of, read_config_dict
from ..weights.loader import load_weights
from ..weights.random_init import random_weights
from .batch import StepEntry, build_step

DTYPES = {"float32": torch.float32, "fp32": torch.float32, "f32": torch.float32,
          "bfloat16": torch.bfloat16, "bf16": torch.bfloat16}


def parse_dtype(name: Union[str, torch.dtype]) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.float32, torch.bfloat16):
            raise ValueError(f"dtype {name} is not supported (float32 or bfloat16)")
        return name
    try:
        return DTYPES[name.lower()]
    except KeyError:
        raise ValueError(f"dtype '{name}' is not supported (float32 or bfloat16)") from None


def default_device() -> torch.device:
    if not torch.cuda.is_available():
        raise RuntimeError("no GPU is visible: this engine runs on an AMD GPU only")
    return torch.device("cuda", torch.cuda.current_device())


def load_model(folder: str, dtype: Union[str, torch.dtype], max_positions: int,
               device: Optional[torch.device] = None) -> Model:
    """Build the model a folder holds: the architecture named in ``config.json`` chooses the
    configuration class and the specification, the safetensors files give the weights."""
    device = device or default_device()
    act = parse_dtype(dtype)
    cfg_dict = read_config_dict(folder)
    arch = architecture_of(cfg_dict)
    cfg = arch.parse_config(cfg_dict)
    spec = arch.build_spec(cfg)
    weights = load_weights(folder, spec.tensor_specs(), act, device, spec.optional_tensors)
    limit = getattr(cfg, "max_position_embeddings", max_positions)
    model = Model(spec, weights, act, device, min(max_positions, limit))
    model.config = cfg
    # generation_config.json first, config.json second (crates/engine/src/tokenizer.rs:64-85)
    model.eos_token_ids = read_eos_token_ids(folder) if os.path.isdir(folder) else ()
    return model


def random_model(config: Union[dict, object], seed: int, dtype: Union[str, torch.dtype],
                 max_positions: int, device: Optional[torch.device] = None,
                 architecture: Optional[str] = None) -> Model:
    """A model with seeded random weights, built in memory from a configuration: a config.json
    dict (its ``architectures`` names the model) or a typed configuration (its ``architecture``
    does); ``architecture`` names it for a configuration that does not."""
    from ..registry import architecture as lookup
    device = device or default_device()
    act = parse_dtype(dtype)
    if isinstance(config, dict):
        arch = lookup(architecture) if architecture else architecture_of(config)
        cfg = arch.parse_config(config)
    else:
        name = architecture or getattr(config, "architecture", None)
        if not name:
            raise ValueError("random_model: the configuration names no architecture")
        arch, cfg = lookup(name), config
    spec = arch.build_spec(cfg)
    weights = random_weights(spec.tensor_specs(), seed, act, device)
    limit = getattr(cfg, "max_position_embeddings", max_positions)
    model = Model(spec, weights, act, device, min(max_positions, limit))
    model.config = cfg
    return model


class ModelRunner:
    """A model with its cache.  ``num_pages`` sizes every page group's pool: one number for
    all of them, or one per group (``cache.pools.pool_pages`` makes those from a budget)."""

    def __init__(self, model: Model, num_pages: Union[int, Sequence[int]], page_size: int = 16,
                 max_num_seqs: int = 64, max_batched_tokens: Optional[int] = None,
                 use_graphs: bool = True):
        self.model = model
        self.use_graphs = use_graphs and model.device.type == "cuda" and model.graph_safe
        self._graphs: Dict[int, object] = {}
        # other steps than pure decode steps are captured when their shape comes back
        # (engine/graph.py::RepeatedSteps)
        self.capture_repeated_steps = True
        self._repeated = None
        self.device = model.device
        self.page_size = page_size
        self.max_num_seqs = max_num_seqs
        self.max_batched_tokens = max_batched_tokens
        if isinstance(num_pages, int):
            per_group = [num_pages] * max(1, len(model.cache_groups))
        else:
            per_group = [int(n) for n in num_pages]
            if len(per_group) != max(1, len(model.cache_groups)):
                raise ValueError(f"{len(per_group)} pool sizes for "
                                 f"{len(model.cache_groups)} page groups")
        groups = [GroupSpec(n, g.request.window) for n, g in zip(per_group, model.cache_groups)]
        if not groups:
            groups = [GroupSpec(per_group[0], None)]   # the manager always has one group
        self.cache = CacheManager(page_size, groups,
                                  max_num_seqs if model.state_bytes else 0)
        self.pools = CachePools(model.cache_groups, per_group[:len(model.cache_groups)],
                                page_size, model.act_dtype, model.device,
                                max_num_seqs if model.state_bytes else 0, model.state_bytes)
        self.vocab_size = model.spec.vocab_size

    # ------------------------------------------------------------------- pages
    def reserve(self, seq_id: int, total_tokens: int) -> None:
        """Make positions ``[0, total_tokens)`` of a request addressable; raises
        ``OutOfPages`` (and changes nothing) when the pools cannot hold them."""
        if total_tokens > self.model.max_positions:
            raise ValueError(f"sequence of {total_tokens} positions exceeds max_seq_len "
                             f"{self.model.max_positions}")
        self.apply_copies(self.cache.reserve(seq_id, total_tokens))

    def apply_copies(self, copies) -> None:
        by_group: Dict[int, List] = {}
        for c in copies:
            by_group.setdefault(c.group, []).append(c)
        for g, cs in by_group.items():
            if g < len(self.pools.arrays):
                self.pools.copy_pages(g, [c.src for c in cs], [c.dst for c in cs])

    def fork(self, parent: int, child: int) -> None:
        """``child`` continues from what ``parent`` has computed: it shares those pages (the
        first of the two to write into a shared page gets its own copy, made when it reserves)
        and starts from a copy of the parent's state."""
        src, dst = self.cache.fork(parent, child)
        if src >= 0 and dst >= 0:
            self.pools.copy_state(src, dst)

    def free(self, seq_id: int) -> None:
        self.cache.free(seq_id)

    def num_computed(self, seq_id: int) -> int:
        return self.cache.num_computed(seq_id)

    # -------------------------------------------------------------------- step
    def step(self, entries: Sequence[StepEntry], keep: bool = True) -> torch.Tensor:
        """Run one batch; returns float32 logits ``(wanted rows, vocab)`` in the order of the
        entries and of their ``want`` lists.  The tensor is the caller's to keep; with
        ``keep=False`` it may be a view of a captured step's static output, which the next
        step overwrites (for callers that are done with the logits before they step again)."""
        if len(entries) > self.max_num_seqs:
            raise ValueError(f"{len(entries)} requests in one step, max_num_seqs is "
                             f"{self.max_num_seqs}")
        total = sum(len(e.tokens) for e in entries)
        if self.use_graphs and total == len(entries) and total > 0:
            return self._decode_step(entries, keep)
        if self.max_batched_tokens is not None and total > self.max_batched_tokens:
            raise ValueError(f"{total} tokens in one step, max_batched_tokens is "
                             f"{self.max_batched_tokens}")
        step = build_step(entries, self.cache, self.device, self.vocab_size,
                          self.model.step_planners)
        if step.max_context > self.model.max_positions:
            raise ValueError(f"sequence of {step.max_context} positions exceeds max_seq_len "
                             f"{self.model.max_positions}")
        if self.pools.state is not None:
            # a fresh (or recomputed) request starts from cleared state
            self.pools.zero_states([slot for start, slot in zip(step.host_start_pos,
                                                                step.host_state_slots)
                                    if start == 0])
        logits = None
        if self.use_graphs and self.capture_repeated_steps:
            if self._repeated is None:
                from .graph import RepeatedSteps
                self._repeated = RepeatedSteps(self)
            logits = self._repeated.run(step)
            if logits is not None and keep:
                logits = logits.clone()
        if logits is None:
            logits = self.model.forward(step, self.pools)
        for i, start in zip(step.host_order, step.host_start_pos):
            self.cache.advance(entries[i].seq_id, start + len(entries[i].tokens))
        return logits

    def step_sampled(self, seq_ids: Sequence[int], tokens: Sequence[int],
                     modes: Sequence[Tuple[int, float]]) -> Optional[Callable[[], List[int]]]:
        """A step of one token per request with the sampling kernel inside the captured step:
        request ``seq_ids[i]`` brings ``tokens[i]``, and ``modes[i]`` is its (key, 1/T) as
        ``Sampler.device_mode`` gives them.  The step is launched and a function comes back
        that waits for it and returns the sampled tokens in the order of the requests (what the
        host has to do meanwhile it does before calling it); None when this runner has no
        captured steps: then nothing has happened and ``step`` is to be called."""
        if not self.use_graphs or not seq_ids or len(seq_ids) > self.max_num_seqs:
            return None
        return self._decode_lists(seq_ids, tokens, modes)

    def step_chained(self, seq_ids: Sequence[int], modes: Sequence[Tuple[int, float]],
                     side: int) -> Callable[[], List[int]]:
        """The step that follows a ``step_sampled`` or ``step_chained`` of the same requests in
        the same order, launched while that step may still be running: every request brings
        the token that step samples for it, which is on the device and nowhere else yet.
        ``side`` (0 or 1) names the host buffers that the step uses; a step takes the side that
        the step before it did not (``step_sampled`` takes side 0), and the tokens of the step
        that had this side last must have been taken: at most two steps are under way.
        Positions must be reserved as for any step.  Returns the function that waits for this
        step's tokens."""
        if not self.use_graphs:
            raise ValueError("chained steps need captured steps")
        return self._decode_lists(seq_ids, None, modes, side)

    def capture_decode_steps(self, longest: Optional[int] = None, sampled: bool = True,
                             max_batch: Optional[int] = None) -> int:
        """Capture now what decode steps would capture at first use: the step of every batch
        bucket up to ``max_batch`` requests (``max_num_seqs`` by default) for every context
        bucket up to ``longest`` positions (the model's limit by default); with ``sampled`` the
        steps that sample inside, else those that return logits.  The captures run on padding
        and move no request's cache or state.  Returns how many graphs were captured (0
        without captured steps)."""
        if not self.use_graphs:
            return 0
        from .graph import LOGITS, SAMPLED, DecodeGraph, bucket_for, context_bucket
        limit = self.model.max_positions
        longest = limit if longest is None else max(1, min(longest, limit))
        top = self.max_num_seqs if max_batch is None else max(1, min(max_batch, self.max_num_seqs))
        buckets, n = [], 1
        while True:
            b = bucket_for(n, self.max_num_seqs)
            buckets.append(b)
            if b >= top:
                break
            n = b + 1
        contexts, c = [], 1
        while True:
            cb = context_bucket(c, limit)
            contexts.append(cb)
            if cb >= longest:
                break
            c = cb + 1
        made = 0
        kind = SAMPLED if sampled else LOGITS
        for b in buckets:
            graph = self._graphs.get(b)
            if graph is None:
                graph = self._graphs[b] = DecodeGraph(self, b)
            for cb in contexts:
                if (cb, kind) not in graph.graphs:
                    graph._capture(cb, kind)
                    made += 1
        return made

    def _decode_step(self, entries: Sequence[StepEntry], keep: bool = True) -> torch.Tensor:
        """A step of one token per request, replayed from the HIP graph of its batch-size
        bucket (captured at first use).  Same kernels, same results as the eager step.  The
        graph's output is static; ``keep`` copies what is returned out of it."""
        S = len(entries)
        rows: List[int] = []
        for i, e in enumerate(entries):
            for w in e.want:
                if int(w) != 0:
                    raise ValueError(f"request {e.seq_id}: wanted index {w} is outside its 1 tokens")
                rows.append(i)
        logits = self._decode_lists([e.seq_id for e in entries],
                                    [int(e.tokens[0]) for e in entries], None)
        if rows == list(range(S)):
            return logits.clone() if keep else logits
        if not rows:
            return logits[:0].clone()
        return logits[torch.tensor(rows, device=logits.device)]      # (indexing copies)

    def _decode_lists(self, seq_ids: Sequence[int], tokens: Optional[Sequence[int]],
                      modes: Optional[Sequence[Tuple[int, float]]], side: int = 0):
        """The captured step for requests ``seq_ids`` bringing ``tokens``: the logits of all of
        them, or with ``modes`` (the graph samples too) the function that waits for the tokens.
        ``tokens`` None: the chained step, on the tokens that the step before left on the
        device."""
        from .graph import DecodeGraph, bucket_for, context_bucket
        S = len(seq_ids)
        if len(set(seq_ids)) != S:
            raise ValueError("a request appears twice in one step")
        if tokens is not None and (min(tokens) < 0 or max(tokens) >= self.vocab_size):
            raise ValueError(f"a token id is outside the vocabulary of {self.vocab_size}")
        bucket = bucket_for(S, self.max_num_seqs)
        graph = self._graphs.get(bucket)
        if graph is None:
            if tokens is None:
                raise ValueError("a chained step follows a captured step of the same requests")
            graph = self._graphs[bucket] = DecodeGraph(self, bucket)
        positions = graph.prepare(seq_ids, tokens, modes, side)
        # Everything that can refuse the step is checked before anything is launched.
        longest = int(positions.max()) + 1
        if longest > self.model.max_positions:
            raise ValueError(f"sequence of {longest} positions exceeds max_seq_len "
                             f"{self.model.max_positions}")
        if self.pools.state is not None:
            # a request whose first token this is starts from cleared state
            slots = graph.sides[side].h["state_slots"]
            self.pools.zero_states([int(slots[i]) for i in range(S) if positions[i] == 0])
        ends = (positions + 1).tolist()
        limit = context_bucket(longest, self.model.max_positions)
        if modes is not None:
            result = graph.launch_sampled(S, limit, side, chained=tokens is None)
        else:
            result = graph.launch(S, limit)
        for seq, end in zip(seq_ids, ends):
            self.cache.advance(seq, end)
        return result
