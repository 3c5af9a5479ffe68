"""The request loop: admit, schedule, step, sample, finish, free.

What the reference's engine thread does each iteration (crates/engine/src/engine.rs:500-531,
617-726), without the thread and the channels: ``add_request`` validates and queues a request,
``step`` runs one scheduled batch through the model and samples a token for every request
whose tokens are all computed, ``generate`` loops until its requests are finished.

Finishing follows ``Sequence::accept`` (engine.rs:404-429): an EOS token (unless
``ignore_eos``) ends the request with reason ``stop`` and is not appended; reaching
``max_tokens`` ends it with reason ``length``.  When pages run out the scheduler preempts the
newest request, which later recomputes its prompt and its generated tokens in one prefill and,
its sampling being keyed by position, continues with the same tokens (engine.rs tests
157-194)."""
from __future__ import annotations

import time
from dataclasses import dataclass
from typing import Callable, Dict, Iterable, List, Optional, Sequence, Tuple, Union

import torch

from ..cache.pools import pool_pages
from ..config.engine import EngineConfig
from ..models.spec import Model
from ..sampling.params import SamplingParams
from ..sampling.sampler import Sampler, sample_on_device
from .batch import StepEntry
from .runner import ModelRunner, load_model
from .scheduler import Scheduler


@dataclass
class Completion:
    """What a finished request returns (engine.rs:139-158 ``Finish``)."""
    request_id: int
    token_ids: List[int]
    finish_reason: str                 # "stop", "length" or "error"
    prompt_tokens: int
    ttft: float                        # seconds from arrival to the first token
    decode_time: float                 # seconds from the first token to the last
    error: Optional[str] = None        # with "error": what the failed step said

    @property
    def completion_tokens(self) -> int:
        return len(self.token_ids)

    @property
    def decode_tokens_per_sec(self) -> float:
        """(completion - 1) / decode_time (engine.rs:150-157)."""
        if self.completion_tokens < 2 or self.decode_time <= 0:
            return 0.0
        return (self.completion_tokens - 1) / self.decode_time


@dataclass
class EngineStats:
    steps: int = 0
    prefill_tokens: int = 0
    generated_tokens: int = 0
    preemptions: int = 0
    running: int = 0
    waiting: int = 0
    pages_used: int = 0
    pages_total: int = 0


@dataclass
class _Flight:
    """A launched step of one token per request whose tokens the host has not taken yet."""
    ids: List[int]                     # the requests, in the order of the step's rows
    wait: Callable[[], List[int]]      # waits for the step, returns their tokens
    side: int                          # which of the runner's two host buffers it used
    appended: bool = False             # the scheduler has been told of its tokens already


class _Sequence:
    def __init__(self, seq_id: int, prompt: Sequence[int], params: SamplingParams):
        self.id = seq_id
        self.tokens = [int(t) for t in prompt]
        self.prompt_len = len(self.tokens)
        self.params = params
        self.sampler = Sampler(params)
        self.arrived = time.perf_counter()
        self.first_token_at: Optional[float] = None
        self.last_token_at: Optional[float] = None
        self.finish_reason: Optional[str] = None

    @property
    def output_len(self) -> int:
        return len(self.tokens) - self.prompt_len


class Engine:
    """``Engine(model, config)`` where ``model`` is a built ``Model`` or a model folder."""

    def __init__(self, model: Union[Model, str], config: Optional[EngineConfig] = None,
                 dtype: str = "bfloat16", eos_token_ids: Optional[Iterable[int]] = None):
        self.config = config or EngineConfig()
        self.config.validate()
        cfg = self.config
        if isinstance(model, str):
            model = load_model(model, dtype, max_positions=cfg.max_seq_len)
        self.model = model
        budget = max(cfg.max_batched_tokens, cfg.max_num_seqs)
        if model.device.type == "cuda":
            # steps that fill the budget are the common ones: their products are tried out
            from .. import ops
            ops.LIBRARY_TUNE_ROWS.add(budget)
        if cfg.num_pages is not None:
            pools = [cfg.num_pages] * max(1, len(model.cache_groups))
        else:
            # engine.rs:252-262: pool bytes / (bytes of K and V per token * block size), here
            # per group from its own arrays, dtypes and window
            pools = pool_pages(model.cache_groups, model.act_dtype, cfg.block_size,
                               int(cfg.kv_cache_gb * (1 << 30)), cfg.max_num_seqs, budget,
                               min(cfg.max_seq_len, model.max_positions)) or [2]
        num_pages = min(pools)
        if num_pages < 2:
            raise ValueError(f"the cache pool holds {num_pages} pages; at least 2 are needed")
        watermark = cfg.watermark_pages
        if watermark is None:
            watermark = max(1, num_pages // 100)            # engine.rs:263-271
        self.runner = ModelRunner(model, num_pages=pools, page_size=cfg.block_size,
                                  max_num_seqs=cfg.max_num_seqs,
                                  max_batched_tokens=max(cfg.max_batched_tokens, cfg.max_num_seqs),
                                  use_graphs=cfg.use_graphs)
        self.scheduler = Scheduler(self.runner.cache, cfg.max_num_seqs,
                                   max(cfg.max_batched_tokens, cfg.max_num_seqs),
                                   watermark_pages=watermark, policy=cfg.scheduler)
        # engine.rs:280: the longest request is bounded by the rope table and by the pool
        self.max_seq_len = min(model.max_positions, self.scheduler.max_seq_tokens)
        if eos_token_ids is None:
            # what the folder's generation_config.json or config.json named (load_model), else
            # what the typed configuration carries (a model built in memory)
            eos_token_ids = getattr(model, "eos_token_ids", None)
            if eos_token_ids is None:
                eos_token_ids = getattr(getattr(model, "config", None), "eos_token_ids", ())
        self.eos_token_ids = set(int(t) for t in eos_token_ids)
        self._seqs: Dict[int, _Sequence] = {}
        self._finished: Dict[int, Completion] = {}
        self._flight: Optional[_Flight] = None
        self._next_id = 0
        self.stats_ = EngineStats(pages_total=pools[0])

    # ----------------------------------------------------------------- requests
    def add_request(self, prompt_ids: Sequence[int], params: Optional[SamplingParams] = None
                    ) -> int:
        """Queue a request; refuses what could never run (engine.rs:332-356)."""
        params = params or SamplingParams()
        params.validate()
        if len(prompt_ids) == 0 or params.max_tokens == 0:
            raise ValueError("empty prompt or max_tokens of 0")
        total = len(prompt_ids) + params.max_tokens
        if total > self.max_seq_len:
            raise ValueError(f"{total} tokens exceeds max_seq_len {self.max_seq_len}")
        vocab = self.model.spec.vocab_size
        for t in prompt_ids:
            if not 0 <= int(t) < vocab:
                raise ValueError(f"token id {t} is outside the vocabulary of {vocab}")
        seq_id = self._next_id
        self._next_id += 1
        self._seqs[seq_id] = _Sequence(seq_id, prompt_ids, params)
        self.scheduler.add(seq_id, len(prompt_ids))
        return seq_id

    def cancel(self, seq_id: int) -> None:
        """Drop a request wherever it is; its pages are free at once (engine.rs:562-573)."""
        if seq_id in self._seqs:
            self.scheduler.remove(seq_id)
            del self._seqs[seq_id]

    def has_work(self) -> bool:
        return self.scheduler.has_work()

    def warm_up(self) -> int:
        """Capture the decode steps of every batch size and context that this engine can see
        (they are captured at first use otherwise, some tens of milliseconds each, inside the
        step that needs them); returns how many were captured.  The reference has no such
        call: it has no captured steps."""
        return self.runner.capture_decode_steps(self.max_seq_len)

    # --------------------------------------------------------------------- step
    def step(self) -> List[Tuple[int, Optional[int], bool]]:
        """One scheduled batch.  Returns ``(request id, token or None, finished)`` for every
        request that produced a token (``None`` with ``finished``: it stopped at an EOS).
        If the model step raises, the requests of that batch finish with reason ``error``
        and the exception goes on to the caller; requests outside the batch are untouched.

        Decoding runs one step ahead where it can: when every request of a step brings one
        token and will bring one more whatever it samples (no request can be admitted, none
        reaches its ``max_tokens``, pages are at hand), the next step is launched on the
        tokens as they lie on the device before the host has seen them, and this call returns
        the tokens of the step before.  A request that stops at an EOS meanwhile has computed
        one position in vain; its row of the step in flight is dropped."""
        while True:
            if self._flight is None:
                out = self._start_step()
                if self._flight is None:
                    return out
            flight, self._flight = self._flight, None
            ahead = self._launch_ahead(flight) if self.config.launch_ahead else None
            out = self._take(flight)
            self._flight = ahead
            if out or not self.scheduler.has_work():
                return out
            # every request of that step had gone already: on to the next one

    def _start_step(self) -> List[Tuple[int, Optional[int], bool]]:
        """Schedule a batch and run it.  A step of single tokens that the device samples is
        only launched (``self._flight`` holds it then); any other is finished here."""
        sched = self.scheduler.schedule()
        self.stats_.preemptions = self.scheduler.num_preemptions
        if not sched.seqs:
            if self.scheduler.has_work():
                # engine.rs:516-522: a schedule without sequences while work exists is a bug
                for seq_id in list(self._seqs):
                    self.cancel(seq_id)
                raise RuntimeError("scheduler made no progress")
            return []
        # A step in which every request brings one token and the device kernel can sample for
        # all of them runs as one captured graph, sampling included; the book-keeping goes on
        # while it runs, and only then are the tokens waited for.
        wait = None
        singles = self._single_tokens(sched)
        try:
            self.runner.apply_copies(sched.copies)
            if singles is not None:
                wait = self.runner.step_sampled(*singles)
            if wait is None:
                # (single tokens lead the step, the longest contexts first, as above)
                in_order = sorted(sched.seqs, key=lambda t: (t[2] - t[1] != 1, -t[2]))
                entries, final = [], []
                for seq_id, start, end in in_order:
                    seq = self._seqs[seq_id]
                    last = end == len(seq.tokens)
                    entries.append(StepEntry(seq_id, seq.tokens[start:end],
                                             [end - start - 1] if last else []))
                    final.append(last)
                logits = self.runner.step(entries, keep=False)    # sampled from at once
        except Exception as exc:
            # engine.rs:523-528: a failed step fails its own requests and no others; their
            # pages are free again and the engine goes on with the rest.
            self._fail([seq_id for seq_id, _, _ in sched.seqs], exc)
            raise
        self.stats_.steps += 1
        if wait is not None:
            for seq_id, start, end in sched.seqs:
                self.scheduler.advance(seq_id, end)
                # (a prompt's last token, or a recomputed one, may come alone)
                self.stats_.prefill_tokens += max(0, min(end, self._seqs[seq_id].prompt_len) - start)
            self._flight = _Flight(singles[0], wait, side=0)
            return []
        # Rows that yield a token, split between the device kernel and the host sampler.
        device_rows, device_modes, host_rows = [], [], []
        row = 0
        for (seq_id, start, end), last in zip(in_order, final):
            self.scheduler.advance(seq_id, end)
            seq = self._seqs[seq_id]
            # prompt tokens of this portion (recomputed ones after a preemption count again)
            self.stats_.prefill_tokens += max(0, min(end, seq.prompt_len) - start)
            if not last:
                continue
            mode = seq.sampler.device_mode(len(seq.tokens))
            if mode is not None:
                device_rows.append((row, seq_id))
                device_modes.append(mode)
            else:
                host_rows.append((row, seq_id))
            row += 1
        picked: Dict[int, int] = {}
        if device_rows:
            idx = [r for r, _ in device_rows]
            sub = logits if len(idx) == logits.shape[0] else logits[
                torch.tensor(idx, device=logits.device)].contiguous()
            for (_, seq_id), tok in zip(device_rows, sample_on_device(sub, device_modes)):
                picked[seq_id] = tok
        if host_rows:
            idx = torch.tensor([r for r, _ in host_rows], device=logits.device)
            host_logits = logits[idx].cpu().numpy()
            for (_, seq_id), lrow in zip(host_rows, host_logits):
                seq = self._seqs[seq_id]
                picked[seq_id] = seq.sampler.sample(lrow, seq.tokens, len(seq.tokens))
        out, grown = [], []
        now = time.perf_counter()
        for (seq_id, _, _), last in zip(in_order, final):
            if last:
                out.append(self._accept(self._seqs[seq_id], picked[seq_id], now, grown))
        self.scheduler.append_tokens(grown)
        self._note_stats()
        return out

    def _launch_ahead(self, flight: _Flight) -> Optional[_Flight]:
        """Launch the step that follows ``flight`` before its tokens are known, if that step
        is the same requests with one more token each whatever the tokens are; else None, and
        nothing has changed."""
        ids, seqs = flight.ids, self._seqs
        sch = self.scheduler
        if sch.num_running != len(ids):
            return None
        if sch.num_waiting and len(ids) < self.config.max_num_seqs \
                and self.config.scheduler != "static":
            return None                      # the next step may admit a request
        modes = []
        for seq_id in ids:
            seq = seqs.get(seq_id)
            # gone (stopped or cancelled while in flight), or the token in flight is its last
            if seq is None or seq.output_len + 1 >= seq.params.max_tokens:
                return None
            mode = seq.sampler.device_mode(len(seq.tokens) + 1)
            if mode is None:
                return None
            modes.append(mode)
        cache = self.runner.cache
        if any(cache.num_free_pages(g) < len(ids) for g in range(cache.num_groups)):
            return None                      # the scheduler might have to preempt
        sch.append_tokens(ids)
        flight.appended = True
        sched = sch.schedule()
        if sched.copies or sched.preempted or sorted(s for s, _, _ in sched.seqs) != sorted(ids) \
                or any(end - start != 1 for _, start, end in sched.seqs):
            raise RuntimeError("the schedule of a step launched ahead is not the step before "
                               "it with one more token each")
        try:
            wait = self.runner.step_chained(ids, modes, 1 - flight.side)
        except Exception as exc:
            self._fail(ids, exc)
            raise
        self.stats_.steps += 1
        for seq_id, _, end in sched.seqs:
            sch.advance(seq_id, end)
        return _Flight(ids, wait, side=1 - flight.side)

    def _take(self, flight: _Flight) -> List[Tuple[int, Optional[int], bool]]:
        """Wait for a launched step and take its tokens; rows of requests that have gone
        meanwhile are dropped."""
        try:
            tokens = flight.wait()
        except Exception as exc:
            self._fail(flight.ids, exc)
            raise
        out, grown = [], []
        now = time.perf_counter()
        for seq_id, token in zip(flight.ids, tokens):
            seq = self._seqs.get(seq_id)
            if seq is not None:
                out.append(self._accept(seq, token, now, grown))
        if not flight.appended:
            self.scheduler.append_tokens(grown)
        self._note_stats()
        return out

    def _fail(self, seq_ids: Sequence[int], exc: Exception) -> None:
        for seq_id in seq_ids:
            seq = self._seqs.get(seq_id)
            if seq is not None:
                self._finish(seq, "error", error=f"{type(exc).__name__}: {exc}")

    def _note_stats(self) -> None:
        self.stats_.running = self.scheduler.num_running
        self.stats_.waiting = self.scheduler.num_waiting
        self.stats_.pages_used = self.stats_.pages_total - self.runner.cache.num_free_pages(0)

    def _single_tokens(self, sched) -> Optional[Tuple[List[int], List[int], List[Tuple[int, float]]]]:
        """(request ids, their tokens, their (key, 1/T)) when every request of the schedule brings
        its last known token alone and the device kernel can sample for it; else None.  The
        longest contexts come first: the attention kernel's workgroups start in the batch's
        order, and the long walks should not be the last to start.  (A row does not depend on
        its place in the batch, and the order holds while the same requests go on decoding.)"""
        rows = []
        seqs = self._seqs
        for seq_id, start, end in sched.seqs:
            seq = seqs[seq_id]
            if end - start != 1 or end != len(seq.tokens):
                return None
            mode = seq.sampler.device_mode(end)
            if mode is None:
                return None
            rows.append((-end, len(rows), seq_id, seq.tokens[start], mode))
        rows.sort()
        return [r[2] for r in rows], [r[3] for r in rows], [r[4] for r in rows]

    def _accept(self, seq: _Sequence, token: int, now: float, grown: List[int]
                ) -> Tuple[int, Optional[int], bool]:
        """Take a request's sampled token at time ``now``; a request that goes on is added to
        ``grown`` (the scheduler hears of those in one call)."""
        if seq.first_token_at is None:
            seq.first_token_at = now
        seq.last_token_at = now
        stops = (not seq.params.ignore_eos and token in self.eos_token_ids) \
            or token in seq.params.stop_token_ids
        if stops:
            self._finish(seq, "stop")
            return (seq.id, None, True)
        seq.tokens.append(token)
        self.stats_.generated_tokens += 1
        if seq.output_len >= seq.params.max_tokens:
            self._finish(seq, "length")
            return (seq.id, token, True)
        grown.append(seq.id)
        return (seq.id, token, False)

    def _finish(self, seq: _Sequence, reason: str, error: Optional[str] = None) -> None:
        seq.finish_reason = reason
        self.scheduler.remove(seq.id)
        del self._seqs[seq.id]
        self._finished[seq.id] = Completion(
            request_id=seq.id, token_ids=seq.tokens[seq.prompt_len:], finish_reason=reason,
            prompt_tokens=seq.prompt_len, ttft=(seq.first_token_at or seq.arrived) - seq.arrived,
            decode_time=(seq.last_token_at or 0.0) - (seq.first_token_at or 0.0), error=error)

    # ----------------------------------------------------------------- generate
    def generate(self, prompts: Sequence[Sequence[int]],
                 params: Union[SamplingParams, Sequence[SamplingParams], None] = None
                 ) -> List[Completion]:
        """Run the prompts to completion under continuous batching; results in their order."""
        if params is None or isinstance(params, SamplingParams):
            params = [params or SamplingParams()] * len(prompts)
        if len(params) != len(prompts):
            raise ValueError("one SamplingParams per prompt, or one for all")
        ids = [self.add_request(p, sp) for p, sp in zip(prompts, params)]
        while any(i in self._seqs for i in ids):
            self.step()
        return [self._finished.pop(i) for i in ids]

    def pop_finished(self, seq_id: int) -> Optional[Completion]:
        return self._finished.pop(seq_id, None)

    def stats(self) -> EngineStats:
        return self.stats_
