"""Perplexity of a token stream the way the reference computes it, which is llama.cpp's:
windows of ``ctx`` tokens, the first token of each replaced by BOS, only the second half of
a window scored (crates/engine/src/perplexity.rs:26-80)."""
from __future__ import annotations

import math
import time
from dataclasses import asdict, dataclass
from typing import Callable, Optional, Sequence

import torch

from .batch import StepEntry
from .runner import ModelRunner


@dataclass
class Perplexity:
    ppl: float
    ppl_stderr: float          # one standard error, from the per-token NLL variance
    mean_nll: float
    tokens_scored: int
    windows: int
    ctx: int
    seconds: float

    def to_dict(self) -> dict:
        return asdict(self)


def perplexity(runner: ModelRunner, tokens: Sequence[int], bos: int, ctx: int,
               max_windows: int = 0,
               progress: Optional[Callable[[int, int, float], None]] = None) -> Perplexity:
    if ctx < 4:
        raise ValueError("ctx must be at least 4")
    windows = len(tokens) // ctx
    if max_windows > 0:
        windows = min(windows, max_windows)
    if windows <= 0:
        raise ValueError(f"corpus of {len(tokens)} tokens is shorter than one window of {ctx}")
    first = ctx // 2
    total = total_sq = 0.0
    n = 0
    t0 = time.perf_counter()
    seq_id = -1
    for w in range(windows):
        chunk = [int(t) for t in tokens[w * ctx:(w + 1) * ctx]]
        chunk[0] = int(bos)
        runner.reserve(seq_id, ctx)
        try:
            # Rows first .. ctx-2 predict tokens first+1 .. ctx-1; the last row has no target.
            logits = runner.step([StepEntry(seq_id, chunk, list(range(first, ctx - 1)))],
                                 keep=False)          # scored before the next window runs
        finally:
            runner.free(seq_id)       # also when the step raises: the next call starts clean
        targets = torch.tensor(chunk[first + 1:], device=logits.device).reshape(-1, 1)
        logp = torch.log_softmax(logits.double(), dim=-1).gather(1, targets).reshape(-1)
        nll = (-logp).cpu()
        total += float(nll.sum())
        total_sq += float((nll * nll).sum())
        n += nll.numel()
        if progress:
            progress(w + 1, windows, math.exp(total / n))
    mean = total / n
    var = max(total_sq / n - mean * mean, 0.0)
    ppl = math.exp(mean)
    return Perplexity(ppl=ppl, ppl_stderr=ppl * math.sqrt(var / n), mean_nll=mean,
                      tokens_scored=n, windows=windows, ctx=ctx,
                      seconds=time.perf_counter() - t0)
