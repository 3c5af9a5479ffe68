"""Picking the next token.

Device path (greedy, temperature-only): one kernel over the float32 logit rows; temperature
rows use Gumbel-max noise keyed by ``row_key(seed, position)``, position being the number of
tokens the sequence holds when drawing, so a draw is reproducible and independent of the
batch (crates/model/src/sampling.rs:1-63; crates/engine/src/sampler.rs:102-113).

Host path (top-k, top-p, repetition penalty), in the reference's order (sampler.rs:60-68,
116-179): repetition penalty, then greedy if temperature is 0, else weights
``exp((l - max) / T)`` in float64, top-k (ties to the lower id), nucleus (smallest descending
prefix whose share reaches top_p, measured against the whole vocabulary, or against the top-k
set when top-k is on), and a draw.  The reference draws from a ChaCha8 stream seeded per
request; here the uniform comes from a counter hash of (seed, position) like the device
path's, so a request recomputed after preemption draws the same tokens.  The stream itself
therefore differs from the reference's: parity with its host draws is unpinned."""
from __future__ import annotations

import os
from typing import List, Optional, Sequence, Tuple

import numpy as np
import torch

from .params import SamplingParams


def lowbias32(x: int) -> int:
    x &= 0xFFFFFFFF
    x ^= x >> 16
    x = (x * 0x7FEB352D) & 0xFFFFFFFF
    x ^= x >> 15
    x = (x * 0x846CA68B) & 0xFFFFFFFF
    x ^= x >> 16
    return x


def row_key(seed: int, position: int) -> int:
    """Noise key for the token drawn at ``position`` of a request seeded with ``seed``."""
    lo, hi = seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF
    return lowbias32(lowbias32(lowbias32(lo) ^ hi) ^ (position & 0xFFFFFFFF))


def random_seed() -> int:
    return int.from_bytes(os.urandom(8), "little")


def argmax(logits: np.ndarray) -> int:
    """Ties go to the lowest index (sampler.rs:237-246)."""
    return int(np.argmax(logits))


def apply_repetition_penalty(logits: np.ndarray, history: Sequence[int], penalty: float) -> None:
    """Each distinct seen token: divided by the penalty if positive, multiplied if not
    (sampler.rs:223-235)."""
    seen = np.unique(np.asarray([t for t in history if 0 <= t < logits.shape[0]], dtype=np.int64))
    vals = logits[seen]
    logits[seen] = np.where(vals > 0, vals / penalty, vals * penalty)


def nucleus(weights: np.ndarray, total: float, top_p: float) -> Optional[int]:
    """Length of the smallest prefix of descending ``weights`` whose share of ``total``
    reaches ``top_p`` (at least one), or None if all fall short (sampler.rs:198-209)."""
    acc = np.cumsum(weights / total)
    hit = np.nonzero(acc >= top_p)[0]
    return int(hit[0]) + 1 if hit.size else None


def draw(weights: np.ndarray, total: float, u: float) -> int:
    """Index drawn with probability proportional to ``weights`` (sampler.rs:211-221)."""
    x = u * total
    acc = np.cumsum(weights)
    idx = int(np.searchsorted(acc, x, side="right"))
    if idx >= weights.shape[0]:
        pos = np.nonzero(weights > 0)[0]
        return int(pos[-1]) if pos.size else 0
    return idx


class Sampler:
    """One request's sampler: its parameters and its resolved seed."""

    def __init__(self, params: SamplingParams):
        params.validate()
        self.params = params
        self.seed = params.seed if params.seed is not None else random_seed()

    def device_mode(self, position: int) -> Optional[Tuple[int, float]]:
        """(key, 1/T) for the device kernel, 1/T == 0 meaning greedy; None: host path."""
        p = self.params
        if not p.is_device_sampleable():
            return None
        if p.is_greedy():
            return (0, 0.0)
        return (row_key(self.seed, position), 1.0 / p.temperature)

    def _uniform(self, position: int) -> float:
        """A uniform in [0, 1) with 53 bits, from two hashed words of (seed, position)."""
        k = row_key(self.seed, position)
        hi, lo = lowbias32(k ^ 0x68E31DA4), lowbias32(k ^ 0xB5297A4D)
        return (((hi << 32) | lo) >> 11) * (1.0 / (1 << 53))

    def sample(self, logits: np.ndarray, history: Sequence[int], position: int) -> int:
        p = self.params
        logits = np.array(logits, dtype=np.float32, copy=True)
        if p.repetition_penalty != 1.0:
            apply_repetition_penalty(logits, history, p.repetition_penalty)
        if p.is_greedy():
            return argmax(logits)
        inv_t = 1.0 / float(p.temperature)
        l64 = logits.astype(np.float64)
        weights = np.exp((l64 - l64.max()) * inv_t)
        vocab = logits.shape[0]
        top_k = 0 if (p.top_k == 0 or p.top_k >= vocab) else p.top_k
        u = self._uniform(position)
        if top_k == 0 and p.top_p >= 1.0:
            return draw(weights, float(weights.sum()), u)
        # Candidates in descending order of logit, ties to the lower id.
        order = np.lexsort((np.arange(vocab), -l64))
        if top_k:
            order = order[:top_k]
        w = weights[order]
        total = float(w.sum()) if top_k else float(weights.sum())
        keep = nucleus(w, total, float(p.top_p)) if p.top_p < 1.0 else len(order)
        if keep is None:
            keep = len(order)
        w = w[:keep]
        return int(order[draw(w, float(w.sum()), u)])


def sample_on_device(logits: torch.Tensor, modes: Sequence[Tuple[int, float]]) -> List[int]:
    """One token per row of ``logits`` with the device kernel; ``modes`` as ``device_mode``."""
    from .. import ops
    # keys (32-bit patterns) and inverse temperatures travel in one buffer, one copy
    both = np.empty((2, len(modes)), dtype=np.uint32)
    both[0] = [k for k, _ in modes]
    both[1] = np.asarray([t for _, t in modes], dtype=np.float32).view(np.uint32)
    host = torch.from_numpy(both.view(np.int32))
    if logits.is_cuda:
        host = host.pin_memory()
    dev = host.to(logits.device, non_blocking=True)
    keys, inv_t = dev[0], dev[1].view(torch.float32)
    return ops.sample_rows(logits, keys, inv_t).tolist()
