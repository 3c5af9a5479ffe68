"""Token agreement between a reduced-precision run and the plain float32 implementation.

The reference's rule (crates/model/tests/parity.rs:17-35, 218-240): float32 must reproduce the
reference's tokens exactly; a 16-bit run may pick another token only where the reference's
top-2 margin is below a frozen threshold that the measured logit noise explains (there: f16
noise up to 0.06 on real weights, threshold 0.02 on the margin).  Here the threshold is fixed
from this engine's own frozen bfloat16 logit gate on the tiny models (2e-2 per logit, measured
worst 6.5e-3): two logits that each move by less than the gate can swap only if they were
less than twice the gate apart.

The reference ends a prompt's comparison at its first near-tie flip.  Here the comparison goes
on: the plain implementation is run on the engine's own tokens (prompt + what it generated), so
every generated token is judged against the float32 scores *for the prefix the engine really
had*, flip or no flip."""
from typing import Sequence

import plain_llama as plain

BF16_LOGIT_GATE = 2e-2
TIE_MARGIN = 2 * BF16_LOGIT_GATE


def margin_for(dtype: str) -> float:
    return 0.0 if dtype in ("float32", "fp32", "f32") else TIE_MARGIN


def near_tie_picks(w, cfg, prompt: Sequence[int], tokens: Sequence[int], margin: float,
                   temperature: float = 0.0, seed: int = 0) -> int:
    """Checks ``tokens`` (generated after ``prompt``, greedy or by seeded temperature
    sampling) against the plain implementation; returns how many of them are not the float32
    winner but within ``margin`` of it.  A token further off fails."""
    if not tokens:
        return 0
    logits = plain.forward(w, cfg, list(prompt) + list(tokens[:-1]))
    inv_t = 0.0 if temperature < 1e-5 else 1.0 / temperature
    picks = 0
    for i, tok in enumerate(tokens):
        position = len(prompt) + i                      # the index of the token being drawn
        scores = plain.sample_scores(logits[position - 1], plain.row_key(seed, position), inv_t)
        best = plain.sample_row(logits[position - 1], plain.row_key(seed, position), inv_t)
        if tok == best:
            continue
        gap = float(scores[best] - scores[tok])
        # the logits' noise is scaled by 1 / T before the (exact) Gumbel noise is added
        allowed = margin * max(1.0, inv_t)
        assert gap < allowed, (f"token {i} after a prompt of {len(prompt)}: got {tok}, the float32 "
                               f"winner is {best}, {gap:.4f} ahead (near-tie margin {allowed:.4f})")
        picks += 1
    return picks
