"""Per-request sampling settings, with the reference's names, meanings and defaults
(crates/engine/src/sampler.rs:9-58)."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional


@dataclass
class SamplingParams:
    temperature: float = 0.0          # 0 means greedy
    top_p: float = 1.0                # 1.0 disables nucleus filtering
    top_k: int = 0                    # 0 disables top-k filtering
    repetition_penalty: float = 1.0   # 1.0 disables it
    seed: Optional[int] = None        # None: a random seed per request
    max_tokens: int = 16
    stop_token_ids: List[int] = field(default_factory=list)   # token-id form of `stop`
    ignore_eos: bool = False          # keep generating through EOS until max_tokens

    def validate(self) -> None:
        if self.temperature < 0:
            raise ValueError("temperature must be >= 0")
        if not 0 < self.top_p <= 1:
            raise ValueError("top_p must be in (0, 1]")
        if self.top_k < 0:
            raise ValueError("top_k must be >= 0")
        if self.repetition_penalty <= 0:
            raise ValueError("repetition_penalty must be positive")

    @classmethod
    def greedy(cls, max_tokens: int) -> "SamplingParams":
        return cls(max_tokens=max_tokens)

    def is_greedy(self) -> bool:
        return self.temperature < 1e-5                      # sampler.rs:48-50

    def is_device_sampleable(self) -> bool:
        """Greedy or temperature-only: picked on the device without the logits leaving it;
        top-k, top-p and the repetition penalty take the host path (sampler.rs:52-57)."""
        return self.repetition_penalty == 1.0 and (
            self.is_greedy() or (self.top_k == 0 and self.top_p >= 1.0))
