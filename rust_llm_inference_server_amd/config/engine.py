"""Engine options, named as the reference names them (crates/engine/src/engine.rs:31-63 and the
``EngineArgs`` of crates/server/src/main.rs:106-127): how many sequences and tokens one step
may hold, the page size and the size of the page pool, and the scheduling policy."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional


@dataclass
class EngineConfig:
    max_num_seqs: int = 64
    max_batched_tokens: int = 2048
    kv_cache_gb: float = 1.0
    block_size: int = 16
    scheduler: str = "continuous"          # or "static"
    max_seq_len: int = 2048
    # Given directly, it overrides kv_cache_gb (tests use pools of a few pages).
    num_pages: Optional[int] = None
    # Free pages kept back at admission so running sequences can grow
    # (engine.rs:263-271: max(1, num_blocks / 100)); None means that rule.
    watermark_pages: Optional[int] = None
    use_graphs: bool = True
    # Decode steps are launched one ahead of the tokens that the host has seen, where the next
    # step does not depend on them (False: every step waits for the one before).
    launch_ahead: bool = True

    def validate(self) -> None:
        if self.max_num_seqs <= 0:
            raise ValueError("max_num_seqs must be positive")
        if self.block_size <= 0:
            raise ValueError("block_size must be positive")
        if self.max_batched_tokens <= 0:
            raise ValueError("max_batched_tokens must be positive")
        # A budget below max_num_seqs is raised to it by the engine, as the reference does
        # (engine.rs:263-271): the scheduler needs one decode token per sequence
        # (scheduler.rs:113-117).
        if self.scheduler not in ("continuous", "static"):
            raise ValueError(f"scheduler must be 'continuous' or 'static', got {self.scheduler!r}")
