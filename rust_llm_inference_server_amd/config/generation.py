"""What a model folder says about generation beside the architecture's own configuration.

The end-of-sequence ids come from ``generation_config.json`` when it names them and from
``config.json`` otherwise; either may hold one id or a list (crates/engine/src/tokenizer.rs:
64-85).  Instruct checkpoints of Llama 3 keep their end-of-turn id in the first file only."""
from __future__ import annotations

import json
import os
from typing import Tuple

from .errors import ConfigError


def read_eos_token_ids(folder: str) -> Tuple[int, ...]:
    """The folder's end-of-sequence ids: the first of ``generation_config.json`` and
    ``config.json`` that exists and holds ``eos_token_id`` as a number or a list decides (a
    file without the key, or with another kind of value there, is passed over, as the reference
    does); ``()`` when neither names any (the reference refuses such a folder; folders of random
    weights are like that, and their requests end by length)."""
    for name in ("generation_config.json", "config.json"):
        path = os.path.join(folder, name)
        try:
            with open(path, "r", encoding="utf-8") as f:
                d = json.load(f)
        except FileNotFoundError:
            continue
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path}: not valid JSON ({e})") from None
        eos = d.get("eos_token_id") if isinstance(d, dict) else None
        if isinstance(eos, bool):
            continue
        if isinstance(eos, int):
            return (eos,)
        if isinstance(eos, list):
            return tuple(int(e) for e in eos if isinstance(e, int) and not isinstance(e, bool)
                         and e >= 0)
    return ()
