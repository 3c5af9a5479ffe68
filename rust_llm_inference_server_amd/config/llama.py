"""Typed configuration of the dense Llama decoder, read from a Hugging Face ``config.json``.

Every size and every constant the model uses comes from here; nothing in the parts or the
kernels repeats one.  The keys and which of them are required follow the reference's
``LlamaConfig`` (crates/model/src/config.rs:5-36, parsed by ``from_file`` at 39-42):
``head_dim`` falls back to ``hidden_size / num_attention_heads`` (config.rs:44-47),
``tie_word_embeddings`` defaults to false (config.rs:19-20), ``rope_scaling`` is optional and
when present carries all five llama3 fields (config.rs:28-36).

Where the reference silently accepts a configuration it would then compute wrongly, this
parser refuses it with an error that names the key: an unknown ``rope_scaling.rope_type``
(the reference falls through to unscaled frequencies, rope.rs:99-121), an activation other
than SiLU, projection biases, a head count the KV heads do not divide, an odd head size.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import Any, Dict, Optional, Tuple


from .errors import ConfigError  # noqa: E402  (also found here by its older importers)


def _need(d: Dict[str, Any], key: str, typ, where: str = "config.json"):
    if key not in d or d[key] is None:
        raise ConfigError(f"{where}: required key '{key}' is missing")
    return _typed(d[key], key, typ, where)


def _typed(v, key: str, typ, where: str):
    if typ is int:
        if isinstance(v, bool) or not isinstance(v, int):
            if isinstance(v, float) and float(v).is_integer():
                return int(v)
            raise ConfigError(f"{where}: key '{key}' must be an integer, got {v!r}")
        return v
    if typ is float:
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"{where}: key '{key}' must be a number, got {v!r}")
        return float(v)
    if typ is bool:
        if not isinstance(v, bool):
            raise ConfigError(f"{where}: key '{key}' must be true or false, got {v!r}")
        return v
    if typ is str:
        if not isinstance(v, str):
            raise ConfigError(f"{where}: key '{key}' must be a string, got {v!r}")
        return v
    raise AssertionError(typ)


@dataclass(frozen=True)
class RopeScaling:
    """Frequency-dependent RoPE scaling, ``rope_type: "llama3"`` (config.rs:28-36)."""

    rope_type: str
    factor: float
    low_freq_factor: float
    high_freq_factor: float
    original_max_position_embeddings: int

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> Optional["RopeScaling"]:
        where = "config.json rope_scaling"
        if not isinstance(d, dict):
            raise ConfigError(f"{where}: must be an object, got {d!r}")
        # ``type`` is the key older Hugging Face files use for the same field.
        rope_type = d.get("rope_type", d.get("type"))
        if rope_type is None:
            raise ConfigError(f"{where}: required key 'rope_type' is missing")
        rope_type = _typed(rope_type, "rope_type", str, where)
        if rope_type == "default":
            return None
        if rope_type != "llama3":
            raise ConfigError(
                f"{where}: rope_type '{rope_type}' is not supported (known: 'llama3', 'default')"
            )
        out = cls(
            rope_type=rope_type,
            factor=_need(d, "factor", float, where),
            low_freq_factor=_need(d, "low_freq_factor", float, where),
            high_freq_factor=_need(d, "high_freq_factor", float, where),
            original_max_position_embeddings=_need(
                d, "original_max_position_embeddings", int, where
            ),
        )
        if out.factor <= 0:
            raise ConfigError(f"{where}: 'factor' must be positive, got {out.factor}")
        if out.high_freq_factor == out.low_freq_factor:
            raise ConfigError(f"{where}: 'high_freq_factor' must differ from 'low_freq_factor'")
        if out.original_max_position_embeddings <= 0:
            raise ConfigError(f"{where}: 'original_max_position_embeddings' must be positive")
        return out

    def to_dict(self) -> Dict[str, Any]:
        return {
            "rope_type": self.rope_type,
            "factor": self.factor,
            "low_freq_factor": self.low_freq_factor,
            "high_freq_factor": self.high_freq_factor,
            "original_max_position_embeddings": self.original_max_position_embeddings,
        }


@dataclass(frozen=True)
class LlamaConfig:
    """The subset of a Llama ``config.json`` the forward pass needs (config.rs:5-26)."""

    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    vocab_size: int
    rms_norm_eps: float
    rope_theta: float
    max_position_embeddings: int
    rope_scaling: Optional[RopeScaling] = None
    tie_word_embeddings: bool = False
    bos_token_id: Optional[int] = None
    eos_token_ids: Tuple[int, ...] = ()
    architecture: str = "LlamaForCausalLM"
    extra: Dict[str, Any] = field(default_factory=dict, compare=False, hash=False)

    # ------------------------------------------------------------------ parsing
    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "LlamaConfig":
        if not isinstance(d, dict):
            raise ConfigError("config.json: top level must be an object")
        hidden = _need(d, "hidden_size", int)
        heads = _need(d, "num_attention_heads", int)
        if heads <= 0:
            raise ConfigError("config.json: 'num_attention_heads' must be positive")
        # The reference requires num_key_value_heads (config.rs:10); files written by
        # Hugging Face omit it for plain multi-head models, where it equals the head count.
        kv = d.get("num_key_value_heads")
        kv = heads if kv is None else _typed(kv, "num_key_value_heads", int, "config.json")
        head_dim = d.get("head_dim")
        if head_dim is None:
            if hidden % heads:
                raise ConfigError(
                    f"config.json: 'hidden_size' {hidden} is not a multiple of "
                    f"'num_attention_heads' {heads} and no 'head_dim' is given"
                )
            head_dim = hidden // heads
        else:
            head_dim = _typed(head_dim, "head_dim", int, "config.json")
        scaling = d.get("rope_scaling")
        archs = d.get("architectures") or ["LlamaForCausalLM"]
        if not isinstance(archs, list) or not archs or not isinstance(archs[0], str):
            raise ConfigError("config.json: 'architectures' must be a list of names")
        eos = d.get("eos_token_id")
        if eos is None:
            eos_ids: Tuple[int, ...] = ()
        elif isinstance(eos, list):
            eos_ids = tuple(_typed(e, "eos_token_id", int, "config.json") for e in eos)
        else:
            eos_ids = (_typed(eos, "eos_token_id", int, "config.json"),)
        bos = d.get("bos_token_id")
        known = {
            "hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads",
            "num_key_value_heads", "head_dim", "vocab_size", "rms_norm_eps", "rope_theta",
            "max_position_embeddings", "rope_scaling", "tie_word_embeddings", "bos_token_id",
            "eos_token_id", "architectures",
        }
        cfg = cls(
            hidden_size=hidden,
            intermediate_size=_need(d, "intermediate_size", int),
            num_hidden_layers=_need(d, "num_hidden_layers", int),
            num_attention_heads=heads,
            num_key_value_heads=kv,
            head_dim=head_dim,
            vocab_size=_need(d, "vocab_size", int),
            rms_norm_eps=_need(d, "rms_norm_eps", float),
            rope_theta=_need(d, "rope_theta", float),
            max_position_embeddings=_need(d, "max_position_embeddings", int),
            rope_scaling=None if scaling is None else RopeScaling.from_dict(scaling),
            tie_word_embeddings=_typed(d.get("tie_word_embeddings", False),
                                       "tie_word_embeddings", bool, "config.json"),
            bos_token_id=None if bos is None else _typed(bos, "bos_token_id", int, "config.json"),
            eos_token_ids=eos_ids,
            architecture=archs[0],
            extra={k: v for k, v in d.items() if k not in known},
        )
        cfg.validate()
        return cfg

    @classmethod
    def from_json_file(cls, path: str) -> "LlamaConfig":
        if os.path.isdir(path):
            path = os.path.join(path, "config.json")
        try:
            with open(path, "r", encoding="utf-8") as f:
                d = json.load(f)
        except FileNotFoundError:
            raise ConfigError(f"{path}: no such file") from None
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path}: not valid JSON ({e})") from None
        return cls.from_dict(d)

    # --------------------------------------------------------------- validation
    def validate(self) -> None:
        for key in ("hidden_size", "intermediate_size", "num_hidden_layers",
                    "num_attention_heads", "num_key_value_heads", "head_dim", "vocab_size",
                    "max_position_embeddings"):
            if getattr(self, key) <= 0:
                raise ConfigError(f"config.json: '{key}' must be positive, got {getattr(self, key)}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"config.json: 'num_attention_heads' {self.num_attention_heads} is not a multiple "
                f"of 'num_key_value_heads' {self.num_key_value_heads}"
            )
        if self.head_dim % 2:
            raise ConfigError(f"config.json: 'head_dim' {self.head_dim} must be even for rotation")
        if not (self.rms_norm_eps >= 0.0):
            raise ConfigError(f"config.json: 'rms_norm_eps' must be >= 0, got {self.rms_norm_eps}")
        if not (self.rope_theta > 0.0):
            raise ConfigError(f"config.json: 'rope_theta' must be positive, got {self.rope_theta}")
        act = self.extra.get("hidden_act", "silu")
        if act != "silu":
            raise ConfigError(f"config.json: 'hidden_act' '{act}' is not supported (only 'silu')")
        for key in ("attention_bias", "mlp_bias"):
            if self.extra.get(key, False):
                raise ConfigError(f"config.json: '{key}' = true is not supported (no biases)")

    # ------------------------------------------------------------------ derived
    @property
    def group_size(self) -> int:
        return self.num_attention_heads // self.num_key_value_heads

    def kv_bytes_per_token(self, elem_size: int) -> int:
        """Bytes of K plus V per token across all layers (config.rs:49-52)."""
        return 2 * self.num_hidden_layers * self.num_key_value_heads * self.head_dim * elem_size

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {
            "architectures": [self.architecture],
            "model_type": "llama",
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "vocab_size": self.vocab_size,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "rope_scaling": None if self.rope_scaling is None else self.rope_scaling.to_dict(),
            "max_position_embeddings": self.max_position_embeddings,
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_act": "silu",
            "attention_bias": False,
            "mlp_bias": False,
        }
        if self.bos_token_id is not None:
            d["bos_token_id"] = self.bos_token_id
        if self.eos_token_ids:
            d["eos_token_id"] = (self.eos_token_ids[0] if len(self.eos_token_ids) == 1
                                 else list(self.eos_token_ids))
        return d
