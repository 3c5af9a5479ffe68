"""The dense Llama decoder as a ``ModelSpec``: token embedding, ``num_hidden_layers`` pre-norm
blocks of grouped-query attention with rotary encoding and a SwiGLU feed-forward, final
RMSNorm, tied or untied head.  Tensor names are the Hugging Face ones the reference reads
(crates/model/src/llama.rs:22-30, 142-156; attention.rs:47-51; layers.rs:120-122, 169-175).
``scale = 1 / sqrt(head_dim)`` is fixed by the architecture (attention.rs:147, 210), so it is
derived here, once, from the configuration."""
from __future__ import annotations

import math

from ..config.llama import LlamaConfig
from ..parts.base import PartSpec
from ..registry import Architecture, register_architecture
from .spec import LayerSpec, ModelSpec


def llama_spec(cfg: LlamaConfig) -> ModelSpec:
    H, d = cfg.hidden_size, cfg.head_dim
    position = PartSpec("rope", {
        "rot_dim": d,
        "theta": cfg.rope_theta,
        "scaling": None if cfg.rope_scaling is None else cfg.rope_scaling.to_dict(),
    })
    norm = PartSpec("rmsnorm", {"size": H, "eps": cfg.rms_norm_eps})
    block = PartSpec("prenorm", {
        "mixer": PartSpec("attention", {
            "hidden_size": H, "num_heads": cfg.num_attention_heads,
            "num_kv_heads": cfg.num_key_value_heads, "head_dim": d,
            "scale": 1.0 / math.sqrt(d), "window": None, "position": position,
        }),
        "feed_forward": PartSpec("swiglu", {"hidden_size": H,
                                            "intermediate_size": cfg.intermediate_size}),
        "mixer_norm": norm,
        "ffn_norm": norm,
        "names": {"mixer_norm": "input_layernorm", "mixer": "self_attn",
                  "ffn_norm": "post_attention_layernorm", "feed_forward": "mlp"},
    })
    tied = cfg.tie_word_embeddings
    return ModelSpec(
        hidden_size=H,
        vocab_size=cfg.vocab_size,
        embedding=PartSpec("token", {"vocab_size": cfg.vocab_size, "hidden_size": H}),
        embedding_prefix="model.embed_tokens",
        layers=[LayerSpec(block, f"model.layers.{i}") for i in range(cfg.num_hidden_layers)],
        final_norm=norm,
        final_norm_prefix="model.norm",
        head=PartSpec("linear", {"vocab_size": cfg.vocab_size, "hidden_size": H,
                                 "tied_to": "model.embed_tokens.weight" if tied else None}),
        head_prefix="lm_head",
        optional_tensors=("lm_head.weight",) if tied else (),
    )


register_architecture(Architecture(
    name="LlamaForCausalLM",
    parse_config=LlamaConfig.from_dict,
    build_spec=llama_spec,
    config_to_dict=lambda cfg: cfg.to_dict(),
))
