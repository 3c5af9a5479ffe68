"""Builds and calls the second plain implementation (``plain_llama_host.cpp``, scalar loops on
the host): compiled with g++ into a temporary folder at first use."""
import ctypes
import os
import shutil
import subprocess
import tempfile
from ctypes import POINTER, c_float, c_int

import torch

_LIB = None


class PlainConfig(ctypes.Structure):
    _fields_ = [(n, c_int) for n in ("hidden", "intermediate", "layers", "heads", "kv_heads",
                                     "head_dim", "vocab", "tied")] + \
               [("eps", c_float), ("theta", c_float), ("scaled", c_int)] + \
               [(n, c_float) for n in ("factor", "low_freq_factor", "high_freq_factor",
                                       "original_max_positions")]


class PlainLayer(ctypes.Structure):
    _fields_ = [(n, POINTER(c_float)) for n in ("input_norm", "q", "k", "v", "o", "post_norm",
                                                "gate", "up", "down")]


def available() -> bool:
    return shutil.which("g++") is not None


def library():
    global _LIB
    if _LIB is None:
        src = os.path.join(os.path.dirname(os.path.abspath(__file__)), "plain_llama_host.cpp")
        out = os.path.join(tempfile.mkdtemp(prefix="plain_host_"), "libplain_host.so")
        subprocess.run(["g++", "-O2", "-ffp-contract=off", "-fPIC", "-shared", "-std=c++17", src,
                        "-o", out], check=True)
        _LIB = ctypes.CDLL(out)
        _LIB.plain_host_forward.restype = c_int
    return _LIB


def forward(w, cfg, ids) -> torch.Tensor:
    """Logits ``(len(ids), vocab)`` of one whole sequence from float32 weights by name."""
    keep = {k: v.to(torch.float32).contiguous() for k, v in w.items()}
    ptr = lambda name: ctypes.cast(keep[name].data_ptr(), POINTER(c_float))
    sc = cfg.get("rope_scaling") or None
    scaled = bool(sc) and sc.get("rope_type", sc.get("type")) == "llama3"
    c = PlainConfig(cfg["hidden_size"], cfg["intermediate_size"], cfg["num_hidden_layers"],
                    cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"],
                    cfg["vocab_size"], int(bool(cfg.get("tie_word_embeddings"))),
                    cfg["rms_norm_eps"], cfg["rope_theta"], int(scaled),
                    *((sc["factor"], sc["low_freq_factor"], sc["high_freq_factor"],
                       sc["original_max_position_embeddings"]) if scaled else (1.0, 1.0, 1.0, 1.0)))
    layers = (PlainLayer * cfg["num_hidden_layers"])()
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}"
        layers[i] = PlainLayer(ptr(f"{p}.input_layernorm.weight"), ptr(f"{p}.self_attn.q_proj.weight"),
                               ptr(f"{p}.self_attn.k_proj.weight"), ptr(f"{p}.self_attn.v_proj.weight"),
                               ptr(f"{p}.self_attn.o_proj.weight"),
                               ptr(f"{p}.post_attention_layernorm.weight"),
                               ptr(f"{p}.mlp.gate_proj.weight"), ptr(f"{p}.mlp.up_proj.weight"),
                               ptr(f"{p}.mlp.down_proj.weight"))
    head = None if cfg.get("tie_word_embeddings") else ptr("lm_head.weight")
    tokens = (c_int * len(ids))(*[int(t) for t in ids])
    out = torch.empty((len(ids), cfg["vocab_size"]), dtype=torch.float32)
    rc = library().plain_host_forward(ctypes.byref(c), ptr("model.embed_tokens.weight"), layers,
                                      ptr("model.norm.weight"), head, tokens, len(ids),
                                      ctypes.cast(out.data_ptr(), POINTER(c_float)))
    if rc != 0:
        raise ValueError(f"plain_host_forward refused its arguments (code {rc})")
    return out
