import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an AMD GPU (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


# Two tiny configurations that differ in every size and option: layers, width, head counts
# and grouping (one KV head for four query heads vs two for six), head size, feed-forward
# width, vocabulary, rotary base, frequency scaling on/off, norm eps, tied/untied head.
TINY_A = {
    "architectures": ["LlamaForCausalLM"], "hidden_size": 64, "intermediate_size": 128,
    "num_hidden_layers": 2, "num_attention_heads": 4, "num_key_value_heads": 1, "head_dim": 16,
    "vocab_size": 256, "rms_norm_eps": 1e-5, "rope_theta": 10000.0, "rope_scaling": None,
    "max_position_embeddings": 128, "tie_word_embeddings": True,
}
TINY_B = {
    "architectures": ["LlamaForCausalLM"], "hidden_size": 192, "intermediate_size": 320,
    "num_hidden_layers": 3, "num_attention_heads": 6, "num_key_value_heads": 2, "head_dim": 32,
    "vocab_size": 384, "rms_norm_eps": 1e-6, "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                     "high_freq_factor": 4.0, "original_max_position_embeddings": 64},
    "max_position_embeddings": 256, "tie_word_embeddings": False,
}
# Sizes that are no power of two and not multiples of 8: the width, the feed-forward width
# and the vocabulary are odd multiples of small primes, head_dim 48 with 5 query heads of
# their own KV head each (plain multi-head attention), head_dim * heads != hidden.
TINY_C = {
    "architectures": ["LlamaForCausalLM"], "hidden_size": 100, "intermediate_size": 172,
    "num_hidden_layers": 2, "num_attention_heads": 5, "num_key_value_heads": 5, "head_dim": 48,
    "vocab_size": 331, "rms_norm_eps": 1e-5, "rope_theta": 10000.0, "rope_scaling": None,
    "max_position_embeddings": 512, "tie_word_embeddings": False,
}
# Head size 64 (the smallest for which the decode kernel rotates and stores by itself), a width
# that is neither a power of two nor heads * head size, a prime vocabulary, frequency scaling.
TINY_D = {
    "architectures": ["LlamaForCausalLM"], "hidden_size": 136, "intermediate_size": 200,
    "num_hidden_layers": 2, "num_attention_heads": 6, "num_key_value_heads": 2, "head_dim": 64,
    "vocab_size": 523, "rms_norm_eps": 1e-5, "rope_theta": 100000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 4.0, "low_freq_factor": 1.0,
                     "high_freq_factor": 4.0, "original_max_position_embeddings": 32},
    "max_position_embeddings": 256, "tie_word_embeddings": True,
}
TINY = {"a": TINY_A, "b": TINY_B, "c": TINY_C, "d": TINY_D}


def make_model_folder(path, config, seed, dtype=torch.float32):
    from rust_llm_inference_server_amd.registry import architecture_of
    from rust_llm_inference_server_amd.weights import write_model_folder
    arch = architecture_of(config)
    spec = arch.build_spec(arch.parse_config(config))
    write_model_folder(str(path), config, spec.tensor_specs(), seed, dtype)
    return str(path)


@pytest.fixture
def cpu_ops(monkeypatch):
    import cpu_ops as double
    double.install(monkeypatch)
    return double


@pytest.fixture(scope="session")
def tiny_folders(tmp_path_factory):
    """Model folders (float32 weights) for the tiny configurations, by name."""
    out = {}
    for i, (name, cfg) in enumerate(TINY.items()):
        out[name] = make_model_folder(tmp_path_factory.mktemp(f"tiny_{name}"), cfg, seed=i)
    return out


@pytest.fixture(scope="session")
def tiny_folders_bf16(tmp_path_factory):
    """The same models with weights stored in bfloat16: what a bfloat16 engine computes with,
    so that the plain float32 implementation can run on exactly those numbers."""
    out = {}
    for i, (name, cfg) in enumerate(TINY.items()):
        out[name] = make_model_folder(tmp_path_factory.mktemp(f"tiny16_{name}"), cfg, seed=i,
                                      dtype=torch.bfloat16)
    return out
