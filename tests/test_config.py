"""Configuration parsing and the architecture registry."""
import json

import pytest

from conftest import TINY_A, TINY_B
from rust_llm_inference_server_amd.config import (ConfigError, LlamaConfig, preset_dict,
                                                  preset_names)
from rust_llm_inference_server_amd.registry import (architecture, architecture_names,
                                                    architecture_of)


def test_presets_parse_and_cover_the_benchmark_shapes():
    assert preset_names() == ["llama-3.1-8b", "llama-3.2-1b", "llama-3.2-3b", "tiny-a", "tiny-b"]
    c = LlamaConfig.from_dict(preset_dict("llama-3.2-1b"))
    assert (c.hidden_size, c.num_hidden_layers, c.num_attention_heads, c.num_key_value_heads,
            c.head_dim, c.intermediate_size, c.vocab_size) == (2048, 16, 32, 8, 64, 8192, 128256)
    assert c.tie_word_embeddings and c.rope_scaling.factor == 32.0
    # 32 KiB of K and V per token in bf16 (crates/model/src/config.rs:49-52)
    assert c.kv_bytes_per_token(2) == 32 * 1024
    c8 = LlamaConfig.from_dict(preset_dict("llama-3.1-8b"))
    assert not c8.tie_word_embeddings and c8.kv_bytes_per_token(2) == 128 * 1024
    for name in preset_names():
        LlamaConfig.from_dict(preset_dict(name))


def test_round_trip_through_config_json(tmp_path):
    for cfg in (TINY_A, TINY_B):
        c = LlamaConfig.from_dict(cfg)
        (tmp_path / "config.json").write_text(json.dumps(c.to_dict()))
        assert LlamaConfig.from_json_file(str(tmp_path)) == c


def test_head_dim_defaults_to_hidden_over_heads():
    d = dict(TINY_A)
    del d["head_dim"]
    assert LlamaConfig.from_dict(d).head_dim == 64 // 4      # config.rs:44-47
    d["head_dim"] = 32                                        # need not equal hidden / heads
    assert LlamaConfig.from_dict(d).head_dim == 32


def test_defaults_of_optional_keys():
    d = {k: v for k, v in TINY_A.items() if k not in ("tie_word_embeddings", "rope_scaling")}
    c = LlamaConfig.from_dict(d)
    assert c.tie_word_embeddings is False and c.rope_scaling is None   # config.rs:16-21
    assert c.group_size == 4


@pytest.mark.parametrize("key", ["hidden_size", "intermediate_size", "num_hidden_layers",
                                 "num_attention_heads", "vocab_size", "rms_norm_eps", "rope_theta",
                                 "max_position_embeddings"])
def test_missing_required_key_is_named(key):
    d = dict(TINY_B)
    del d[key]
    with pytest.raises(ConfigError, match=key):
        LlamaConfig.from_dict(d)


@pytest.mark.parametrize("patch,needle", [
    ({"num_key_value_heads": 4}, "num_key_value_heads"),           # 6 heads, 4 KV heads
    ({"head_dim": 31}, "head_dim"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"attention_bias": True}, "attention_bias"),
    ({"mlp_bias": True}, "mlp_bias"),
    ({"hidden_size": "192"}, "hidden_size"),
    ({"rope_scaling": {"rope_type": "yarn", "factor": 2.0}}, "rope_type"),
    ({"rope_scaling": {"rope_type": "llama3", "factor": 8.0}}, "low_freq_factor"),
    ({"rope_scaling": {"factor": 8.0}}, "rope_type"),
    ({"vocab_size": 0}, "vocab_size"),
    ({"rope_theta": -1.0}, "rope_theta"),
])
def test_unsupported_values_are_refused_by_name(patch, needle):
    d = dict(TINY_B)
    d.update(patch)
    with pytest.raises(ConfigError, match=needle):
        LlamaConfig.from_dict(d)


def test_rope_scaling_variants():
    d = dict(TINY_B)
    d["rope_scaling"] = {"rope_type": "default"}
    assert LlamaConfig.from_dict(d).rope_scaling is None
    d["rope_scaling"] = dict(TINY_B["rope_scaling"])
    d["rope_scaling"]["type"] = d["rope_scaling"].pop("rope_type")     # the older key
    assert LlamaConfig.from_dict(d).rope_scaling.rope_type == "llama3"


def test_eos_ids_number_or_list():
    d = dict(TINY_A)
    d["eos_token_id"] = 7
    assert LlamaConfig.from_dict(d).eos_token_ids == (7,)
    d["eos_token_id"] = [7, 9]
    assert LlamaConfig.from_dict(d).eos_token_ids == (7, 9)


def test_eos_ids_come_from_generation_config_first(tmp_path):
    """crates/engine/src/tokenizer.rs:64-85: ``generation_config.json`` decides when it holds
    ``eos_token_id`` as a number or a list, else ``config.json`` does; a file without the key
    (or with something else there) is passed over.  ``load_model`` hands the ids to the engine."""
    import json
    from rust_llm_inference_server_amd.config import read_eos_token_ids
    folder = tmp_path / "m"
    folder.mkdir()
    assert read_eos_token_ids(str(folder)) == ()
    (folder / "config.json").write_text(json.dumps(dict(TINY_A, eos_token_id=7)))
    assert read_eos_token_ids(str(folder)) == (7,)
    (folder / "generation_config.json").write_text(json.dumps({"temperature": 0.6}))
    assert read_eos_token_ids(str(folder)) == (7,)                   # no key there: passed over
    (folder / "generation_config.json").write_text(json.dumps({"eos_token_id": "</s>"}))
    assert read_eos_token_ids(str(folder)) == (7,)                   # not a number or a list
    (folder / "generation_config.json").write_text(json.dumps({"eos_token_id": [9, 11, 13]}))
    assert read_eos_token_ids(str(folder)) == (9, 11, 13)            # the instruct models' case
    (folder / "generation_config.json").write_text(json.dumps({"eos_token_id": 5}))
    assert read_eos_token_ids(str(folder)) == (5,)
    (folder / "generation_config.json").write_text("{broken")
    with pytest.raises(ConfigError, match="generation_config.json: not valid JSON"):
        read_eos_token_ids(str(folder))


def test_registry_names_the_model_by_its_architecture():
    assert architecture_names() == ["LlamaForCausalLM"]
    arch = architecture_of(TINY_A)
    spec = arch.build_spec(arch.parse_config(TINY_A))
    assert len(spec.layers) == 2 and spec.vocab_size == 256
    with pytest.raises(ConfigError, match="MistralForCausalLM.*known: LlamaForCausalLM"):
        architecture("MistralForCausalLM")
    with pytest.raises(ConfigError, match="architectures"):
        architecture_of({"hidden_size": 4})


def test_bad_files(tmp_path):
    with pytest.raises(ConfigError, match="no such file"):
        LlamaConfig.from_json_file(str(tmp_path))
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="not valid JSON"):
        LlamaConfig.from_json_file(str(tmp_path))
