"""Safetensors reading and writing, the checked loader and seeded random weights."""
import json
import os
import struct

import pytest
import torch

from conftest import TINY_A, TINY_B, make_model_folder
from rust_llm_inference_server_amd.registry import architecture_of
from rust_llm_inference_server_amd.weights import (SafetensorsError, WeightError, load_weights,
                                                   open_folder, random_weights, save_file)

CPU = torch.device("cpu")


def specs_of(cfg):
    arch = architecture_of(cfg)
    return arch.build_spec(arch.parse_config(cfg))


def test_round_trip_against_the_safetensors_package(tmp_path):
    from safetensors import safe_open
    from safetensors.torch import save_file as their_save
    tensors = {"a": torch.randn(3, 5), "b": torch.randn(7).to(torch.bfloat16),
               "c": torch.arange(6, dtype=torch.int64).reshape(2, 3), "d": torch.randn(2, 2).half()}
    save_file(tensors, str(tmp_path / "ours.safetensors"), metadata={"k": "v"})
    with safe_open(str(tmp_path / "ours.safetensors"), framework="pt") as f:      # they read ours
        assert f.metadata() == {"k": "v"}
        for k, t in tensors.items():
            assert torch.equal(f.get_tensor(k), t)
    their_save(tensors, str(tmp_path / "theirs.safetensors"))                       # we read theirs
    (tmp_path / "ours.safetensors").unlink()
    (f,) = open_folder(str(tmp_path))
    for k, t in tensors.items():
        assert torch.equal(f.tensor(k), t) and f.info(k) == (t.dtype, tuple(t.shape))


def test_names_follow_the_hugging_face_layout():
    names = [s.name for s in specs_of(TINY_B).tensor_specs()]
    assert names[0] == "model.embed_tokens.weight" and names[-1] == "lm_head.weight"
    assert "model.layers.2.self_attn.k_proj.weight" in names
    assert "model.layers.0.post_attention_layernorm.weight" in names
    assert "model.layers.1.mlp.down_proj.weight" in names and "model.norm.weight" in names
    assert len(names) == 1 + 3 * 9 + 1 + 1
    tied = [s.name for s in specs_of(TINY_A).tensor_specs()]
    assert "lm_head.weight" not in tied                  # crates/model/src/llama.rs:152-156


def test_loader_dtype_policy(tmp_path):
    spec = specs_of(TINY_A)
    folder = make_model_folder(tmp_path / "f32", TINY_A, 0, torch.float32)
    w = load_weights(folder, spec.tensor_specs(), torch.bfloat16, CPU)
    assert all(t.dtype == torch.float32 for t in w.values())     # stored in 32 bits: stays so
    folder = make_model_folder(tmp_path / "bf16", TINY_A, 0, torch.bfloat16)
    w = load_weights(folder, spec.tensor_specs(), torch.bfloat16, CPU)
    assert all(t.dtype == torch.bfloat16 for t in w.values())
    w = load_weights(folder, spec.tensor_specs(), torch.float32, CPU)
    assert all(t.dtype == torch.float32 for t in w.values())     # a float32 run is float32 throughout


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    spec = specs_of(TINY_A)
    w = random_weights(spec.tensor_specs(), 0, torch.float32)
    del w["model.layers.1.mlp.up_proj.weight"]
    del w["model.norm.weight"]
    w["model.layers.0.self_attn.q_proj.weight"] = torch.zeros(64, 32)
    w["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)      # ignored buffer
    w["model.layers.9.extra.weight"] = torch.zeros(3)
    w["lm_head.weight"] = torch.zeros(256, 64)       # stored beside tied embeddings: tolerated
    os.makedirs(tmp_path / "m")
    save_file(w, str(tmp_path / "m" / "model.safetensors"))
    with pytest.raises(WeightError) as e:
        load_weights(str(tmp_path / "m"), spec.tensor_specs(), torch.float32, CPU,
                     spec.optional_tensors)
    err = e.value
    assert err.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.9.extra.weight"]
    assert len(err.wrong_shape) == 1 and "expected shape [64, 64], checkpoint has [64, 32]" in err.wrong_shape[0]
    text = str(err)
    for needle in ("missing tensors (2)", "unexpected tensors (1)", "wrong shapes (1)",
                   "model.norm.weight", "model.layers.9.extra.weight", "q_proj.weight"):
        assert needle in text


def test_broken_files(tmp_path):
    with pytest.raises(SafetensorsError, match="no .safetensors files"):        # llama.rs:131-135
        open_folder(str(tmp_path))
    p = tmp_path / "model.safetensors"
    save_file({"a": torch.randn(4, 4)}, str(p))
    data = p.read_bytes()
    p.write_bytes(data[:-8])
    with pytest.raises(SafetensorsError, match="truncated or corrupt"):
        open_folder(str(tmp_path))
    p.write_bytes(struct.pack("<Q", 1 << 40) + b"{}")
    with pytest.raises(SafetensorsError, match="header length"):
        open_folder(str(tmp_path))
    hdr = json.dumps({"a": {"dtype": "F8_E4M3", "shape": [1], "data_offsets": [0, 1]}}).encode()
    p.write_bytes(struct.pack("<Q", len(hdr)) + hdr + b"\0")
    with pytest.raises(SafetensorsError, match="unknown dtype"):
        open_folder(str(tmp_path))


def test_random_weights_are_seeded_and_have_the_stated_distributions():
    spec = specs_of(TINY_B)
    a = random_weights(spec.tensor_specs(), 5, torch.float32)
    b = random_weights(spec.tensor_specs(), 5, torch.float32)
    c = random_weights(spec.tensor_specs(), 6, torch.float32)
    assert all(torch.equal(a[k], b[k]) for k in a)
    assert not torch.equal(a["model.embed_tokens.weight"], c["model.embed_tokens.weight"])
    e = a["model.embed_tokens.weight"]
    assert abs(e.mean().item()) < 1e-3 and abs(e.std().item() - 0.02) < 1e-3
    n = a["model.layers.0.input_layernorm.weight"]
    assert abs(n.mean().item() - 1.0) < 0.01 and 0.01 < n.std().item() < 0.03
    # a tensor's values do not depend on which other tensors exist
    fewer = random_weights(spec.tensor_specs()[:3], 5, torch.float32)
    assert torch.equal(fewer["model.embed_tokens.weight"], e)
    # bf16 weights are the float32 ones rounded
    h = random_weights(spec.tensor_specs(), 5, torch.bfloat16)
    assert torch.equal(h["lm_head.weight"], a["lm_head.weight"].to(torch.bfloat16))


def test_random_values_are_a_function_of_seed_tensor_and_element():
    """The generator written out a second time, in plain Python integers and ``math``: value i
    of tensor t under seed s is Box-Muller of two splitmix64 hashes of (s, t, i // 2).  The
    native code must give the same float32 values (to the last bit, give or take a library's
    last digit of log and cos in double precision: one float32 step at most, and next to never),
    on one thread as on many."""
    import math
    from rust_llm_inference_server_amd.weights.random_init import normal_fill
    mask = (1 << 64) - 1

    def mix(x):
        x = (x + 0x9E3779B97F4A7C15) & mask
        x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & mask
        x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & mask
        return x ^ (x >> 31)

    def twin(n, seed, tensor, mean, std):
        key = mix(seed ^ mix(tensor))
        out = []
        for j in range((n + 1) // 2):
            u1 = ((mix((key + 2 * j) & mask) >> 11) + 0.5) / 2.0 ** 53
            u2 = ((mix((key + 2 * j + 1) & mask) >> 11) + 0.5) / 2.0 ** 53
            r = math.sqrt(-2.0 * math.log(u1))
            out += [mean + std * (r * math.cos(2 * math.pi * u2)),
                    mean + std * (r * math.sin(2 * math.pi * u2))]
        return torch.tensor(out[:n], dtype=torch.float64).to(torch.float32)

    for n, seed, tensor, mean, std in ((1, 0, 0, 0.0, 0.02), (7, 5, 3, 1.0, 0.02), (4001, 2 ** 63 + 9, 146, 0.0, 1.0)):
        got = normal_fill(n, seed, tensor, mean, std, threads=1)
        want = twin(n, seed, tensor, mean, std)
        step = torch.maximum(want.abs(), torch.tensor(1e-30)) * 2.0 ** -23
        assert ((got - want).abs() <= step).all()
        assert (got != want).sum().item() <= 1
    # any number of threads, the same bits; a long tensor is cut among them
    big = normal_fill(300001, 7, 2, 0.0, 0.02, threads=1)
    for threads in (2, 3, 16, 0):
        assert torch.equal(normal_fill(300001, 7, 2, 0.0, 0.02, threads=threads), big)
    assert abs(big.mean().item()) < 2e-4 and abs(big.std().item() - 0.02) < 2e-4
    # a prefix of a tensor is the tensor's beginning; another tensor index, other values
    assert torch.equal(normal_fill(1000, 7, 2, 0.0, 0.02), big[:1000])
    assert not torch.equal(normal_fill(1000, 7, 3, 0.0, 0.02), big[:1000])
    # the normal's tails are there and nothing is off the scale
    z = big / 0.02
    assert 3.5 < z.abs().max().item() < 6.5 and abs((z.abs() < 1).float().mean().item() - 0.6827) < 0.005


def test_written_folder_loads_back(tmp_path):
    folder = make_model_folder(tmp_path / "m", TINY_B, 3)
    assert sorted(os.listdir(folder)) == ["config.json", "model.safetensors"]
    spec = specs_of(TINY_B)
    w = load_weights(folder, spec.tensor_specs(), torch.float32, CPU)
    want = random_weights(spec.tensor_specs(), 3, torch.float32)
    assert all(torch.equal(w[k], want[k]) for k in want)
    assert json.load(open(os.path.join(folder, "config.json")))["hidden_size"] == 192
