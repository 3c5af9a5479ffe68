"""Configurations drawn at random within what config.json allows (head sizes in steps of 16, any
number of heads and groups, widths and vocabularies that are no power of two or multiple of
8), each replayed as a mixed trace with page reuse, in float32 and bfloat16, against the plain
implementation.  The point is sizes that no hand-picked configuration happens to have."""
import random

import pytest
import torch

import plain_llama as plain
import traces
from conftest import make_model_folder
from test_replay_gpu import TOL, check, make_runner

pytestmark = pytest.mark.gpu


def draw_config(seed: int) -> dict:
    rng = random.Random(seed)
    head_dim = rng.choice([16, 32, 48, 64, 80, 96, 112, 128])
    kv = rng.choice([1, 2, 3, 4])
    heads = kv * rng.choice([1, 2, 3, 4, 7])
    scaling = None
    if rng.random() < 0.5:
        scaling = {"rope_type": "llama3", "factor": rng.choice([2.0, 8.0, 32.0]),
                   "low_freq_factor": 1.0, "high_freq_factor": rng.choice([2.0, 4.0]),
                   "original_max_position_embeddings": rng.choice([16, 64])}
    return {
        "architectures": ["LlamaForCausalLM"],
        "hidden_size": rng.choice([36, 72, 100, 136, 200, 264, 328]) + rng.choice([0, 2, 4]),
        "intermediate_size": rng.randrange(24, 400),
        "num_hidden_layers": rng.choice([1, 2, 3]),
        "num_attention_heads": heads, "num_key_value_heads": kv, "head_dim": head_dim,
        "vocab_size": rng.randrange(50, 700),
        "rms_norm_eps": rng.choice([1e-5, 1e-6, 1e-3]),
        "rope_theta": rng.choice([10000.0, 500000.0, 1e6]),
        "rope_scaling": scaling,
        "max_position_embeddings": 160,
        "tie_word_embeddings": rng.random() < 0.5,
    }


@pytest.mark.parametrize("seed", range(8))
def test_random_configuration_mixed_trace(seed, tmp_path):
    cfg = draw_config(seed)
    lengths = [3, 40, 17, 70, 1, 130, 9]
    for dtype, tdt in (("float32", torch.float32), ("bfloat16", torch.bfloat16)):
        folder = make_model_folder(tmp_path / dtype, cfg, seed=seed, dtype=tdt)
        w, c = plain.read_weights(folder), plain.read_config(folder)
        reqs = traces.random_requests(cfg["vocab_size"], lengths, seed=seed + 1)
        ref = {k: plain.forward(w, c, t) for k, t in reqs.items()}
        steps, max_tokens = traces.trace_mixed(reqs, seed=seed)
        runner = make_runner(folder, dtype, max_tokens, page_size=16)
        outputs = traces.replay_in_process(runner, steps)
        worst = check(steps, outputs, reqs, ref, cfg["vocab_size"], TOL[dtype])
        print(f"seed {seed} {dtype}: {cfg['hidden_size']}x{cfg['num_attention_heads']}/"
              f"{cfg['num_key_value_heads']}x{cfg['head_dim']} worst |diff| {worst:.3e}")
        assert runner.cache.num_free_pages(0) == runner.cache.num_pages(0)


# Layer sizes of the larger shapes the engine is meant for (Llama-3.2-3B and Llama-3.1-8B), with
# one layer and a small vocabulary so that the plain implementation stays quick: widths of 12
# and 16 k items, a feed-forward width that takes two k slices, head size 128.  The whole
# prompts bring more than 64 rows to the down projection, whose k of 8,192 and 14,336 then goes
# to the library in slices.
LARGE_LAYERS = {
    "3b-layer": dict(hidden_size=3072, intermediate_size=8192, num_attention_heads=24,
                     num_key_value_heads=8, head_dim=128, factor=32.0, tie=True),
    "8b-layer": dict(hidden_size=4096, intermediate_size=14336, num_attention_heads=32,
                     num_key_value_heads=8, head_dim=128, factor=8.0, tie=False),
}


@pytest.mark.parametrize("name", sorted(LARGE_LAYERS))
def test_layer_sizes_of_larger_models(name, tmp_path):
    p = LARGE_LAYERS[name]
    cfg = {
        "architectures": ["LlamaForCausalLM"], "hidden_size": p["hidden_size"],
        "intermediate_size": p["intermediate_size"], "num_hidden_layers": 1,
        "num_attention_heads": p["num_attention_heads"],
        "num_key_value_heads": p["num_key_value_heads"], "head_dim": p["head_dim"],
        "vocab_size": 1000, "rms_norm_eps": 1e-5, "rope_theta": 500000.0,
        "rope_scaling": {"rope_type": "llama3", "factor": p["factor"], "low_freq_factor": 1.0,
                         "high_freq_factor": 4.0, "original_max_position_embeddings": 8192},
        "max_position_embeddings": 128, "tie_word_embeddings": p["tie"],
    }
    folder = make_model_folder(tmp_path / "m", cfg, seed=11, dtype=torch.bfloat16)
    w, c = plain.read_weights(folder), plain.read_config(folder)
    reqs = traces.random_requests(cfg["vocab_size"], [100, 9, 40], seed=5)
    ref = {k: plain.forward(w, c, t) for k, t in reqs.items()}
    spread = max(r.abs().max().item() for r in ref.values())
    from rust_llm_inference_server_amd import ops
    assert ops.library_slices(100, p["intermediate_size"]) > 1
    for dtype in ("float32", "bfloat16"):
        # float32: the reference's absolute gate of 1e-4 as it is (measured 2.1e-5 and 2.9e-5 on
        # logits of up to 5.1 and 6.0).  bfloat16: the tiny models' gate of 2e-2 is for logits of
        # about +-1 and goes with the size of these (measured 0.047 and 0.060, 0.009 and 0.010
        # of the largest logit).
        tol = TOL[dtype] if dtype == "float32" else TOL[dtype] * max(1.0, spread)
        for build in (traces.trace_whole, traces.trace_tail, traces.trace_mixed):
            steps, max_tokens = build(reqs)
            runner = make_runner(folder, dtype, max_tokens, page_size=16)
            outputs = traces.replay_in_process(runner, steps)
            worst = check(steps, outputs, reqs, ref, cfg["vocab_size"], tol)
            print(f"{name} {dtype} {build.__name__}: worst |diff| {worst:.3e}, largest |logit| {spread:.2f}")


def test_whole_llama_1b_shape(tmp_path):
    """All 16 layers of the Llama-3.2-1B shape with random weights: the 32-bit path within the
    reference's gate for its own parity run (1e-4), bfloat16 within a gate that goes with the size
    of these logits, for the tail-decoded and the mixed trace."""
    from rust_llm_inference_server_amd.config import preset_dict
    cfg = preset_dict("llama-3.2-1b")
    cfg["max_position_embeddings"] = 256
    folder = make_model_folder(tmp_path / "m", cfg, seed=0, dtype=torch.bfloat16)
    w, c = plain.read_weights(folder), plain.read_config(folder)
    reqs = traces.random_requests(cfg["vocab_size"], [48, 9, 33], seed=5)
    ref = {k: plain.forward(w, c, t) for k, t in reqs.items()}
    spread = max(r.abs().max().item() for r in ref.values())
    # bfloat16 through 16 layers: measured 0.019 of the largest |logit| (every kernel choice
    # gives the same figure: it is the rounding of the activations); the gate is 0.03 of it.
    for dtype, tol in (("float32", TOL["float32"]), ("bfloat16", 0.03 * max(1.0, spread))):
        for build in (traces.trace_tail, traces.trace_mixed):
            steps, max_tokens = build(reqs)
            runner = make_runner(folder, dtype, max_tokens, page_size=16)
            outputs = traces.replay_in_process(runner, steps)
            worst = check(steps, outputs, reqs, ref, cfg["vocab_size"], tol)
            print(f"1b {dtype} {build.__name__}: worst |diff| {worst:.3e}, largest |logit| {spread:.2f}")
            del runner
            torch.cuda.empty_cache()


@pytest.mark.parametrize("tokens", [2048, 512, 100])
def test_captured_prompt_steps_at_the_1b_layer_sizes(tokens, monkeypatch):
    """Whole prompts of one length, one after the other, at the layer sizes of the 1B shape (two
    layers, a small vocabulary): from the second on (here; later by default) the step is a
    captured HIP graph.  At these
    sizes the products are the library's (at 512 and 100 rows the down projection in slices of
    k, with a norm that adds partial sums) and the attention takes tiles of 64 or 128 queries
    with key runs; every replay, with other tokens on other pages and an eager step of another
    shape in between, must give what the runner without captured steps gives, bit for bit."""
    from rust_llm_inference_server_amd.config import preset_dict
    from rust_llm_inference_server_amd.engine import ModelRunner, StepEntry, random_model
    from rust_llm_inference_server_amd.engine.graph import RepeatedSteps
    monkeypatch.setattr(RepeatedSteps, "CAPTURE_AT", 2)
    cfg = preset_dict("llama-3.2-1b")
    cfg.update(num_hidden_layers=2, vocab_size=1000, max_position_embeddings=4096)
    model = random_model(cfg, seed=3, dtype="bfloat16", max_positions=4096)
    g = torch.Generator().manual_seed(tokens)
    runners = []
    for captures in (False, True):
        r = ModelRunner(model, num_pages=3 * (tokens // 16 + 2) + 2, page_size=16, max_num_seqs=4)
        r.capture_repeated_steps = captures
        runners.append(r)
    for i in range(5):
        prompt = torch.randint(0, 1000, (tokens,), generator=g).tolist()
        other = torch.randint(0, 1000, (7 + i,), generator=g).tolist()
        got = []
        for r in runners:
            r.reserve(10 + i, len(other))                       # an eager step of another shape
            r.step([StepEntry(10 + i, other, [0])])
            r.free(10 + i)
            r.reserve(i, tokens)
            got.append(r.step([StepEntry(i, prompt, [0, tokens // 2, tokens - 1])]))
            torch.cuda.synchronize()
            if i % 2:
                r.free(i)                                        # the next prompt takes these pages
        assert torch.equal(got[0], got[1]), f"prompt {i}"
        assert torch.isfinite(got[0]).all() and got[0].abs().max() > 0
    assert runners[1]._repeated.replays == 4 and runners[0]._repeated is None
