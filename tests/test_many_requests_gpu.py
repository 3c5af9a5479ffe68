"""Steps of 17 to 64 live requests, where a decode step changes its kernels: the products of
up to 16 rows stream the weights with the norm and the SwiGLU inside, 17 to 64 rows take the
kernels for that range, more rows the library; captured steps take the buckets of 32 and 64
requests, and the decode attention deals its partitions out by the size of the batch.  Tokens
through the engine (the reference's engine tests at their largest batch,
crates/engine/tests/engine.rs:58-83, 157-210) and logits through the step function, against
the plain implementation, in float32 and bfloat16, on tiny A (head size 16: vector-unit
attention in both dtypes), tiny D (head size 64: the matrix-core decode kernel with the
rotation inside) and a configuration whose widths the streaming kernels take with 17 to 64
rows as well."""
import pytest
import torch

import near_ties
import plain_llama as plain
import traces
from conftest import TINY, make_model_folder
from rust_llm_inference_server_amd.config import EngineConfig
from rust_llm_inference_server_amd.sampling import SamplingParams

pytestmark = pytest.mark.gpu

TOL = {"float32": 1e-4, "bfloat16": 2e-2}          # the replay tests' gates

# Widths in whole k items of 256 (hidden 256, feed-forward 512), which the streaming kernels take
# with 17 to 64 rows too: the output and down projections then join the residual themselves and
# the products behind the norms scale by the sums they hand over, as with up to 16 rows.
TINY_W = {
    "architectures": ["LlamaForCausalLM"], "hidden_size": 256, "intermediate_size": 512,
    "num_hidden_layers": 2, "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 64,
    "vocab_size": 300, "rms_norm_eps": 1e-5, "rope_theta": 10000.0, "rope_scaling": None,
    "max_position_embeddings": 128, "tie_word_embeddings": False,
}
CONFIGS = dict(TINY, w=TINY_W)


@pytest.fixture(scope="module", params=["a", "d", "w"])
def case(request, tmp_path_factory):
    name = request.param
    out = {}
    for dtype, tdt in (("float32", torch.float32), ("bfloat16", torch.bfloat16)):
        folder = make_model_folder(tmp_path_factory.mktemp(f"many_{name}_{dtype}"), CONFIGS[name],
                                   seed=13, dtype=tdt)
        out[dtype] = (folder, plain.read_weights(folder), plain.read_config(folder))
    return name, CONFIGS[name], out


def load(folder, dtype, max_positions):
    from rust_llm_inference_server_amd.engine import load_model
    return load_model(folder, dtype, max_positions)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("launch_ahead", [True, False])
def test_forty_requests_through_the_engine(case, dtype, launch_ahead):
    """40 requests with prompts of 1 to 60 tokens and 10 to 30 new tokens each, half greedy and
    half with seeded temperature, up to 64 at a time under a budget of 256 tokens a step: the
    number of decoding requests climbs past 16 and 32 and falls again as they end.  Every
    token is the plain implementation's (bfloat16: but for near-ties); all pages come back."""
    from rust_llm_inference_server_amd.engine import Engine
    name, cfg, per_dtype = case
    folder, w, c = per_dtype[dtype]
    g = torch.Generator().manual_seed(17)
    lengths = torch.randint(1, 61, (40,), generator=g).tolist()
    news = torch.randint(10, 31, (40,), generator=g).tolist()
    prompts = [torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for n in lengths]
    params = [SamplingParams.greedy(n) if i % 2 == 0 else
              SamplingParams(temperature=0.8, seed=100 + i, max_tokens=n)
              for i, n in enumerate(news)]
    engine = Engine(load(folder, dtype, 128), EngineConfig(
        max_num_seqs=64, max_batched_tokens=256, num_pages=40 * 6 + 8, block_size=16,
        max_seq_len=128, watermark_pages=1, launch_ahead=launch_ahead))
    rows = []
    real_sampled, real_chained, real_step = (engine.runner.step_sampled, engine.runner.step_chained,
                                             engine.runner.step)
    engine.runner.step_sampled = lambda i, t, m: rows.append(len(i)) or real_sampled(i, t, m)
    engine.runner.step_chained = lambda i, m, s: rows.append(len(i)) or real_chained(i, m, s)
    engine.runner.step = lambda e, **kw: rows.append(sum(len(x.tokens) for x in e)) or real_step(e, **kw)
    outs = engine.generate(prompts, params)
    margin = near_ties.margin_for(dtype)
    picks = 0
    for p, o, sp, n in zip(prompts, outs, params, news):
        assert o.finish_reason == "length" and len(o.token_ids) == n
        picks += near_ties.near_tie_picks(w, c, p, o.token_ids, margin, sp.temperature, sp.seed or 0)
    if dtype == "float32":
        assert picks == 0
    # the steps did cross the boundaries: 17 to 32 rows, 33 to 64 rows, and fewer again
    assert any(16 < r <= 32 for r in rows) and any(32 < r <= 64 for r in rows), sorted(set(rows))
    assert any(r <= 16 for r in rows)
    if engine.runner.use_graphs:
        assert {32, 64} <= set(engine.runner._graphs), sorted(engine.runner._graphs)
    assert engine.runner.cache.num_free_pages() == 40 * 6 + 8
    engine.runner.cache.check_invariants()
    print(f"{name} {dtype} ahead={launch_ahead}: {len(rows)} steps, {picks} near-tie picks, "
          f"largest step {max(rows)} rows")


def rows_trace(reqs, prompt_len, counts):
    """The requests' prompts in steps of at most 96 tokens (the last token of each prompt
    wanted), then one decode step per entry of ``counts`` with that many of the requests, the
    first ones, all rows wanted; a count beyond the number of requests is made up by a
    two-token portion of a further request's prompt beside ``count - 2`` single tokens."""
    keys = list(reqs)
    steps, pos = [], {k: 0 for k in keys}

    def add(entries, end=()):
        steps.append({"step": len(steps), "entries": entries, "end": list(end)})

    batch = []
    for k in keys[:-1]:
        batch.append({"id": k, "tokens": reqs[k][:prompt_len[k]],
                      "want": [prompt_len[k] - 1]})
        pos[k] = prompt_len[k]
        if sum(len(e["tokens"]) for e in batch) >= 96 - 12:
            add(batch)
            batch = []
    if batch:
        add(batch)
    extra = keys[-1]
    for n in counts:
        portion = n > len(keys) - 1
        live = [k for k in keys[:-1][:n - 2 if portion else n] if pos[k] < len(reqs[k])]
        entries = [{"id": k, "tokens": [reqs[k][pos[k]]], "want": [0]} for k in live]
        for k in live:
            pos[k] += 1
        if portion and pos[extra] + 2 <= len(reqs[extra]):
            entries.append({"id": extra, "tokens": reqs[extra][pos[extra]:pos[extra] + 2],
                            "want": [0, 1]})
            pos[extra] += 2
        add(entries)
    steps[-1]["end"] = keys
    return steps


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_logits_of_steps_with_17_33_and_64_rows(case, dtype):
    """64 requests with prompts of 1 to 12 tokens decode together, and the number of rows in
    a step moves through 16, 17, 32, 1, 24, ... 64, 33, 65 (63 single tokens beside a two-token
    portion), 48, 64 ...: a request's consecutive tokens are computed by the kernels of each range in
    turn.  Every logit is the plain implementation's within the replay tests' gates; captured
    steps give bit for bit what eager steps give while the engine's own kernels compute (all
    of float32, and bfloat16 up to the first step that brings the library's products in), and
    the same within the gate from there on."""
    from rust_llm_inference_server_amd.engine import ModelRunner
    name, cfg, per_dtype = case
    folder, w, c = per_dtype[dtype]
    g = torch.Generator().manual_seed(23)
    prompt_len = {f"r{i}": int(n) for i, n in enumerate(torch.randint(1, 13, (65,), generator=g))}
    counts = [16, 17, 32, 1, 24, 16, 32, 17, 64, 33, 65, 48, 64, 66, 33, 16, 64]
    reqs = {k: torch.randint(0, cfg["vocab_size"], (n + len(counts) + 2,), generator=g).tolist()
            for k, n in prompt_len.items()}
    reqs["r64"] = reqs["r64"][:10]
    prompt_len["r64"] = 0
    steps = rows_trace(reqs, prompt_len, counts)
    sizes = [sum(len(e["tokens"]) for e in s["entries"]) for s in steps]
    assert {17, 33, 64, 65, 16, 32, 1} <= set(sizes)
    ref = {k: plain.forward(w, c, t) for k, t in reqs.items()}
    outputs = {}
    for graphs in (True, False):
        runner = ModelRunner(load(folder, dtype, 64), num_pages=65 * 2, page_size=16,
                             max_num_seqs=65, use_graphs=graphs)
        outputs[graphs] = traces.replay_in_process(runner, steps)
        if graphs and runner.use_graphs:
            assert {1, 16, 32, 64} <= set(runner._graphs), sorted(runner._graphs)
        assert runner.cache.num_free_pages(0) == runner.cache.num_pages(0)
    got = traces.collect(steps, outputs[True], cfg["vocab_size"])
    worst = 0.0
    for k, positions in got.items():
        for p, row in positions.items():
            diff = (row - ref[k][p]).abs().max().item()
            assert diff <= TOL[dtype], f"request {k} position {p}: |diff| {diff:.3e}"
            worst = max(worst, diff)
    assert sum(len(v) for v in got.values()) > 600
    # A captured step runs its bucket's rows, the eager one the step's own count.  Where the
    # engine's kernels compute, a row's bits do not depend on the count; the library's products
    # (bfloat16 beyond the rows that the streaming kernels take: 32 for widths that are a
    # multiple of 256, else 16) may take another algorithm for another count (each is tried out
    # on its own) and then sum a row's k in another order.  From the first such step on the two
    # runs' caches differ by rounding, and so does everything behind it.
    own = 1 << 30 if dtype == "float32" else (32 if name == "w" else 16)
    single = [all(len(e["tokens"]) == 1 for e in s["entries"]) for s in steps]
    exact = True
    for k in sorted(outputs[False]):
        exact = exact and not (single[k] and own < sizes[k] <= 64)
        if exact:
            assert torch.equal(outputs[True][k], outputs[False][k]), f"step {k} ({sizes[k]} rows)"
        else:
            assert (outputs[True][k] - outputs[False][k]).abs().max().item() <= TOL[dtype], \
                f"step {k} ({sizes[k]} rows)"
    print(f"{name} {dtype}: worst |diff| {worst:.3e} over {sum(len(v) for v in got.values())} rows")
