"""The request loop end to end on tiny random models, as the reference's engine tests do
(crates/engine/tests/engine.rs:58-275): every case runs on the GPU (``-m gpu``) and, with the
kernels replaced by the slow torch double, on the CPU, where it tests the host logic alone."""
import pytest
import torch

import near_ties
import plain_llama as plain
from rust_llm_inference_server_amd.config import EngineConfig
from rust_llm_inference_server_amd.sampling import SamplingParams

BACKENDS = ["double", pytest.param("gpu", marks=pytest.mark.gpu)]


@pytest.fixture(params=BACKENDS)
def backend(request):
    if request.param == "double":
        import cpu_ops
        cpu_ops.install(request.getfixturevalue("monkeypatch"))
        return torch.device("cpu")
    return torch.device("cuda", 0)


@pytest.fixture(params=["float32", pytest.param("bfloat16", marks=pytest.mark.gpu)])
def dtype(request, backend):
    """The engine's behaviours hold in both precisions; bfloat16 runs on the GPU only."""
    if request.param == "bfloat16" and backend.type != "cuda":
        pytest.skip("bfloat16 runs on the GPU only")
    return request.param


@pytest.fixture
def folders(dtype, tiny_folders, tiny_folders_bf16):
    """Model folders whose stored weights are the numbers the engine computes with."""
    return tiny_folders if dtype == "float32" else tiny_folders_bf16


class Judge:
    """Generated tokens against the plain float32 implementation on the same weights: equal in
    float32; in bfloat16 equal except at near-ties of the float32 scores (near_ties.py)."""

    def __init__(self, folder, dtype):
        self.w, self.c = plain.read_weights(folder), plain.read_config(folder)
        self.margin = near_ties.margin_for(dtype)
        self.picks = 0

    def check(self, prompts, outputs, params):
        if isinstance(params, SamplingParams):
            params = [params] * len(prompts)
        for p, o, sp in zip(prompts, outputs, params):
            tokens = o if isinstance(o, list) else o.token_ids
            self.picks += near_ties.near_tie_picks(self.w, self.c, p, tokens, self.margin,
                                                   sp.temperature, sp.seed or 0)

    def same(self, a, b):
        """Two runs of the same requests: the same tokens; in bfloat16 they may part at a
        near-tie (each run has been checked on its own)."""
        if self.margin == 0.0:
            assert a == b
        return sum(x != y for x, y in zip(a, b))


def load(folder, device, dtype="float32", max_positions=256):
    from rust_llm_inference_server_amd.engine import load_model
    return load_model(folder, dtype, max_positions, device)


def engine_for(model, **kw):
    from rust_llm_inference_server_amd.engine import Engine
    cfg = dict(max_num_seqs=8, max_batched_tokens=64, num_pages=64, block_size=8,
               max_seq_len=256, watermark_pages=1)
    cfg.update(kw)
    return Engine(model, EngineConfig(**cfg))


def prompts_for(vocab, lengths, seed=0):
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, vocab, (n,), generator=g).tolist() for n in lengths]


def test_greedy_generation_matches_the_plain_implementation(backend, dtype, folders):
    """Prompts of 5, 17 and 33 tokens (and 1, 9 and 40), 8 greedy tokens each."""
    for name, lengths in (("a", [5, 17, 33]), ("b", [1, 9, 40])):
        folder = folders[name]
        judge = Judge(folder, dtype)
        prompts = prompts_for(judge.c["vocab_size"], lengths, seed=1)
        engine = engine_for(load(folder, backend, dtype), max_batched_tokens=24)
        outs = engine.generate(prompts, SamplingParams.greedy(8))
        judge.check(prompts, outs, SamplingParams.greedy(8))
        for p, o in zip(prompts, outs):
            if dtype == "float32":
                assert o.token_ids == plain.greedy_generate(judge.w, judge.c, p, 8)
            assert o.finish_reason == "length" and o.prompt_tokens == len(p)
        assert engine.runner.cache.num_free_pages() == 64


def test_batched_equals_solo_and_chunked_equals_single_shot(backend, dtype, folders):
    model = load(folders["b"], backend, dtype)
    judge = Judge(folders["b"], dtype)
    prompts = prompts_for(384, [30, 3, 57, 12], seed=2)
    sp = SamplingParams.greedy(6)
    together = [o.token_ids for o in engine_for(model).generate(prompts, sp)]
    solo = [engine_for(model).generate([p], sp)[0].token_ids for p in prompts]
    chunked = [o.token_ids for o in engine_for(model, max_batched_tokens=16).generate(prompts, sp)]
    static = [o.token_ids for o in engine_for(model, scheduler="static").generate(prompts, sp)]
    for run in (together, solo, chunked, static):
        judge.check(prompts, run, sp)
    judge.same(together, solo)
    judge.same(chunked, together)                   # engine.rs tests: budget 16 == single shot
    judge.same(static, together)


def test_preemption_and_recompute_do_not_change_the_output(backend, dtype, folders):
    """So few pages that running requests are preempted (engine.rs tests 157-194): the victims
    recompute prompt and generated tokens and continue with the same tokens."""
    model = load(folders["a"], backend, dtype, max_positions=128)
    judge = Judge(folders["a"], dtype)
    prompts = prompts_for(256, [9] * 6, seed=3)
    for sp in (SamplingParams.greedy(24), SamplingParams(temperature=0.8, seed=11, max_tokens=24)):
        roomy = engine_for(model, num_pages=64)
        want = [o.token_ids for o in roomy.generate(prompts, sp)]
        assert roomy.stats().preemptions == 0
        tight = engine_for(model, num_pages=12, watermark_pages=0)
        got = [o.token_ids for o in tight.generate(prompts, sp)]
        assert tight.stats().preemptions > 0
        judge.check(prompts, want, sp)
        judge.check(prompts, got, sp)
        judge.same(got, want)
        assert tight.runner.cache.num_free_pages() == 12
        tight.runner.cache.check_invariants()


def test_seeded_temperature_ignores_the_neighbours(backend, dtype, folders):
    model = load(folders["b"], backend, dtype)
    judge = Judge(folders["b"], dtype)
    prompts = prompts_for(384, [1, 9, 40, 100], seed=4)
    sp = SamplingParams(temperature=0.8, seed=1234, max_tokens=12)
    among = [o.token_ids for o in engine_for(model, max_batched_tokens=24).generate(prompts, sp)]
    alone = [engine_for(model).generate([p], sp)[0].token_ids for p in prompts]
    again = [o.token_ids for o in engine_for(model).generate(prompts, sp)]
    for run in (among, alone, again):
        judge.check(prompts, run, sp)
    judge.same(among, alone)
    judge.same(again, among)                         # same seed, same tokens
    other = engine_for(model).generate(prompts[2:3], SamplingParams(temperature=0.8, seed=5, max_tokens=12))
    assert other[0].token_ids != among[2]
    assert len(set(among[3])) > 1


def test_steps_that_sample_inside_the_graph_pick_the_eager_steps_tokens(backend, dtype, folders):
    """Decode steps whose every request the device kernel can sample for run as one captured
    graph, metadata copy, model, sampling kernel and the tokens' way to the host included: the
    same tokens as the engine without captured steps, greedy and with seeded temperature, for
    requests that arrive and end at different steps; a request with a host-side sampler in the
    batch sends the step down the other path, to the same tokens again."""
    if backend.type != "cuda":
        pytest.skip("captured steps exist on the GPU only")
    model = load(folders["b"], backend, dtype)
    prompts = prompts_for(384, [3, 17, 40, 9, 1], seed=8)
    params = [SamplingParams.greedy(14), SamplingParams(temperature=0.7, seed=5, max_tokens=9),
              SamplingParams(temperature=1.1, seed=6, max_tokens=14), SamplingParams.greedy(3),
              SamplingParams(temperature=0.9, seed=7, max_tokens=11)]
    runs = {}
    for graphs in (True, False):
        engine = engine_for(model, use_graphs=graphs, max_batched_tokens=32)
        assert engine.runner.use_graphs == graphs
        sampled_steps = []
        if graphs:
            real, chained = engine.runner.step_sampled, engine.runner.step_chained
            engine.runner.step_sampled = lambda i, t, m: sampled_steps.append(len(i)) or real(i, t, m)
            engine.runner.step_chained = lambda i, m, s: sampled_steps.append(len(i)) or chained(i, m, s)
        runs[graphs] = [o.token_ids for o in engine.generate(prompts, params)]
        if graphs:
            assert len(sampled_steps) >= 10 and max(sampled_steps) == 5
    assert runs[True] == runs[False]
    mixed = params[:4] + [SamplingParams(temperature=0.9, top_k=50, seed=7, max_tokens=11)]
    with_host = {}
    for graphs in (True, False):
        engine = engine_for(model, use_graphs=graphs, max_batched_tokens=32)
        with_host[graphs] = [o.token_ids for o in engine.generate(prompts, mixed)]
    assert with_host[True] == with_host[False]
    assert with_host[True][:4] == runs[True][:4]


def test_decode_steps_launched_ahead_give_the_same_completions(backend, dtype, folders):
    """A decode step is launched on the tokens of the step before as they lie on the device,
    before the host has seen them, wherever the next step does not depend on them.  The
    completions are those of an engine that waits for every step: with requests that end at
    different steps by their limit, requests that stop at an EOS (one position computed in
    vain, its row dropped), a request added and one cancelled while steps are in flight, greedy
    and with seeded temperature; and everything is given back at the end."""
    if backend.type != "cuda":
        pytest.skip("captured steps exist on the GPU only")
    from rust_llm_inference_server_amd.engine import Engine
    model = load(folders["b"], backend, dtype)
    prompts = prompts_for(384, [3, 17, 40, 9, 1, 22], seed=18)
    params = [SamplingParams.greedy(30), SamplingParams(temperature=0.7, seed=5, max_tokens=19),
              SamplingParams(temperature=1.1, seed=6, max_tokens=30), SamplingParams.greedy(2),
              SamplingParams(temperature=0.9, seed=7, max_tokens=25), SamplingParams.greedy(12)]

    def run(ahead, eos=(), seats=8):
        cfg = EngineConfig(max_num_seqs=seats, max_batched_tokens=32, num_pages=64, block_size=8,
                           max_seq_len=256, watermark_pages=1, launch_ahead=ahead)
        engine = Engine(model, cfg, eos_token_ids=eos)
        chained = []
        real = engine.runner.step_chained

        def counted(i, m, s):
            chained.append((len(i), engine.scheduler.num_waiting))
            return real(i, m, s)
        engine.runner.step_chained = counted
        ids = [engine.add_request(p, sp) for p, sp in zip(prompts[:4], params[:4])]
        streamed = {}
        calls = 0
        while engine.has_work():
            for seq_id, token, finished in engine.step():
                if token is not None:
                    streamed.setdefault(seq_id, []).append(token)
            calls += 1
            if calls == 6:                 # decoding is under way: one more request, one fewer
                ids.append(engine.add_request(prompts[4], params[4]))
                engine.cancel(ids[2])
            if calls == 9:
                ids.append(engine.add_request(prompts[5], params[5]))
        done = {i: engine.pop_finished(i) for i in ids if i != ids[2]}
        assert all(c is not None for c in done.values())
        for i, c in done.items():
            assert streamed.get(i, []) == c.token_ids
        assert engine.runner.cache.num_free_pages() == 64
        engine.runner.cache.check_invariants()
        engine.scheduler.check()
        return [(c.token_ids, c.finish_reason) for c in done.values()], chained

    waited, none = run(False)
    ahead, chained = run(True)
    assert not none and len(chained) >= 12 and max(n for n, _ in chained) >= 3
    assert ahead == waited
    # with every seat taken nobody can be admitted, and steps are launched ahead past the queue
    # (other steps hold other requests then: in bfloat16 a near-tie may fall the other way)
    crowded, chained = run(True, seats=2)
    assert any(queue for _, queue in chained)
    judge = Judge(folders["b"], dtype)
    kept = [0, 1, 3, 4, 5]
    judge.check([prompts[i] for i in kept], [t for t, _ in crowded], [params[i] for i in kept])
    judge.same([t for t, _ in crowded], [t for t, _ in waited])
    assert [r for _, r in crowded] == [r for _, r in waited]
    # tokens that the runs above produced in the middle of a completion now end their requests
    eos = {waited[0][0][7], waited[1][0][4], waited[3][0][9]}
    stopped, _ = run(False, eos)
    assert [r for _, r in stopped].count("stop") >= 3
    ahead_stopped, chained = run(True, eos)
    assert ahead_stopped == stopped and len(chained) >= 5


def test_warm_up_captures_the_decode_steps_and_moves_nothing(backend, dtype, folders):
    """``Engine.warm_up`` captures the decode steps of every batch and context bucket on
    padding: afterwards no step captures any more, and a warm-up in the middle of a generation
    (with a step in flight) leaves every request's cache, state and tokens as they were."""
    if backend.type != "cuda":
        pytest.skip("captured steps exist on the GPU only")
    from rust_llm_inference_server_amd.engine.graph import DecodeGraph
    model = load(folders["a"], backend, dtype, max_positions=128)
    prompts = prompts_for(256, [5, 17, 33], seed=21)
    params = [SamplingParams.greedy(20), SamplingParams(temperature=0.8, seed=3, max_tokens=16),
              SamplingParams.greedy(9)]
    want = [o.token_ids for o in engine_for(model, max_seq_len=128).generate(prompts, params)]
    captures = []
    real = DecodeGraph._capture

    def counted(self, context_limit, kind):
        captures.append((self.bucket, context_limit, kind))
        return real(self, context_limit, kind)
    DecodeGraph._capture = counted
    try:
        engine = engine_for(model, max_seq_len=128)
        made = engine.warm_up()
        assert made == len(captures) == 4              # batches of 1, 2, 4, 8; one context bucket
        assert engine.warm_up() == 0
        got = [o.token_ids for o in engine.generate(prompts, params)]
        assert len(captures) == 4
        late = engine_for(model, max_seq_len=128)
        ids = [late.add_request(p, sp) for p, sp in zip(prompts, params)]
        for _ in range(5):
            late.step()
        assert late.warm_up() > 0                      # a step is in flight meanwhile
        while late.has_work():
            late.step()
        mid = [late.pop_finished(i).token_ids for i in ids]
    finally:
        DecodeGraph._capture = real
    assert got == want and mid == want


def test_host_sampler_modes_run_and_are_reproducible(backend, tiny_folders):
    model = load(tiny_folders["b"], backend)
    prompts = prompts_for(384, [7, 21], seed=5)
    one = SamplingParams(temperature=0.9, top_k=1, seed=3, max_tokens=6)
    greedy = [o.token_ids for o in engine_for(model).generate(prompts, SamplingParams.greedy(6))]
    assert [o.token_ids for o in engine_for(model).generate(prompts, one)] == greedy
    sp = SamplingParams(temperature=1.2, top_k=20, top_p=0.9, repetition_penalty=1.3, seed=3, max_tokens=6)
    a = [o.token_ids for o in engine_for(model).generate(prompts, sp)]
    b = [o.token_ids for o in engine_for(model).generate(prompts[::-1], sp)][::-1]
    assert a == b


def test_eos_and_limits(backend, tiny_folders):
    model = load(tiny_folders["a"], backend, max_positions=128)
    prompt = prompts_for(256, [6], seed=6)[0]
    from rust_llm_inference_server_amd.engine import Engine
    first = engine_for(model).generate([prompt], SamplingParams.greedy(3))[0].token_ids[0]
    cfg = EngineConfig(max_num_seqs=2, max_batched_tokens=64, num_pages=16, block_size=8, max_seq_len=128)
    stops = Engine(model, cfg, eos_token_ids=[first])
    out = stops.generate([prompt], SamplingParams.greedy(5))[0]
    assert (out.finish_reason, out.token_ids) == ("stop", [])       # EOS is not appended
    out = stops.generate([prompt], SamplingParams(max_tokens=5, ignore_eos=True))[0]
    assert out.finish_reason == "length" and len(out.token_ids) == 5
    with pytest.raises(ValueError, match="empty prompt or max_tokens of 0"):
        stops.add_request([], SamplingParams())
    with pytest.raises(ValueError, match="empty prompt or max_tokens of 0"):
        stops.add_request([1], SamplingParams(max_tokens=0))
    with pytest.raises(ValueError, match="exceeds max_seq_len"):
        stops.add_request([1] * 100, SamplingParams(max_tokens=100))
    with pytest.raises(ValueError, match="outside the vocabulary"):
        stops.add_request([256], SamplingParams())


def test_the_folders_generation_config_names_the_stop_tokens(backend, tiny_folders, tmp_path):
    """An engine built from a folder stops at the ids of its ``generation_config.json``, which
    come before those of ``config.json`` (crates/engine/src/tokenizer.rs:64-85)."""
    import json
    import shutil
    from rust_llm_inference_server_amd.engine import Engine
    prompt = prompts_for(256, [6], seed=6)[0]
    sp = SamplingParams(temperature=2.0, seed=3, max_tokens=4)       # (greedy repeats itself here)
    greedy = engine_for(load(tiny_folders["a"], backend, max_positions=128)).generate(
        [prompt], sp)[0].token_ids
    assert len(set(greedy[:3])) == 3
    folder = tmp_path / "with_generation_config"
    shutil.copytree(tiny_folders["a"], folder)
    config = json.loads((folder / "config.json").read_text())
    config["eos_token_id"] = greedy[2]
    (folder / "config.json").write_text(json.dumps(config))
    cfg = EngineConfig(max_num_seqs=2, max_batched_tokens=64, num_pages=16, block_size=8, max_seq_len=128)

    def run():
        engine = Engine(load(str(folder), backend, max_positions=128), cfg)
        out = engine.generate([prompt], sp)[0]
        return engine.eos_token_ids, out.finish_reason, out.token_ids

    assert run() == ({greedy[2]}, "stop", greedy[:2])               # config.json alone
    (folder / "generation_config.json").write_text(json.dumps({"eos_token_id": [greedy[1], 300]}))
    assert run() == ({greedy[1], 300}, "stop", greedy[:1])          # generation_config.json first
    (folder / "generation_config.json").write_text(json.dumps({"do_sample": True}))
    assert run()[1:] == ("stop", greedy[:2])                        # no ids there: config.json


def test_cancel_returns_the_pages(backend, tiny_folders):
    model = load(tiny_folders["a"], backend, max_positions=128)
    engine = engine_for(model, num_pages=16)
    a = engine.add_request(prompts_for(256, [20])[0], SamplingParams.greedy(50))
    b = engine.add_request(prompts_for(256, [5])[0], SamplingParams.greedy(4))
    engine.step()
    engine.cancel(a)
    while engine.has_work():
        engine.step()
    assert engine.pop_finished(b).finish_reason == "length" and engine.pop_finished(a) is None
    assert engine.runner.cache.num_free_pages() == 16


def test_decoding_requests_go_to_the_step_longest_context_first(backend, tiny_folders, monkeypatch):
    """The attention kernel's workgroups start in the batch's order, so the engine hands the
    requests of a step over with single tokens first and the longest contexts in front; what
    each request generates does not depend on that (the other tests), and steps launched
    ahead keep the order of the step before them."""
    model = load(tiny_folders["a"], backend, max_positions=128)
    engine = engine_for(model, launch_ahead=True)
    lengths = [5, 31, 12, 40, 7]
    ids = [engine.add_request(p, SamplingParams.greedy(6)) for p in prompts_for(256, lengths, seed=3)]
    runner, seen = engine.runner, []
    real_step, real_sampled, real_chained = runner.step, runner.step_sampled, runner.step_chained

    def note(order):
        held = [len(engine._seqs[i].tokens) for i in order]
        seen.append((list(order), held))

    monkeypatch.setattr(runner, "step", lambda entries, **kw: (
        note([e.seq_id for e in entries if len(e.tokens) == 1]), real_step(entries, **kw))[1])
    monkeypatch.setattr(runner, "step_sampled", lambda i, t, m: (note(i), real_sampled(i, t, m))[1])
    monkeypatch.setattr(runner, "step_chained", lambda i, m, side: (
        seen.append((list(i), None)), real_chained(i, m, side))[1])
    while engine.has_work():
        engine.step()
    assert all(engine.pop_finished(i).finish_reason == "length" for i in ids)
    decoding = [order for order, held in seen if held is not None and len(order) > 1]
    assert decoding, "no step with several decoding requests"
    for order, held in seen:
        if held is not None:
            assert held == sorted(held, reverse=True), (order, held)
    # a step launched ahead lists the requests as the step before it did
    for before, after in zip(seen, seen[1:]):
        if after[1] is None:
            assert after[0] == before[0]


def test_a_failed_step_fails_only_its_own_requests(backend, tiny_folders):
    """crates/engine/src/engine.rs:523-528.  The first step holds a portion of the long request
    alone (it uses the whole budget); the model step is made to raise once."""
    model = load(tiny_folders["a"], backend, max_positions=128)
    engine = engine_for(model, num_pages=16, max_batched_tokens=16)
    a = engine.add_request(prompts_for(256, [20])[0], SamplingParams.greedy(4))
    b = engine.add_request(prompts_for(256, [5], seed=1)[0], SamplingParams.greedy(4))
    real, calls = engine.runner.step, []

    def failing(entries, **kw):
        calls.append([e.seq_id for e in entries])
        if len(calls) == 1:
            raise RuntimeError("the device said no")
        return real(entries, **kw)

    engine.runner.step = failing
    with pytest.raises(RuntimeError, match="the device said no"):
        engine.step()
    assert calls == [[a]]
    failed = engine.pop_finished(a)
    assert failed.finish_reason == "error" and "the device said no" in failed.error
    assert engine.runner.cache.num_free_pages() == 16
    while engine.has_work():
        engine.step()
    done = engine.pop_finished(b)
    assert done.finish_reason == "length" and len(done.token_ids) == 4 and done.error is None
    assert engine.runner.cache.num_free_pages() == 16


def test_perplexity_matches_the_plain_implementation(backend, tiny_folders):
    """crates/engine/src/perplexity.rs:26-80, windows of 16 and of 13 tokens over 70."""
    from rust_llm_inference_server_amd.engine import ModelRunner
    from rust_llm_inference_server_amd.engine.perplexity import perplexity
    folder = tiny_folders["b"]
    w, c = plain.read_weights(folder), plain.read_config(folder)
    tokens = prompts_for(c["vocab_size"], [70], seed=9)[0]
    runner = ModelRunner(load(folder, backend), num_pages=4, page_size=8, max_num_seqs=2)
    for ctx, max_windows in ((16, 0), (13, 3)):
        seen = []
        got = perplexity(runner, tokens, bos=1, ctx=ctx, max_windows=max_windows,
                         progress=lambda done, total, ppl: seen.append((done, total)))
        want = plain.perplexity(w, c, tokens, bos=1, ctx=ctx, max_windows=max_windows)
        assert (got.windows, got.tokens_scored) == (want["windows"], want["tokens_scored"])
        assert seen == [(i + 1, got.windows) for i in range(got.windows)]
        assert abs(got.mean_nll - want["mean_nll"]) < 1e-5
        assert abs(got.ppl - want["ppl"]) < 1e-4 * want["ppl"]
        assert abs(got.ppl_stderr - want["ppl_stderr"]) < 1e-3 * want["ppl"]
    assert runner.cache.num_free_pages() == 4
    with pytest.raises(ValueError, match="ctx must be at least 4"):
        perplexity(runner, tokens, bos=1, ctx=3)
    with pytest.raises(ValueError, match="shorter than one window"):
        perplexity(runner, tokens[:10], bos=1, ctx=16)


def test_perplexity_gives_its_pages_back_when_a_step_fails(backend, tiny_folders):
    from rust_llm_inference_server_amd.engine import ModelRunner
    from rust_llm_inference_server_amd.engine.perplexity import perplexity
    folder = tiny_folders["a"]
    tokens = prompts_for(256, [40], seed=3)[0]
    runner = ModelRunner(load(folder, backend, max_positions=128), num_pages=4, page_size=8, max_num_seqs=2)
    real, calls = runner.step, []

    def failing(entries, **kw):
        calls.append(1)
        if len(calls) == 2:
            raise RuntimeError("the device said no")
        return real(entries, **kw)

    runner.step = failing
    with pytest.raises(RuntimeError, match="the device said no"):
        perplexity(runner, tokens, bos=1, ctx=16)
    assert runner.cache.num_free_pages() == 4 and not runner.cache.contains(-1)
    runner.step = real
    assert perplexity(runner, tokens, bos=1, ctx=16).windows == 2


def test_pool_size_watermark_and_budget_follow_the_references_rules(backend, tiny_folders):
    """crates/engine/src/engine.rs:252-280: pages = pool bytes / (bytes of K and V per token *
    block size); watermark = max(1, pages / 100); the budget is at least max_num_seqs; the
    longest request is bounded by the rope table and by the pool."""
    from rust_llm_inference_server_amd.engine import Engine
    model = load(tiny_folders["a"], backend, max_positions=128)        # float32
    per_token = 2 * 2 * 1 * 16 * 4                                     # K and V, layers, kv heads, d
    cfg = EngineConfig(kv_cache_gb=0.001, block_size=16, max_num_seqs=8, max_batched_tokens=4,
                       max_seq_len=128)
    engine = Engine(model, cfg)
    pages = int(0.001 * (1 << 30)) // (per_token * 16)
    assert engine.runner.cache.num_pages(0) == pages == 262
    assert engine.scheduler.max_batched_tokens == 8
    assert engine.scheduler.max_seq_tokens == (pages - max(1, pages // 100)) * 16
    assert engine.max_seq_len == 128
    small = Engine(model, EngineConfig(num_pages=5, block_size=8, max_num_seqs=2, max_seq_len=128))
    assert small.max_seq_len == (5 - 1) * 8
    with pytest.raises(ValueError, match="at least 2"):
        Engine(model, EngineConfig(num_pages=1, block_size=8, max_num_seqs=2))
    defaults = EngineConfig()                                          # engine.rs:31-63
    assert (defaults.max_num_seqs, defaults.max_batched_tokens, defaults.kv_cache_gb,
            defaults.block_size, defaults.scheduler) == (64, 2048, 1.0, 16, "continuous")
    for bad in (dict(max_num_seqs=0), dict(block_size=0), dict(scheduler="fair"),
                dict(max_batched_tokens=0)):
        with pytest.raises(ValueError):
            EngineConfig(**bad).validate()


@pytest.mark.parametrize("seed", range(4))
def test_random_workloads_give_what_each_request_gives_alone(backend, dtype, folders, seed):
    """Requests of random lengths and sampling parameters, arriving while others run, under a
    random budget, page size and a pool small enough to preempt now and then: every request
    ends with the tokens it produces alone in a roomy engine, and every page comes back."""
    import random
    rng = random.Random(seed)
    name = rng.choice(["a", "b"])
    model = load(folders[name], backend, dtype, max_positions=128)
    judge = Judge(folders[name], dtype)
    vocab = judge.c["vocab_size"]
    n = rng.randrange(4, 9)
    prompts = prompts_for(vocab, [rng.choice([1, 2, 7, 16, 17, 33, 60]) for _ in range(n)], seed)
    params = []
    for i in range(n):
        mt = rng.randrange(1, 20)
        # (the host sampler's draws are not keyed like the device's: judged in float32 only)
        kind = rng.choice(["greedy", "temperature", "host"] if dtype == "float32"
                          else ["greedy", "temperature"])
        if kind == "greedy":
            params.append(SamplingParams.greedy(mt))
        elif kind == "temperature":
            params.append(SamplingParams(temperature=rng.choice([0.5, 1.0]), seed=100 + i, max_tokens=mt))
        else:
            params.append(SamplingParams(temperature=0.9, top_k=rng.choice([0, 5]), top_p=rng.choice([1.0, 0.8]),
                                         repetition_penalty=rng.choice([1.0, 1.2]), seed=200 + i, max_tokens=mt))
    alone = [engine_for(model).generate([p], sp)[0].token_ids for p, sp in zip(prompts, params)]
    block = rng.choice([8, 16])
    longest = max(len(p) + sp.max_tokens for p, sp in zip(prompts, params))
    pages = -(-longest // block) + rng.randrange(1, 6)
    engine = engine_for(model, num_pages=pages, block_size=block, watermark_pages=rng.choice([0, 1]),
                        max_num_seqs=rng.choice([2, 4, 8]), max_batched_tokens=rng.choice([8, 24, 64]))
    ids, pending, steps = {}, list(range(n)), 0
    while pending or engine.has_work():
        for _ in range(rng.randrange(0, 3)):                  # arrivals between steps
            if pending:
                i = pending.pop(0)
                ids[engine.add_request(prompts[i], params[i])] = i
        if engine.has_work():
            engine.step()
        steps += 1
        assert steps < 5000
    got = {ids[k]: engine.pop_finished(k) for k in ids}
    among = [got[i].token_ids for i in range(n)]
    if dtype != "float32":
        judge.check(prompts, among, params)
        judge.check(prompts, alone, params)
    judge.same(among, alone)
    assert engine.runner.cache.num_free_pages() == pages
    engine.runner.cache.check_invariants()
