"""The engine against the plain implementation, request by request and position by position,
under every way of cutting the work: whole prompts; most of a prompt in one step and the last
32 tokens one by one; portions of changing size down to two tokens; and up to four live
requests mixed, portions of some beside single tokens of others, with so few pages that they
are used again.  In float32 (the true 32-bit path) and in bfloat16, for three tiny
configurations that differ in every size and option."""

import pytest
import torch

import plain_llama as plain
import traces
from conftest import TINY, make_model_folder

pytestmark = pytest.mark.gpu

LENGTHS = [5, 17, 33, 100, 64, 1, 150, 47, 2, 129]
# Largest |logit difference| allowed.  float32: the reference's own gate for its tiny model
# (crates/model/src/llama.rs:355: < 1e-4).  bfloat16: measured against the plain float32
# implementation on the same bfloat16-rounded weights, with headroom, then frozen
# (the procedure of crates/model/tests/parity.rs:17-24).
TOL = {"float32": 1e-4, "bfloat16": 2e-2}


@pytest.fixture(scope="module", params=sorted(TINY))
def case(request, tmp_path_factory):
    name = request.param
    cfg = TINY[name]
    out = {}
    for dtype, tdt in (("float32", torch.float32), ("bfloat16", torch.bfloat16)):
        folder = make_model_folder(tmp_path_factory.mktemp(f"{name}_{dtype}"), cfg, seed=7, dtype=tdt)
        w, c = plain.read_weights(folder), plain.read_config(folder)
        lengths = [min(n, cfg["max_position_embeddings"]) for n in LENGTHS]
        reqs = traces.random_requests(cfg["vocab_size"], lengths, seed=3)
        ref = {k: plain.forward(w, c, t) for k, t in reqs.items()}
        out[dtype] = (folder, reqs, ref)
    return name, cfg, out


def make_runner(folder, dtype, max_tokens, page_size=16, use_graphs=True):
    from rust_llm_inference_server_amd.engine import ModelRunner, load_model
    model = load_model(folder, dtype, max_positions=max(64, max_tokens))
    return ModelRunner(model, num_pages=-(-max_tokens // page_size), page_size=page_size,
                       max_num_seqs=16, use_graphs=use_graphs)


def check(steps, outputs, reqs, ref, vocab, tol):
    got = traces.collect(steps, outputs, vocab)
    worst = 0.0
    for k, tokens in reqs.items():
        assert sorted(got[k]) == list(range(len(tokens))), f"request {k}: positions missing"
        mine = torch.stack([got[k][p] for p in range(len(tokens))])
        diff = (mine - ref[k]).abs().max(dim=-1).values
        bad = (diff > tol).nonzero()
        assert bad.numel() == 0, (f"request {k}: first wrong position {int(bad[0])} of "
                                  f"{len(tokens)} (|diff| {diff[bad[0]].item():.3e} > {tol})")
        worst = max(worst, diff.max().item())
    return worst


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("family", ["whole", "tail", "portions", "mixed"])
def test_replay_families(case, dtype, family):
    name, cfg, per_dtype = case
    folder, reqs, ref = per_dtype[dtype]
    build = {"whole": traces.trace_whole, "tail": traces.trace_tail,
             "portions": traces.trace_portions, "mixed": traces.trace_mixed}[family]
    steps, max_tokens = build(reqs)
    runner = make_runner(folder, dtype, max_tokens, page_size=8 if name == "b" else 16)
    outputs = traces.replay_in_process(runner, steps)
    worst = check(steps, outputs, reqs, ref, cfg["vocab_size"], TOL[dtype])
    print(f"{name} {dtype} {family}: worst |diff| {worst:.3e}")
    # every page came back, and the kernels left the runner's counters at zero
    assert runner.cache.num_free_pages(0) == runner.cache.num_pages(0)
    assert int(runner.pools.counters.abs().sum()) == 0


def test_engine_matches_the_second_plain_implementation(case):
    """The engine's float32 logits, prefill and decoded tail, against the scalar-loop host
    implementation (plain_llama_host.cpp), which shares no code with the torch twin either."""
    import plain_host
    if not plain_host.available():
        pytest.skip("g++ is not on the PATH")
    name, cfg, per_dtype = case
    folder, reqs, _ = per_dtype["float32"]
    w, c = plain.read_weights(folder), plain.read_config(folder)
    some = {k: reqs[k] for k in ("r0", "r3", "r5")}            # 5, 100 and 1 tokens
    ref = {k: plain_host.forward(w, c, t) for k, t in some.items()}
    steps, max_tokens = traces.trace_tail(some)
    runner = make_runner(folder, "float32", max_tokens, page_size=8 if name == "b" else 16)
    outputs = traces.replay_in_process(runner, steps)
    check(steps, outputs, some, ref, cfg["vocab_size"], TOL["float32"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_captured_decode_steps_match_eager_ones(case, dtype):
    """Steps of one token per request run from a captured HIP graph.  Replayed many times with
    eager steps (prefill portions, page copies, host synchronisation) in between, every replay
    must give what the eager step gives, bit for bit in both precisions: the padding rows of a
    bucket and the fixed sizes of a captured launch change no row's arithmetic."""
    name, cfg, per_dtype = case
    folder, reqs, ref = per_dtype[dtype]
    page = 8 if name == "b" else 16
    for build in (traces.trace_tail, traces.trace_mixed):
        steps, max_tokens = build(reqs)
        eager = make_runner(folder, dtype, max_tokens, page, use_graphs=False)
        graphed = make_runner(folder, dtype, max_tokens, page, use_graphs=True)
        assert graphed.use_graphs and not eager.use_graphs
        out_e = traces.replay_in_process(eager, steps)
        out_g = traces.replay_in_process(graphed, steps)
        assert graphed._graphs, "no decode step took the graph path"
        check(steps, out_g, reqs, ref, cfg["vocab_size"], TOL[dtype])
        for k in out_e:
            assert torch.equal(out_g[k], out_e[k]), f"step {k}"


def rounds_of_one_schedule(vocab, rounds, page):
    """The same schedule of steps ``rounds`` times over (a portion of a prompt alone; two
    portions side by side; a single token beside a portion), each round with tokens of its own
    and, since a bystander of growing length holds pages meanwhile, on pages of its own."""
    g = torch.Generator().manual_seed(11)
    steps = []
    for r in range(rounds):
        a, b, c = (torch.randint(0, vocab, (n,), generator=g).tolist() for n in (42, 23, 9))
        z = torch.randint(0, vocab, (1 + r * page,), generator=g).tolist()
        n = len(steps)
        steps += [
            {"step": n, "entries": [{"id": f"z{r}", "tokens": z, "want": []}], "end": []},
            {"step": n + 1, "entries": [{"id": f"a{r}", "tokens": a[:17], "want": [16]}], "end": []},
            {"step": n + 2, "entries": [{"id": f"a{r}", "tokens": a[17:41], "want": [0, 23]},
                                        {"id": f"b{r}", "tokens": b, "want": [22]}], "end": []},
            {"step": n + 3, "entries": [{"id": f"a{r}", "tokens": a[41:], "want": [0]},
                                        {"id": f"c{r}", "tokens": c, "want": [3, 8]}],
             "end": [f"a{r}", f"b{r}", f"c{r}", f"z{r}"]},
        ]
    return steps


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_steps_whose_shape_comes_back_are_captured(case, dtype, monkeypatch):
    """A step that is no pure decode step is captured into a HIP graph when its shape (every
    sequence's cached and new positions, the number of wanted rows) has come back often enough,
    here the second time it is seen, and replayed from then on with the new step's metadata.  Five rounds of one schedule, each with
    other tokens on other pages, with eager steps and host synchronisation between the replays:
    every step must give what a runner without captured steps gives, bit for bit."""
    from rust_llm_inference_server_amd.engine.graph import RepeatedSteps
    assert RepeatedSteps.CAPTURE_AT > 2
    monkeypatch.setattr(RepeatedSteps, "CAPTURE_AT", 2)
    name, cfg, per_dtype = case
    folder, _, _ = per_dtype[dtype]
    page = 8 if name == "b" else 16
    rounds = 5
    steps = rounds_of_one_schedule(cfg["vocab_size"], rounds, page)
    max_tokens = 4 * 64 + rounds * page + 64
    eager = make_runner(folder, dtype, max_tokens, page)
    eager.capture_repeated_steps = False
    graphed = make_runner(folder, dtype, max_tokens, page)
    out_e = traces.replay_in_process(eager, steps)
    out_g = traces.replay_in_process(graphed, steps)
    assert eager._repeated is None
    # three shapes come back (the bystander's never does): captured in the second round,
    # replayed in that one and in the three after it
    assert len(graphed._repeated.graphs) == 3 and graphed._repeated.replays == 3 * (rounds - 1)
    assert sorted(out_e) == sorted(out_g) and len(out_g) == 3 * rounds
    for k in out_e:
        assert torch.equal(out_g[k], out_e[k]), f"step {k}"
    assert graphed.cache.num_free_pages(0) == graphed.cache.num_pages(0)
    assert int(graphed.pools.counters.abs().sum()) == 0
    # a fifth shape pushes the least recently used one out
    graphed._repeated.limit = 3
    extra = [{"step": 100 + i, "entries": [{"id": f"x{i}", "tokens": [1, 2, 3], "want": [2]}],
              "end": [f"x{i}"]} for i in range(3)]
    out_x = traces.replay_in_process(graphed, extra)
    assert len(graphed._repeated.graphs) == 3
    assert torch.equal(out_x[100], out_x[101]) and torch.equal(out_x[100], out_x[102])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_chained_steps_sample_what_fed_steps_sample(case, dtype):
    """``step_chained`` runs the same requests once more on the tokens that the sampling kernel
    of the step before left on the device, launched before the host has seen them.  Step after
    step it yields the tokens of a runner whose every step is fed from the host, greedy and
    with temperature, with other graphs captured in the middle of the chain; and it refuses
    to run when something else has been through the bucket's buffers since."""
    from rust_llm_inference_server_amd.engine import StepEntry
    from rust_llm_inference_server_amd.sampling import SamplingParams
    from rust_llm_inference_server_amd.sampling.sampler import Sampler
    name, cfg, per_dtype = case
    folder, reqs, _ = per_dtype[dtype]
    prompts = [list(t)[:n] for t, n in zip(reqs.values(), (9, 4, 13))]
    samplers = [Sampler(SamplingParams.greedy(64)),
                Sampler(SamplingParams(temperature=0.9, seed=4, max_tokens=64)),
                Sampler(SamplingParams(temperature=1.3, seed=9, max_tokens=64))]
    steps = 24

    def start():
        runner = make_runner(folder, dtype, 3 * 64, 8 if name == "b" else 16)
        for i, p in enumerate(prompts):
            runner.reserve(i, len(p) + steps + 1)
        runner.step([StepEntry(i, p[:-1], []) for i, p in enumerate(prompts)])
        return runner, [len(p) for p in prompts]

    ids = [0, 1, 2]
    fed, lens = start()
    tokens, want = [p[-1] for p in prompts], []
    for n in range(steps):
        modes = [s.device_mode(l + n) for s, l in zip(samplers, lens)]
        tokens = fed.step_sampled(ids, tokens, modes)()
        want.append(tokens)

    chained, lens = start()
    modes = [s.device_mode(l) for s, l in zip(samplers, lens)]
    wait = chained.step_sampled(ids, [p[-1] for p in prompts], modes)
    got = []
    for n in range(1, steps):
        modes = [s.device_mode(l + n) for s, l in zip(samplers, lens)]
        ahead = chained.step_chained(ids, modes, n % 2)     # launched before step n - 1 is taken
        if n == steps // 2:
            # (the capture of another kind of step for this very bucket runs a step of
            # padding through the buffers that hold the tokens in flight, and puts them back)
            assert chained.capture_decode_steps(sampled=False, max_batch=4) > 0
        got.append(wait())
        wait = ahead
    got.append(wait())
    assert got == want
    modes = [s.device_mode(l + steps) for s, l in zip(samplers, lens)]
    with pytest.raises(ValueError, match="same requests in the same order"):
        chained.step_chained([1, 0, 2], modes, 0)
    chained.step([StepEntry(i, [want[-1][i]], [0]) for i in ids])   # logits, through the bucket
    for i in ids:
        chained.reserve(i, lens[i] + steps + 2)
    with pytest.raises(ValueError, match="same requests in the same order"):
        chained.step_chained(ids, modes, 0)


def test_capture_beside_the_garbage_of_an_earlier_runner(case):
    """A runner that has captured graphs is dropped while it sits in a reference cycle, so that
    only the cyclic collector can free it, and the collector is off: real garbage with HIP
    graphs, pinned buffers and events in it exists when the next runner captures.  Capture
    collects it *before* the stream starts capturing (destroying such objects under a capturing
    stream is refused by HIP), so the first capture of the second runner is the moment the
    first runner dies."""
    import gc
    import weakref
    name, cfg, per_dtype = case
    folder, reqs, ref = per_dtype["float32"]
    steps, max_tokens = traces.trace_tail(reqs)
    gc.collect()
    gc.disable()
    try:
        first = make_runner(folder, "float32", max_tokens, 16, use_graphs=True)
        traces.replay_in_process(first, steps)
        assert first._graphs
        first.myself = first                      # a cycle: reference counting cannot free it
        alive = weakref.ref(first)
        del first
        assert alive() is not None                # garbage, not yet collected
        second = make_runner(folder, "float32", max_tokens, 16, use_graphs=True)
        assert alive() is not None                # still there when the second runner is built
        outputs = traces.replay_in_process(second, steps)
        assert second._graphs
        assert alive() is None                    # collected on the way into the capture
    finally:
        gc.enable()
    check(steps, outputs, reqs, ref, cfg["vocab_size"], TOL["float32"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_of_a_sequence(case, dtype):
    """Sequences fed one token at a time from position 0 (no prompt step before them), two of
    them side by side and a third that joins later, through captured and through eager decode
    steps: the first positions of a sequence meet an empty cache, a page with one key, and
    partitions without keys."""
    name, cfg, per_dtype = case
    folder, reqs, ref = per_dtype[dtype]
    keys = [k for k, t in reqs.items() if len(t) >= 17][:3]
    small = {k: reqs[k][:17] for k in keys}
    steps = []
    for p in range(17 + 5):
        entries = []
        for i, k in enumerate(keys):
            q = p - (5 if i == 2 else 0)                # the third joins five steps later
            if 0 <= q < 17:
                entries.append({"id": k, "tokens": [small[k][q]], "want": [0]})
        end = [e["id"] for e in entries if (p - (5 if e["id"] == keys[2] else 0)) == 16]
        steps.append({"step": p, "entries": entries, "end": end})
    for use_graphs in (True, False):
        runner = make_runner(folder, dtype, 3 * 64, page_size=8 if name == "b" else 16,
                             use_graphs=use_graphs)
        outputs = traces.replay_in_process(runner, steps)
        small_ref = {k: ref[k][:17] for k in keys}
        check(steps, outputs, small, small_ref, cfg["vocab_size"], TOL[dtype])
        assert runner.cache.num_free_pages(0) == runner.cache.num_pages(0)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_fork_then_both_decode(case, dtype):
    """A request that has reserved far ahead (as the scheduler does at admission) is forked in
    the middle of a page; parent and child go on with different tokens, side by side in the
    same steps, across the next page's edge.  Each must see the shared past and its own
    continuation only: the first write of either into the shared page goes to a copy."""
    from rust_llm_inference_server_amd.engine import StepEntry
    name, cfg, per_dtype = case
    folder, reqs, ref = per_dtype[dtype]
    page = 8 if name == "b" else 16
    tokens = reqs["r3"]                               # 100 tokens (fewer where positions are)
    split = page * 2 + 3                              # in the middle of the third page
    tail = min(len(tokens) - split, page + 6)         # past that page's end
    w, c = plain.read_weights(folder), plain.read_config(folder)
    other = [(t + 1) % cfg["vocab_size"] for t in tokens[split:split + tail]]
    want_parent = ref["r3"]
    want_child = plain.forward(w, c, tokens[:split] + other)
    runner = make_runner(folder, dtype, 4 * 128, page_size=page)
    runner.reserve(0, split + tail)                   # the whole known length at once
    runner.step([StepEntry(0, tokens[:split], [])])
    free_before = runner.cache.num_free_pages(0)
    runner.fork(0, 1)
    assert runner.cache.num_free_pages(0) == free_before          # a fork allocates nothing
    shared = runner.cache.table(0)[:3]
    assert runner.cache.table(1) == shared
    for t in range(tail):
        runner.reserve(0, split + t + 1)
        runner.reserve(1, split + t + 1)
        if t == 0:
            # the parent got a copy of the half-full page, the child keeps the original alone
            assert runner.cache.table(0)[2] != shared[2] and runner.cache.table(1)[2] == shared[2]
            assert runner.cache.table(0)[:2] == runner.cache.table(1)[:2] == shared[:2]
        logits = runner.step([StepEntry(0, [tokens[split + t]], [0]),
                              StepEntry(1, [other[t]], [0])]).float().cpu()
        assert (logits[0] - want_parent[split + t]).abs().max().item() < TOL[dtype], f"parent at {t}"
        assert (logits[1] - want_child[split + t]).abs().max().item() < TOL[dtype], f"child at {t}"
    runner.cache.check_invariants()
    runner.free(0)
    runner.free(1)
    assert runner.cache.num_free_pages(0) == runner.cache.num_pages(0)


LONG = {
    "architectures": ["LlamaForCausalLM"], "hidden_size": 128, "intermediate_size": 176,
    "num_hidden_layers": 2, "num_attention_heads": 8, "num_key_value_heads": 2, "head_dim": 64,
    "vocab_size": 301, "rms_norm_eps": 1e-5, "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                     "high_freq_factor": 4.0, "original_max_position_embeddings": 1024},
    "max_position_embeddings": 4096, "tie_word_embeddings": True,
}


@pytest.mark.parametrize("use_graphs", [False, True], ids=["eager", "graphs"])
def test_decode_logits_do_not_depend_on_the_neighbours(tmp_path, use_graphs):
    """bfloat16, contexts on both sides of a decode partition's length (1,024 keys): the logits
    of a decoding request are bit for bit the same alone in its steps as beside two others, and
    the same from captured steps as from eager ones.  A request's context is cut by its own
    length, the products run the same kernel for 1 and for 3 rows, and a block's output is
    rounded once whichever kernel made it.  Nor do they depend on how many workgroups share a
    context's partitions (what the attention picks by the size of the batch): with one
    workgroup for both partitions of the long context, the same bits."""
    folder = make_model_folder(tmp_path / "long", LONG, seed=6, dtype=torch.bfloat16)
    reqs = traces.random_requests(LONG["vocab_size"], [1500 + 8, 40 + 8, 1020 + 8], seed=5)
    keys = sorted(reqs)

    def run(groups, graphs):
        """Prefill every request whole and alone, then 8 decode steps with the requests of each
        group together; logits by (request, step)."""
        runner = make_runner(folder, "bfloat16", 3 * 1600, page_size=16, use_graphs=graphs)
        from rust_llm_inference_server_amd.engine import StepEntry
        out = {}
        for i, k in enumerate(keys):
            runner.reserve(i, len(reqs[k]))
            runner.step([StepEntry(i, reqs[k][:-8], [])])
        for t in range(8):
            for group in groups:
                logits = runner.step([StepEntry(i, [reqs[keys[i]][len(reqs[keys[i]]) - 8 + t]], [0])
                                      for i in group])
                for row, i in enumerate(group):
                    out[(i, t)] = logits[row].clone()
        return out

    from rust_llm_inference_server_amd import ops
    together = run([[0, 1, 2]], use_graphs)
    alone = run([[0], [1], [2]], use_graphs)
    other = run([[2, 0], [1]], not use_graphs)
    old = ops.DECODE_WALK
    try:
        ops.DECODE_WALK = 2
        walked = run([[0, 1, 2]], use_graphs)
    finally:
        ops.DECODE_WALK = old
    for key in together:
        assert torch.equal(together[key], alone[key]), f"request {key[0]} step {key[1]}: alone"
        assert torch.equal(together[key], other[key]), f"request {key[0]} step {key[1]}: other mode"
        assert torch.equal(together[key], walked[key]), f"request {key[0]} step {key[1]}: walked"
    w, c = plain.read_weights(folder), plain.read_config(folder)
    for i, k in enumerate(keys):
        ref = plain.forward(w, c, reqs[k])
        for t in range(8):
            assert (together[(i, t)].cpu() - ref[len(reqs[k]) - 8 + t]).abs().max().item() < TOL["bfloat16"]


def test_two_runners_decode_on_two_streams_at_once(tmp_path):
    """Two runners over one model, each on a stream and a thread of its own, decode contexts of
    several partitions at the same time.  The decode attention merges a sequence's partitions
    inside the kernel and counts the workgroups' arrivals in memory that each runner owns, so
    neither counts into the other's: both give, step for step and bit for bit, what they give
    one after the other, and both leave their counters at zero.  Their prompts run at the same
    time as well, through the library's products: each stream has a workspace of its own there,
    and the calls on the device's one handle take turns."""
    import threading
    from rust_llm_inference_server_amd.engine import ModelRunner, StepEntry, load_model
    folder = make_model_folder(tmp_path / "long", LONG, seed=6, dtype=torch.bfloat16)
    model = load_model(folder, "bfloat16", max_positions=4096)
    reqs = [traces.random_requests(LONG["vocab_size"], [2100 + 24, 3000 + 24, 1030 + 24], seed=s)
            for s in (5, 6)]
    steps = 24

    def decode(which, stream, out, barrier=None):
        with torch.cuda.stream(stream):
            runner = ModelRunner(model, num_pages=3 * 200, page_size=16, max_num_seqs=4,
                                 use_graphs=False)
            keys = sorted(reqs[which])
            if barrier is not None:
                barrier.wait(timeout=60)         # the prompts run at the same time too
            for i, k in enumerate(keys):
                runner.reserve(i, len(reqs[which][k]))
                runner.step([StepEntry(i, reqs[which][k][:-steps], [])])
            stream.synchronize()
            if barrier is not None:
                barrier.wait(timeout=60)
            rows = []
            for t in range(steps):
                logits = runner.step([StepEntry(i, [reqs[which][k][len(reqs[which][k]) - steps + t]], [0])
                                      for i, k in enumerate(keys)])
                rows.append(logits)
            stream.synchronize()
            out[which] = (torch.stack(rows).cpu(), int(runner.pools.counters.abs().sum()))

    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    apart, together = {}, {}
    for which in (0, 1):
        decode(which, streams[which], apart)
    barrier = threading.Barrier(2)
    threads = [threading.Thread(target=decode, args=(w, streams[w], together, barrier)) for w in (0, 1)]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=120)
    assert all(not th.is_alive() for th in threads) and set(together) == {0, 1}
    for which in (0, 1):
        assert apart[which][1] == 0 and together[which][1] == 0
        assert torch.equal(together[which][0], apart[which][0]), f"runner {which}"
    assert not torch.equal(apart[0][0], apart[1][0])


@pytest.mark.parametrize("wide", [False, True], ids=["tiles64", "tiles128"])
def test_long_prompt_whole_and_in_portions(tmp_path, wide):
    """A prompt of 2,600 tokens in one step and in portions of 512 and 200 beside a decoding
    request, bfloat16: the long walks over cached keys take the prefill attention's forms for
    them (keys cut into runs and merged; tiles of 128 queries), which tiny prompts never reach.
    One key far back is made to stand out for the last token, so that a lost run would show."""
    from rust_llm_inference_server_amd import ops
    folder = make_model_folder(tmp_path / "long", LONG, seed=5, dtype=torch.bfloat16)
    w, c = plain.read_weights(folder), plain.read_config(folder)
    reqs = traces.random_requests(LONG["vocab_size"], [2600, 40], seed=4)
    reqs["r0"][-1] = reqs["r0"][700]                      # the last token meets itself far back
    ref = {k: plain.forward(w, c, t) for k, t in reqs.items()}
    long_t, short_t = reqs["r0"], reqs["r1"]
    steps = [{"step": 0, "entries": [{"id": "whole", "tokens": long_t, "want": [0, 1299, 2599]}],
              "end": ["whole"]},
             {"step": 1, "entries": [{"id": "r1", "tokens": short_t[:30], "want": []}], "end": []}]
    pos, dec = 0, 30
    for n in [512, 200] * 4:
        n = min(n, len(long_t) - pos)
        if n == 0:
            break
        entries = [{"id": "r0", "tokens": long_t[pos:pos + n], "want": [0, n - 1]}]
        if dec < len(short_t):
            entries.append({"id": "r1", "tokens": [short_t[dec]], "want": [0]})
            dec += 1
        steps.append({"step": len(steps), "entries": entries, "end": []})
        pos += n
    assert pos == len(long_t)
    steps[-1]["end"] = ["r0", "r1"]
    from rust_llm_inference_server_amd.ops import attention_plan
    old, call = attention_plan.PREFILL_WIDE_MIN_GROUPS, ops.lib.call
    seen = []                 # (tile_queries, stride of the runs' results) of every prefill launch

    def spy(name, *args):
        if name == "rlis_attn_prefill_mfma":
            seen.append((args[18], args[19]))
        return call(name, *args)

    try:
        attention_plan.PREFILL_WIDE_MIN_GROUPS = 0 if wide else 1 << 30
        ops.lib.call = spy
        runner = make_runner(folder, "bfloat16", 2 * 2624 + 64, page_size=16)
        outputs = traces.replay_in_process(runner, steps)
    finally:
        attention_plan.PREFILL_WIDE_MIN_GROUPS, ops.lib.call = old, call
    assert any(runs > 1 for _, runs in seen) and any(runs == 1 for _, runs in seen)
    assert {tq for tq, _ in seen} == ({128} if wide else {64})
    whole = outputs[0]
    want = ref["r0"]
    assert (whole - want[[0, 1299, 2599]]).abs().max().item() < TOL["bfloat16"]
    pos, dec = 0, 30
    for st in steps[2:]:
        n = len(st["entries"][0]["tokens"])
        got = outputs[st["step"]]
        assert (got[:2] - want[[pos, pos + n - 1]]).abs().max().item() < TOL["bfloat16"], f"portion at {pos}"
        if len(st["entries"]) > 1:
            assert (got[2] - ref["r1"][dec]).abs().max().item() < TOL["bfloat16"], f"decoded token {dec}"
            dec += 1
        pos += n
    assert runner.cache.num_free_pages(0) == runner.cache.num_pages(0)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(case, dtype, tmp_path):
    """The program itself, as a child process fed step by step, on the mixed trace."""
    name, cfg, per_dtype = case
    folder, reqs, ref = per_dtype[dtype]
    steps, max_tokens = traces.trace_mixed(reqs, seed=1)
    outputs = traces.replay_program(folder, dtype, steps, max_tokens, str(tmp_path / "out"),
                                    cfg["vocab_size"])
    check(steps, outputs, reqs, ref, cfg["vocab_size"], TOL[dtype])


def test_mixed_trace_uses_pages_again():
    reqs = traces.random_requests(100, LENGTHS, seed=3)
    steps, peak = traces.trace_mixed(reqs)
    assert peak < sum(traces.rounded(len(t)) for t in reqs.values())
    assert any(len(s["entries"]) > 1 and {len(e["tokens"]) for e in s["entries"]} - {1}
               and 1 in {len(e["tokens"]) for e in s["entries"]} for s in steps)
