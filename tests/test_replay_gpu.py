"""The engine against the plain implementation, request by request and position by position,
under every way of cutting the work: whole prompts; most of a prompt in one step and the last
32 tokens one by one; portions of changing size down to two tokens; and up to four live
requests mixed, portions of some beside single tokens of others, with so few pages that they
are used again.  In float32 (the true 32-bit path) and in bfloat16, for three tiny
configurations that differ in every size and option."""
import os

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
    # every page came back
    assert runner.cache.num_free_pages(0) == runner.cache.num_pages(0)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_captured_decode_steps_match_eager_ones(case, dtype):
    """Steps of one token per request run from a captured HIP graph.  Replayed many times with
    eager steps (prefill portions, page copies, host synchronisation) in between, every replay
    must give what the eager step gives."""
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
            torch.testing.assert_close(out_g[k], out_e[k], atol=TOL[dtype] / 4, rtol=0)


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
def test_trace_run_program(case, dtype, tmp_path):
    """The program itself, as a child process fed step by step, on the mixed trace."""
    name, cfg, per_dtype = case
    if name == "c":
        pytest.skip("one configuration less through the child process keeps the suite short")
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
