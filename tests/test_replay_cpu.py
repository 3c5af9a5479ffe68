"""The host side of the engine (batch layout, block tables, page manager, run order) under
every way of cutting the work, with the kernels replaced by a slow torch double on the CPU.
The kernels themselves are tested on the GPU (test_kernels_gpu.py, test_replay_gpu.py)."""
import pytest
import torch

import plain_llama as plain
import traces
from conftest import TINY


@pytest.fixture(scope="module")
def ref_a(tiny_folders):
    folder = tiny_folders["a"]
    w, c = plain.read_weights(folder), plain.read_config(folder)
    reqs = traces.random_requests(c["vocab_size"], [5, 17, 33, 70, 1, 2, 64, 90], seed=3)
    return folder, reqs, {k: plain.forward(w, c, t) for k, t in reqs.items()}


@pytest.mark.parametrize("family", ["whole", "tail", "portions", "mixed"])
def test_replay_families_cpu(cpu_ops, ref_a, family):
    from rust_llm_inference_server_amd.engine import ModelRunner, load_model
    folder, reqs, ref = ref_a
    build = {"whole": traces.trace_whole, "tail": traces.trace_tail,
             "portions": traces.trace_portions, "mixed": traces.trace_mixed}[family]
    steps, max_tokens = build(reqs)
    model = load_model(folder, "float32", max_positions=128, device=torch.device("cpu"))
    runner = ModelRunner(model, num_pages=max_tokens // 16, page_size=16, max_num_seqs=8)
    outputs = traces.replay_in_process(runner, steps)
    got = traces.collect(steps, outputs, TINY["a"]["vocab_size"])
    for k, tokens in reqs.items():
        mine = torch.stack([got[k][p] for p in range(len(tokens))])
        assert (mine - ref[k]).abs().max().item() < 1e-4
    assert runner.cache.num_free_pages(0) == runner.cache.num_pages(0)


def test_step_errors(cpu_ops, tiny_folders):
    """The step's refusals (crates/model/src/llama.rs:218-240; paged.rs:258-263)."""
    from rust_llm_inference_server_amd.engine import ModelRunner, StepEntry, load_model
    model = load_model(tiny_folders["a"], "float32", max_positions=64, device=torch.device("cpu"))
    runner = ModelRunner(model, num_pages=8, page_size=16, max_num_seqs=2)
    with pytest.raises(ValueError, match="at least one request"):
        runner.step([])
    runner.reserve(1, 4)
    with pytest.raises(ValueError, match="empty sequence"):
        runner.step([StepEntry(1, [], [])])
    with pytest.raises(ValueError, match="no page reserved"):
        runner.step([StepEntry(1, [1, 2, 3, 4, 5], [])])
    with pytest.raises(ValueError, match="no page reserved"):
        runner.step([StepEntry(9, [1], [])])
    with pytest.raises(ValueError, match="outside the vocabulary"):
        runner.step([StepEntry(1, [256], [])])
    with pytest.raises(ValueError, match="wanted index"):
        runner.step([StepEntry(1, [1, 2], [2])])
    with pytest.raises(ValueError, match="appears twice"):
        runner.step([StepEntry(1, [1], []), StepEntry(1, [2], [])])
    with pytest.raises(ValueError, match="exceeds max_seq_len"):
        runner.reserve(1, 65)
    runner.reserve(2, 1)
    with pytest.raises(ValueError, match="max_num_seqs"):
        runner.step([StepEntry(1, [1], []), StepEntry(2, [1], []), StepEntry(3, [1], [])])
    out = runner.step([StepEntry(1, [1, 2], [1]), StepEntry(2, [3], [])])
    assert out.shape == (1, 256)
    assert runner.num_computed(1) == 2 and runner.num_computed(2) == 1


def test_step_layout_puts_single_tokens_first(cpu_ops, tiny_folders):
    """Inside a step the requests that bring one token come first (their rows are the first
    rows, so that a decode kernel can take them beside the portions); the logits come back in
    the order of the entries and of their `want` all the same."""
    from rust_llm_inference_server_amd.engine import ModelRunner, StepEntry, build_step, load_model
    model = load_model(tiny_folders["a"], "float32", max_positions=128, device=torch.device("cpu"))
    runner = ModelRunner(model, num_pages=16, page_size=16, max_num_seqs=8)
    for seq, n in ((1, 40), (2, 9), (3, 70), (4, 5)):
        runner.reserve(seq, n)
    runner.step([StepEntry(2, list(range(8)), []), StepEntry(4, [7, 8, 9, 10], [])])
    entries = [StepEntry(1, list(range(10, 43 - 3)), [0, 29]), StepEntry(2, [5], [0]),
               StepEntry(3, list(range(70)), [69]), StepEntry(4, [6], [])]
    step = build_step(entries, runner.cache, torch.device("cpu"), 256, model.step_planners)
    assert step.host_order == [1, 3, 0, 2] and step.num_single == 2 and not step.all_decode
    assert step.host_new == [1, 1, 30, 70] and step.host_start_pos == [8, 4, 0, 0]
    assert step.max_context == 70
    assert step.lengths.start.tolist() == [8, 4, 0, 0] and step.lengths.num_single == 2
    assert step.ids.tolist()[:2] == [5, 6] and step.positions.tolist()[:3] == [8, 4, 0]
    assert step.cu_seqlens.tolist() == [0, 1, 2, 32, 102]
    assert step.logit_rows.tolist() == [2, 31, 0, 101]            # entry order, then want order
    # the attention mixer's plan rides along (a float32 model plans no tiles, only the depth of
    # the decode grid), under the key of its planner
    (planner,) = model.step_planners
    plan = step.plans[planner.key()]
    assert plan.value("num_units64") == 0 and plan.value("decode_depth") == 1
    assert plan["seq_runs"].tolist() == [1, 1, 1, 1]
    # and the runner's answer does not depend on the order the entries come in
    want = runner.step(entries)
    assert [runner.num_computed(s) for s in (1, 2, 3, 4)] == [30, 9, 70, 5]
    for seq in (1, 2, 3, 4):
        runner.free(seq)
    for seq, n in ((1, 40), (2, 9), (3, 70), (4, 5)):
        runner.reserve(seq, n)
    runner.step([StepEntry(4, [7, 8, 9, 10], []), StepEntry(2, list(range(8)), [])])
    again = runner.step([entries[2], entries[3], entries[1], entries[0]])
    assert (again[[2, 3, 1, 0]] - want).abs().max().item() < 1e-5


def test_no_collection_holds_the_cyclic_collector_off():
    """What graph capture runs under: garbage is collected before the block, none inside it
    (not even at the lowest thresholds), and the collector is back afterwards."""
    import gc
    import weakref
    from rust_llm_inference_server_amd.engine.graph import no_collection

    class Node:
        pass

    def cycle():
        a, b = Node(), Node()
        a.other, b.other = b, a
        return weakref.ref(a)

    before = cycle()
    thresholds = gc.get_threshold()
    gc.set_threshold(1, 1, 1)
    try:
        with no_collection():
            assert before() is None and not gc.isenabled()
            inside = cycle()
            junk = [[i] for i in range(2000)]            # allocations that would trigger a pass
            assert inside() is not None
            del junk
        assert gc.isenabled()
        gc.collect()
        assert inside() is None
    finally:
        gc.set_threshold(*thresholds)
