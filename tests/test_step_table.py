"""The reference's hand-written step table (crates/model/src/paged.rs:397-445): its tiny
configuration, its two token lists, its deliberately scattered block tables ``[9, 2, 14, 5]`` and
``[0, 11, 7, 3]`` with 4 positions a page in a pool of 16 pages, and its four steps (a prompt
beside the first part of another; the rest of that one beside a single token; a single token
alone; three tokens alone).  Every step's last-row logits must equal the whole-sequence
logits of the plain implementation within the reference's 1e-4.

The page manager hands out pages in its own order, so the tables are given to the step builder
through a stand-in that answers what the manager would."""
import pytest
import torch

import plain_llama as plain
from conftest import make_model_folder

BACKENDS = ["double", pytest.param("gpu", marks=pytest.mark.gpu)]

# LlamaConfig::tiny (crates/model/src/config.rs:55-72)
REFERENCE_TINY = {
    "architectures": ["LlamaForCausalLM"], "hidden_size": 64, "intermediate_size": 128,
    "num_hidden_layers": 2, "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 16,
    "vocab_size": 97, "rms_norm_eps": 1e-5, "rope_theta": 10000.0, "rope_scaling": None,
    "max_position_embeddings": 128, "tie_word_embeddings": True, "bos_token_id": 1,
}
A = [1, 5, 9, 33, 2, 70, 41, 8, 96, 3, 4]
B = [7, 7, 60, 12, 13]
TABLES = {0: [9, 2, 14, 5], 1: [0, 11, 7, 3]}
STEPS = [[(0, 6), (0, 3)], [(6, 7), (3, 5)], [(7, 8), (5, 5)], [(8, 11), (5, 5)]]


class FixedTables:
    """Answers the step builder as the page manager would, with block tables that are given."""

    class Group:
        window = None

    def __init__(self, page_size, tables):
        self.page_size, self.tables = page_size, tables
        self.num_groups, self.groups = 1, [self.Group()]
        self.computed = {k: 0 for k in tables}

    def contains(self, seq):
        return seq in self.tables

    def _get_info(self, seq):
        return len(self.tables[seq]) * self.page_size, self.computed[seq], -1

    def table(self, seq, group=0):
        return list(self.tables[seq])


@pytest.fixture(params=BACKENDS)
def device(request):
    if request.param == "double":
        import cpu_ops
        cpu_ops.install(request.getfixturevalue("monkeypatch"))
        return torch.device("cpu")
    return torch.device("cuda", 0)


def test_the_references_step_table(device, tmp_path):
    from rust_llm_inference_server_amd.cache.pools import CachePools
    from rust_llm_inference_server_amd.engine import StepEntry, build_step, load_model
    folder = make_model_folder(tmp_path / "ref_tiny", REFERENCE_TINY, seed=0)
    w, c = plain.read_weights(folder), plain.read_config(folder)
    want = {0: plain.forward(w, c, A), 1: plain.forward(w, c, B)}
    model = load_model(folder, "float32", max_positions=64, device=device)
    pools = CachePools(model.cache_groups, [16], 4, torch.float32, device)
    cache = FixedTables(4, TABLES)
    tokens = {0: A, 1: B}
    for step in STEPS:
        entries, rows = [], []
        for seq, (s, e) in enumerate(step):
            if s == e:
                continue
            entries.append(StepEntry(seq, tokens[seq][s:e], [e - s - 1]))
            rows.append((seq, e - 1))
        ctx = build_step(entries, cache, device, 97, model.step_planners)
        logits = model.forward(ctx, pools).cpu()
        for row, (seq, pos) in enumerate(rows):
            diff = (logits[row] - want[seq][pos]).abs().max().item()
            assert diff < 1e-4, f"step {step}: sequence {seq} position {pos}: logit diff {diff}"
        for seq, (s, e) in enumerate(step):
            cache.computed[seq] = e
    # the pages the tables name hold the keys, and no other page was written
    k = pools.arrays[0]["k"][0]
    used = sorted(TABLES[0][:3] + TABLES[1][:2])          # 11 and 5 positions of 4 a page
    written = [p for p in range(16) if k[p].abs().sum().item() > 0]
    assert written == used


def test_the_runtimes_step_layout_is_the_python_twins():
    """The host runtime lays a step's common arrays out exactly as ``build_step_in_python``
    does: random steps (single tokens among portions, windows that have given pages back, state
    slots, wanted rows in the entries' order) over two page groups, array by array; and the same
    complaints about steps that cannot run."""
    import numpy as np
    from rust_llm_inference_server_amd.cache.manager import CacheManager, GroupSpec
    from rust_llm_inference_server_amd.engine import StepEntry, build_step
    from rust_llm_inference_server_amd.ops.attention_plan import AttentionPlanner
    from rust_llm_inference_server_amd.stepplan import HostPlan, StepPlanner

    class Wordy(StepPlanner):
        """A planner whose arrays outgrow the room the builder keeps for plans."""

        def key(self):
            return "wordy"

        def plan(self, lengths):
            n = int(lengths.new.sum())
            return HostPlan({"many": np.arange(5000 + n, dtype=np.int32),
                             "few": np.asarray(lengths.start, dtype=np.int32)}, {"n": n})

    rng = np.random.default_rng(7)
    cache = CacheManager(8, [GroupSpec(400, None), GroupSpec(400, 24)], num_state_slots=16)
    cpu = torch.device("cpu")
    planners = [AttentionPlanner(4, 2, 16), Wordy()]
    lengths = {}
    for trial in range(40):
        live = list(lengths)
        for seq in rng.permutation(live)[:rng.integers(0, 3)]:
            cache.free(int(seq))
            del lengths[int(seq)]
        while len(lengths) < 6:
            lengths[int(rng.integers(0, 10_000))] = 0
        entries = []
        for seq in rng.permutation(list(lengths))[:rng.integers(1, 6)]:
            seq = int(seq)
            n = int(rng.choice([1, 1, 1, 2, 5, 17, 40]))
            cache.reserve(seq, lengths[seq] + n)
            want = sorted({int(w) for w in rng.integers(0, n, size=rng.integers(0, 3))})
            entries.append(StepEntry(seq, rng.integers(0, 97, size=n).tolist(), want))
        a = build_step(entries, cache, cpu, 97, planners, native=True)
        b = build_step(entries, cache, cpu, 97, planners, native=False)
        for name in ("ids", "positions", "seq_of_token", "cu_seqlens", "start_pos", "ctx_lens",
                     "logit_rows", "state_slots"):
            assert torch.equal(getattr(a, name), getattr(b, name)), (trial, name)
        for ga, gb in zip(a.groups, b.groups):
            assert torch.equal(ga.block_tables, gb.block_tables) and torch.equal(ga.slots, gb.slots)
            assert (ga.page_size, ga.window) == (gb.page_size, gb.window)
        for field in ("num_tokens", "num_seqs", "num_logit_rows", "max_context", "max_new",
                      "all_decode", "num_single", "host_start_pos", "host_new",
                      "host_state_slots", "host_order"):
            assert getattr(a, field) == getattr(b, field), (trial, field)
        assert a.plans.keys() == b.plans.keys()
        for key in a.plans:
            assert a.plans[key].values == b.plans[key].values
            for name in a.plans[key].arrays:
                assert torch.equal(a.plans[key][name], b.plans[key][name]), (trial, name)
        for e in entries:
            lengths[e.seq_id] += len(e.tokens)
            cache.advance(e.seq_id, lengths[e.seq_id])
    seq = next(iter(lengths))
    cache.reserve(seq, lengths[seq] + 4)
    for native in (True, False):
        for bad, message in (([], "at least one request"),
                             ([StepEntry(seq, [], [])], "empty sequence"),
                             ([StepEntry(123456, [1], [])], "no page reserved"),
                             ([StepEntry(seq, [1] * 5, [])], "no page reserved"),
                             ([StepEntry(seq, [1, 97], [])], "outside the vocabulary"),
                             ([StepEntry(seq, [1, -1], [])], "outside the vocabulary"),
                             ([StepEntry(seq, [1, 2], [2])], "wanted index"),
                             ([StepEntry(seq, [1], []), StepEntry(seq, [2], [])], "appears twice")):
            with pytest.raises(ValueError, match=message):
                build_step(bad, cache, cpu, 97, planners, native=native)
