"""The bookkeeping of captured steps other than decode steps (engine/graph.py::RepeatedSteps),
on the CPU with the capture itself replaced: when a shape is captured, which one is dropped,
and that a shape whose capture is refused stays eager."""
from types import SimpleNamespace

import pytest
import torch

from rust_llm_inference_server_amd.engine.graph import RepeatedSteps


class FakeRunner:
    pass


class FakeGraph:
    def __init__(self):
        self.replays = 0

    def replay(self):
        self.replays += 1


def fake_step(start, new, rows=1, slots=None, tokens=None):
    n = sum(new)
    return SimpleNamespace(buffer=torch.arange(16 + n, dtype=torch.int32), over=lambda b: None,
                           num_tokens=n if tokens is None else tokens, host_start_pos=list(start),
                           host_new=list(new), host_state_slots=list(slots or [0] * len(new)),
                           num_logit_rows=rows)


def steps_with_fake_captures(**kw):
    runner = FakeRunner()
    rs = RepeatedSteps(runner, **kw)
    rs._keep = runner                      # (the steps hold their runner weakly)
    made = []

    def capture(shape, step):
        while len(rs.graphs) >= rs.limit:
            rs.graphs.popitem(last=False)
        held = rs.graphs[shape] = (FakeGraph(), torch.zeros_like(step.buffer), object())
        made.append(shape)
        return held
    rs._capture = capture
    return rs, made


def test_a_shape_is_captured_when_it_has_come_back_often_enough():
    rs, made = steps_with_fake_captures()
    a, b = fake_step([0], [40]), fake_step([40], [40])
    for i in range(RepeatedSteps.CAPTURE_AT - 1):
        assert rs.run(a) is None and rs.run(b) is None
    assert not made
    out = rs.run(a)
    assert out is not None and made == [RepeatedSteps.shape_of(a)] and rs.replays == 1
    graph, buffer, logits = rs.graphs[made[0]]
    assert out is logits and graph.replays == 1 and torch.equal(buffer, a.buffer)
    again = fake_step([0], [40])
    again.buffer += 7                       # other data, same shape
    assert rs.run(again) is logits and graph.replays == 2 and torch.equal(buffer, again.buffer)
    assert len(made) == 1


def test_what_makes_two_steps_one_shape():
    shape = RepeatedSteps.shape_of
    base = fake_step([0, 16], [8, 1], rows=2, slots=[0, 1])
    assert shape(base) == shape(fake_step([0, 16], [8, 1], rows=2, slots=[0, 1]))
    for other in (fake_step([0, 17], [8, 1], rows=2, slots=[0, 1]),      # cached positions
                  fake_step([0, 16], [7, 1], rows=2, slots=[0, 1]),      # new tokens
                  fake_step([0, 16], [8, 1], rows=1, slots=[0, 1]),      # wanted rows
                  fake_step([0, 16], [8, 1], rows=2, slots=[0, 2])):     # a state slot
        assert shape(base) != shape(other)


def test_the_least_recently_used_shape_is_dropped(monkeypatch):
    monkeypatch.setattr(RepeatedSteps, "CAPTURE_AT", 1)
    rs, made = steps_with_fake_captures(limit=2)
    a, b, c = (fake_step([0], [n]) for n in (3, 4, 5))
    assert rs.run(a) is not None and rs.run(b) is not None
    assert rs.run(a) is not None                 # a is now the more recently used
    assert rs.run(c) is not None                 # ... so b goes
    assert list(rs.graphs) == [RepeatedSteps.shape_of(a), RepeatedSteps.shape_of(c)]
    assert rs.run(b) is not None and len(made) == 4


def test_long_steps_and_steps_without_one_buffer_stay_eager(monkeypatch):
    monkeypatch.setattr(RepeatedSteps, "CAPTURE_AT", 1)
    rs, made = steps_with_fake_captures(max_tokens=100)
    assert rs.run(fake_step([0], [101])) is None
    loose = fake_step([0], [5])
    loose.buffer = None
    assert rs.run(loose) is None and not made
    assert rs.run(fake_step([0], [100])) is not None


def test_a_shape_whose_capture_is_refused_stays_eager():
    rs = RepeatedSteps(runner := FakeRunner())
    tried = []

    def refuse(shape, step):
        tried.append(shape)
        raise RuntimeError("operation not permitted when stream is capturing")
    rs._capture = refuse
    step = fake_step([0], [5])
    for i in range(RepeatedSteps.CAPTURE_AT - 1):
        assert rs.run(step) is None
    with pytest.warns(UserWarning, match="stays eager"):
        assert rs.run(step) is None
    for i in range(3 * RepeatedSteps.CAPTURE_AT):
        assert rs.run(step) is None
    assert len(tried) == 1 and not rs.graphs and runner is not None


def test_the_rule_for_slices_of_k_follows_from_rows_and_k_alone():
    """How the library's product over a long k is cut into slices when its consumer takes partial
    sums (ops.library_slices): eight slices up to 256 rows, four up to 1,024, two up to 2,048,
    fewer where k does not divide into slices of whole 16-byte pieces; one product below 65
    rows, beyond 2,048 and for a short k."""
    from rust_llm_inference_server_amd import ops
    cut = ops.library_slices
    assert [cut(t, 8192) for t in (64, 65, 256, 257, 1024, 1025, 2048, 2049)] == [1, 8, 8, 4, 4, 2, 2, 1]
    assert [cut(t, 14336) for t in (100, 300, 1500)] == [8, 4, 2]
    assert cut(512, 4096) == 1 and cut(512, 8192 + 8) == 1
    assert cut(100, 8192 + 32) == 4 and cut(100, 8192 + 16) == 2 and cut(300, 8192 + 16) == 2
    for t in (65, 200, 512, 2000):
        for k in (8192, 8200, 8208, 11008, 14336, 28672):
            n = cut(t, k)
            assert k % n == 0 and (k // n) % 8 == 0
