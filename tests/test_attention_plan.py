"""The attention kernels' per-step plan (``ops/attention_plan.py``), on the host: what a
sequence gets (tile form, key runs, the depth of the decode grid) follows from its own lengths
and from constants, never from its neighbours; every tile of every portion is listed once per
run; and the kernels' partition rule matches the host's."""
import numpy as np
import pytest

from rust_llm_inference_server_amd.ops import attention_plan as ap
from rust_llm_inference_server_amd.stepplan import StepLengths


def lengths(cached, new, page_size=16):
    single = 0
    for n in new:
        if n != 1:
            break
        single += 1
    return StepLengths(np.asarray(cached, dtype=np.int64), np.asarray(new, dtype=np.int64), single,
                       page_size)


def units_of(plan, name):
    return [tuple(u) for u in plan.arrays[name].reshape(-1, 4).tolist()]


def test_every_tile_is_listed_once_per_run_and_longest_first():
    planner = ap.AttentionPlanner(32, 8, 64)
    cached, new = [10, 300, 0, 40, 3000, 100], [1, 1, 300, 70, 200, 5000]
    plan = planner.plan(lengths(cached, new))
    assert plan.values["num_decode"] == 2 and plan.values["tile_row0"] == 2
    runs = plan.arrays["seq_runs"].tolist()
    assert runs[:2] == [1, 1]
    seen = {}
    for tile, name in ((64, "units64"), (128, "units128")):
        units = units_of(plan, name)
        assert len(units) == plan.values["num_" + name]
        work = []
        for s, qb, r, nr in units:
            assert s >= 2 and nr == runs[s] and 0 <= r < nr and qb % tile == 0 and qb < new[s]
            assert planner.tile_queries(cached[s], new[s]) == tile
            seen.setdefault((s, qb), []).append(r)
            work.append(-(-(cached[s] + min(new[s], qb + tile)) // nr))
        assert work == sorted(work, reverse=True)
    for s in range(2, 6):
        tile = planner.tile_queries(cached[s], new[s])
        for qb in range(0, new[s], tile):
            assert sorted(seen.pop((s, qb))) == list(range(runs[s]))
    assert not seen
    assert plan.values["max_runs"] == max(runs)
    # the short portion on a long context is cut into runs, the long prompt is not
    assert runs[4] > 1 and runs[5] == 1
    assert planner.tile_queries(3000, 200) == 128 and planner.tile_queries(0, 300) == 64


def test_a_sequence_is_planned_the_same_alone_and_among_neighbours():
    rng = np.random.default_rng(0)
    for nh, nkv, d in ((32, 8, 64), (24, 8, 128), (6, 2, 32), (16, 2, 256)):
        planner = ap.AttentionPlanner(nh, nkv, d)
        for _ in range(20):
            S = int(rng.integers(1, 9))
            new = sorted((int(rng.choice([1, 1, 2, 17, 64, 200, 513, 3000])) for _ in range(S)),
                         key=lambda n: n != 1)
            cached = [int(rng.choice([0, 5, 1023, 1024, 2047, 2048, 4095, 9000])) for _ in range(S)]
            both = planner.plan(lengths(cached, new))
            for s in range(S):
                if new[s] == 1:
                    continue
                one = planner.plan(lengths([cached[s]], [new[s]]))
                assert one.arrays["seq_runs"].tolist() == [both.arrays["seq_runs"][s]]
                for name in ("units64", "units128"):
                    mine = sorted((qb, r, nr) for q, qb, r, nr in units_of(both, name) if q == s)
                    assert mine == sorted((qb, r, nr) for _, qb, r, nr in units_of(one, name))


def test_decode_partitions_follow_the_sequence_alone():
    assert ap.decode_parts(1) == 1 and ap.decode_parts(1024) == 1 and ap.decode_parts(1025) == 2
    assert ap.decode_parts(16 * 1024) == 16 and ap.decode_parts(16 * 1024 + 1) == 9
    assert ap.decode_parts(131072) == 16
    assert ap.decode_depth(700) == 1 and ap.decode_depth(4096) == 4 and ap.decode_depth(1 << 20) == 16
    for ctx in (1, 999, 1024, 5000, 16384, 16385, 40000, 131072):
        assert ap.decode_parts(ctx) <= ap.decode_depth(ctx)
    planner = ap.AttentionPlanner(32, 8, 64)
    plan = planner.plan(lengths([0, 4999, 20], [1, 1, 1]))
    assert plan.values["num_decode"] == 3 and plan.values["decode_depth"] == 5
    assert plan.values["num_units64"] == plan.values["num_units128"] == 0
    fixed = planner.plan_captured(8, 2048, 16)
    assert not fixed.arrays and fixed.values["decode_depth"] == 2 and fixed.values["num_decode"] == 8


def test_partitions_are_dealt_out_by_how_far_the_batch_fills_the_chip():
    """(workgroups per sequence and KV head, most partitions in one): a workgroup per partition
    where sequences times KV heads leave compute units idle, one workgroup for all of them
    where the batch fills the chip by itself; never more in one than the LDS holds parked sums
    for, and one each unless partitions are whole pairs of chunks."""
    units = 256
    # 8 sequences x 8 KV heads: 64 of them want 4 workgroups each at head size 128, 8 at 64
    assert ap.decode_shares(8, 8, 4, 4, 128, units) == (4, 1)
    assert ap.decode_shares(8, 8, 8, 4, 128, units) == (4, 2)
    assert ap.decode_shares(8, 8, 5, 4, 128, units) == (4, 2)     # 5 partitions: 1, 1, 1, 2
    assert ap.decode_shares(8, 8, 8, 4, 64, units) == (8, 1)
    # 64 x 8 fill the chip: one workgroup takes a sequence's partitions, as far as the LDS goes
    assert ap.decode_shares(64, 8, 2, 3, 128, units) == (1, 2)
    assert ap.decode_shares(64, 8, 4, 4, 64, units) == (1, 4)
    assert ap.decode_shares(32, 8, 16, 4, 128, units) == (1, 9)   # 16.6 KB of parked sums each
    assert ap.decode_shares(32, 8, 16, 3, 128, units) == (1, 13)
    assert ap.decode_shares(64, 8, 16, 4, 64, units) == (1, 7)    # 8.4 KB each, in 64 KB
    assert ap.decode_shares(64, 8, 16, 16, 256, units) == (16, 1)  # 132 KB each: none to spare
    assert ap.decode_shares(1, 8, 16, 4, 64, units) == (16, 1)
    assert ap.decode_shares(64, 8, 1, 4, 64, units) == (1, 1)
    for seqs in (1, 3, 8, 24, 64, 300):
        for depth in range(1, 17):
            for group, d in ((1, 48), (4, 64), (3, 128), (4, 128), (8, 128), (4, 256)):
                groups, cap = ap.decode_shares(seqs, 8, depth, group, d, units)
                assert 1 <= groups <= depth and 1 <= cap <= depth
                assert cap == 1 or cap * 8 * group * (d + 2) * 4 <= (64 if d <= 64 else 159) * 1024
                assert groups == depth if cap == 1 else groups * cap >= depth or cap < depth
    old = ap.DECODE_PART_KEYS
    try:
        ap.DECODE_PART_KEYS = 768                             # a chunk and a half per wave
        assert ap.decode_shares(64, 8, 4, 4, 64, units) == (4, 1)
    finally:
        ap.DECODE_PART_KEYS = old


def test_layouts_the_matrix_kernels_do_not_take_plan_no_tiles():
    # float32, or pages that are no power of two: only the depth of the decode grid is planned
    for planner, ps in ((ap.AttentionPlanner(4, 1, 16, matrix=False), 16),
                        (ap.AttentionPlanner(4, 1, 16), 12),
                        (ap.AttentionPlanner(4, 1, 24), 16)):
        plan = planner.plan(lengths([5, 0], [1, 40], ps))
        assert plan.values["num_units64"] == plan.values["num_units128"] == 0
        assert plan.values["num_decode"] == 0
    # 17 query heads per KV head are more than the decode kernel takes: single tokens get tiles
    wide_group = ap.AttentionPlanner(34, 2, 16)
    plan = wide_group.plan(lengths([5, 0], [1, 40]))
    assert plan.values["num_decode"] == 0 and plan.values["num_units64"] == 2
    assert plan.values["tile_row0"] == 0
