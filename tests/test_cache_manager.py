"""The page manager: vectors the reference's tests hold (crates/kvcache/src/lib.rs:445-502),
its property test (lib.rs:570-636) under random orders of requests with hypothesis, and the
parts the reference lacks: windowed groups that give pages back early, several groups, and
state slots.  After every operation: no page lost, held twice or freed twice."""
import pytest
from hypothesis import given, settings
from hypothesis import strategies as st

from rust_llm_inference_server_amd.cache import CacheManager, GroupSpec, OutOfPages, PageCopy


def test_reserve_grows_by_whole_pages():
    m = CacheManager(4, [GroupSpec(8)])
    m.reserve(1, 5)
    assert len(m.table(1)) == 2
    m.reserve(1, 8)
    assert len(m.table(1)) == 2
    m.reserve(1, 9)
    assert len(m.table(1)) == 3 and m.num_free_pages() == 5
    m.free(1)
    assert m.num_free_pages() == 8


def test_pages_come_lifo_with_page_zero_first():
    m = CacheManager(4, [GroupSpec(8)])
    m.reserve(1, 12)
    assert m.table(1) == [0, 1, 2]                  # lib.rs:75: (0..n).rev() so 0 pops first
    m.reserve(2, 4)
    m.free(1)
    m.reserve(3, 8)
    assert m.table(3) == [2, 1]                     # the pages freed last are used again first
    m.check_invariants()


def test_out_of_pages_changes_nothing():
    m = CacheManager(4, [GroupSpec(2)])
    m.reserve(1, 4)
    with pytest.raises(OutOfPages):
        m.reserve(1, 13)
    assert m.num_tokens(1) == 4 and m.num_free_pages() == 1
    m.check_invariants()


def test_fork_shares_and_writes_copy_on_write():
    """lib.rs:470-502, with the positions computed (a fork shares what is computed)."""
    m = CacheManager(4, [GroupSpec(8)])
    m.reserve(1, 6)
    m.advance(1, 6)
    assert m.fork(1, 2) == (-1, -1)                 # no state slots to copy
    assert m.num_free_pages() == 6                  # fork allocates nothing
    assert m.num_tokens(2) == 6 and m.num_computed(2) == 6
    shared_last = m.table(1)[1]
    copies = m.reserve(2, 7)                        # writes into the shared, half-full last page
    mine = m.table(2)[1]
    assert copies == [PageCopy(0, shared_last, mine)] and mine != shared_last
    assert m.table(2)[0] == m.table(1)[0]           # the full page stays shared
    assert m.reserve(1, 7) == []                    # request 1 now owns its last page alone
    m.check_invariants()


def test_full_shared_pages_need_no_copy():
    m = CacheManager(4, [GroupSpec(8)])
    m.reserve(1, 8)
    m.advance(1, 8)
    m.fork(1, 2)
    assert m.reserve(2, 9) == []
    assert m.pages_needed(1, 9) == 1


def test_fork_of_a_request_that_reserved_ahead():
    """The scheduler reserves a request's whole known length at admission, far ahead of what is
    computed.  A fork shares the computed positions only; the page both will write next is
    copied for whichever of the two reserves a range that touches it, the parent included,
    although the parent had that page reserved all along."""
    m = CacheManager(4, [GroupSpec(8)], num_state_slots=3)
    m.reserve(1, 14)                                # pages 0..3
    m.advance(1, 6)
    parent_slot = m.state_slot(1)
    assert m.fork(1, 2) == (parent_slot, m.state_slot(2)) and m.state_slot(2) != parent_slot
    assert m.table(2) == m.table(1)[:2] and m.num_tokens(2) == 6
    assert m.refcount(0, m.table(1)[1]) == 2 and m.refcount(0, m.table(1)[2]) == 1
    assert m.pages_needed(1, 7) == 1                # the parent's next write lands in a shared page
    before = m.table(1)
    copies = m.reserve(1, 7)                        # within what it had reserved: still a copy
    assert copies == [PageCopy(0, before[1], m.table(1)[1])] and m.num_tokens(1) == 14
    assert m.reserve(2, 9) == [] and len(m.table(2)) == 3      # the child's page is its own now
    m.check_invariants()
    m.free(1)
    m.free(2)
    assert m.num_free_pages() == 8 and m.num_free_slots() == 3


def test_window_group_gives_pages_back_as_the_window_passes():
    m = CacheManager(4, [GroupSpec(16), GroupSpec(16, window=6)])
    m.reserve(1, 20)
    assert m.num_free_pages(0) == 11 and m.num_free_pages(1) == 11
    m.advance(1, 9)       # the next query, at position 9, sees keys 4..9: page 0 (0..3) is dead
    assert m.table(1, 1) == [-1, 1, 2, 3, 4] and m.num_free_pages(1) == 12
    m.advance(1, 19)      # position 19 sees 14..19: pages 0..2 are dead
    assert m.table(1, 1)[:3] == [-1, -1, -1] and m.num_free_pages(1) == 14
    assert m.table(1, 0) == [0, 1, 2, 3, 4]         # the full group keeps everything
    m.check_invariants()
    m.reserve(2, 12)                                # freed pages are used again
    assert set(m.table(2, 1)) == {2, 1, 0}
    m.reserve(1, 24)
    assert len(m.table(1, 1)) == 6 and m.table(1, 1)[5] >= 0
    m.free(1)
    m.free(2)
    assert m.num_free_pages(0) == 16 and m.num_free_pages(1) == 16
    m.check_invariants()


def test_window_longer_than_the_sequence_keeps_everything():
    m = CacheManager(8, [GroupSpec(4, window=100)])
    m.reserve(1, 30)
    m.advance(1, 30)
    assert m.table(1) == [0, 1, 2, 3]


def test_all_groups_or_none():
    m = CacheManager(4, [GroupSpec(8), GroupSpec(2, window=4)])
    with pytest.raises(OutOfPages):
        m.reserve(1, 12)                            # the small group cannot hold 3 pages
    assert not m.contains(1) and m.num_free_pages(0) == 8 and m.num_free_pages(1) == 2
    m.check_invariants()


def test_state_slots_are_taken_and_returned():
    m = CacheManager(4, [GroupSpec(8)], num_state_slots=2)
    m.reserve(1, 1)
    m.reserve(2, 1)
    assert {m.state_slot(1), m.state_slot(2)} == {0, 1} and m.num_free_slots() == 0
    with pytest.raises(OutOfPages, match="state slots"):
        m.reserve(3, 1)
    assert not m.contains(3) and m.num_free_pages() == 6
    slot = m.state_slot(1)
    m.free(1)
    m.reserve(3, 1)
    assert m.state_slot(3) == slot                  # so few slots that they are used again
    m.check_invariants()


def test_unknown_requests():
    m = CacheManager(4, [GroupSpec(4)])
    m.free(99)                                      # ignored (lib.rs:356-364)
    with pytest.raises(KeyError):
        m.table(99)
    with pytest.raises(ValueError):
        m.advance(99, 1)
    m.reserve(1, 3)
    with pytest.raises(ValueError, match="past the reserved"):
        m.advance(1, 4)


OPS = st.one_of(
    st.tuples(st.just("reserve"), st.integers(0, 5), st.integers(1, 19)),
    st.tuples(st.just("reserve"), st.integers(0, 5), st.integers(1, 19)),
    st.tuples(st.just("advance"), st.integers(0, 5), st.integers(0, 100)),
    st.tuples(st.just("fork"), st.integers(0, 5), st.integers(0, 5)),
    st.tuples(st.just("free"), st.integers(0, 5), st.just(0)),
)


@settings(max_examples=400, deadline=None)
@given(ops=st.lists(OPS, min_size=1, max_size=60), page=st.integers(1, 5),
       window=st.sampled_from([None, 1, 3, 7]), slots=st.sampled_from([0, 4, 8]))
def test_random_operations_keep_the_invariants(ops, page, window, slots):
    """lib.rs:570-636: random reserve / fork / free (and advance) never leak, free twice or
    break reference counts; a failed reservation changes nothing; freeing everything fills
    the pools again."""
    groups = [GroupSpec(12), GroupSpec(12, window=window)]
    m = CacheManager(page, groups, num_state_slots=slots)
    for kind, a, b in ops:
        if kind == "reserve":
            have = m.num_tokens(a) if m.contains(a) else 0
            before_free = [m.num_free_pages(g) for g in range(2)]
            before_tables = [m.table(a, g) for g in range(2)] if m.contains(a) else None
            needed = [m.pages_needed(a, have + b, g) for g in range(2)]
            try:
                copies = m.reserve(a, have + b)
            except OutOfPages:
                assert (any(n > f for n, f in zip(needed, before_free))
                        or (before_tables is None and slots and m.num_free_slots() == 0))
                assert [m.num_free_pages(g) for g in range(2)] == before_free
                assert (m.contains(a) and [m.table(a, g) for g in range(2)] == before_tables) \
                    or (not m.contains(a) and before_tables is None)
            else:
                assert [bf - m.num_free_pages(g) for g, bf in enumerate(before_free)] == needed
                assert len(copies) <= 2 and m.num_tokens(a) == have + b
                for g in range(2):
                    # every page the new positions land in is this request's alone
                    for p in m.table(a, g)[have // page:]:
                        assert p < 0 or m.refcount(g, p) == 1
        elif kind == "advance":
            if m.contains(a):
                m.advance(a, min(b, m.num_tokens(a)))
        elif kind == "fork":
            if m.contains(a) and not m.contains(b) and (slots == 0 or m.num_free_slots() > 0):
                m.fork(a, b)
        else:
            m.free(a)
        m.check_invariants()
    for seq in range(6):
        m.free(seq)
    assert m.num_free_pages(0) == 12 and m.num_free_pages(1) == 12
    assert m.num_free_slots() == slots
    m.check_invariants()


# ------------------------------------------------------------------ the pools' sizing rule
class _Layout:
    """What the pools look at of a model's page group: its cache request and its layer slots."""

    def __init__(self, request, slots):
        self.request, self.writer_runs = request, list(range(slots))


def test_pools_are_sized_per_group_from_their_own_bytes_and_window():
    """All groups keep everything: the reference's rule, budget / bytes of one page across all
    groups (crates/engine/src/engine.rs:252-262).  A windowed group is capped at what
    ``max_num_seqs`` requests can hold of it (window + one step + a page each) but holds one
    request of the longest length, and the groups that keep everything get what that leaves."""
    import torch
    from rust_llm_inference_server_amd.cache.pools import CachePools, pool_pages
    from rust_llm_inference_server_amd.parts.base import PAGE, CacheRequest, PageArray
    full = _Layout(CacheRequest.kv(2, 16), slots=3)                  # 3 layers of K and V
    bf16, f32 = torch.bfloat16, torch.float32
    per_token = 3 * 2 * 2 * 16
    budget = 1 << 20
    assert pool_pages([full], bf16, 16, budget, 8, 64, 512) == [budget // (per_token * 2 * 16)]
    assert pool_pages([full], f32, 16, budget, 8, 64, 512) == [budget // (per_token * 4 * 16)]
    assert pool_pages([], bf16, 16, budget, 8, 64, 512) == []
    # a page array with a dtype of its own is counted by it
    latent = _Layout(CacheRequest((PageArray("latent", (PAGE, 20), dtype=f32),)), slots=2)
    assert latent.request.bytes_per_token(bf16) == latent.request.bytes_per_token(f32) == 80
    both = pool_pages([full, latent], bf16, 16, budget, 8, 64, 512)
    assert both == [budget // ((per_token * 2 + 2 * 80) * 16)] * 2
    # a window of 32 in one layer: 8 requests x (ceil((32 + 64) / 16) + 1) = 56 pages, but one
    # request of 2,048 positions needs 129; the full group gets what is left of the budget
    win = _Layout(CacheRequest.kv(2, 16, window=32), slots=1)
    budget = 4 << 20
    pages = pool_pages([full, win], bf16, 16, budget, 8, 64, 2048)
    even = budget // ((per_token + 2 * 2 * 16) * 2 * 16)
    assert even > 129 and pages[1] == 129
    assert pages[0] == (budget - 129 * (2 * 2 * 16) * 2 * 16) // (per_token * 2 * 16) > even
    assert pool_pages([full, win], bf16, 16, budget, 8, 64, 128)[1] == 56
    # never more than an even split would give the windowed group
    assert pool_pages([full, win], bf16, 16, 1 << 16, 8, 64, 2048)[1] == (1 << 16) // (
        (per_token + 2 * 2 * 16) * 2 * 16)
    # the pools follow: each group its own count (+ one scratch page), each array its own dtype
    pools = CachePools([full, latent, win], [7, 5, 3], 16, bf16, torch.device("cpu"))
    assert pools.arrays[0]["k"].shape == (3, 8, 2, 16, 16) and pools.arrays[0]["k"].dtype == bf16
    assert pools.arrays[0]["v"].shape == (3, 8, 2, 16, 16)
    assert pools.arrays[1]["latent"].shape == (2, 6, 16, 20) and pools.arrays[1]["latent"].dtype == f32
    assert pools.arrays[2]["k"].shape == (1, 4, 2, 16, 16)
    assert pools.scratch_pages == [7, 5, 3]
    assert pools.bytes_per_page(1) == 2 * 16 * 20 * 4 and pools.bytes_per_page(0) == per_token * 2 * 16
    with pytest.raises(ValueError, match="dtype"):
        PageArray("x", (PAGE, 4), dtype="float32")
