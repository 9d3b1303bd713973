"""The cache manager without a GPU: no page lost, held twice or freed twice, under random
orders of requests; windows return pages; appends are atomic."""

import pytest
from hypothesis import given, settings
from hypothesis import strategies as st

from llmserve.cache import BlockAllocator, CacheManager, OutOfBlocks, group_layers
from llmserve.parts.spec import PagedCacheSpec, StateCacheSpec


def test_allocator_contract():
    # the reference's own cases (tests/test_paged.py:21-30)
    a = BlockAllocator(3)
    got = [a.allocate() for _ in range(3)]
    assert sorted(got) == [0, 1, 2]
    with pytest.raises(OutOfBlocks):
        a.allocate()
    a.free([got[0]])
    with pytest.raises(ValueError):
        a.free([got[0]])
    with pytest.raises(ValueError):
        a.free([got[1], got[1]])  # twice in one call: nothing is freed
    assert a.num_used == 2
    # a freed page waits its turn behind the pages that are still free
    b = BlockAllocator(4)
    first = b.allocate()
    b.free([first])
    assert [b.allocate() for _ in range(4)] == [1, 2, 3, first]


@settings(max_examples=60, deadline=None)
@given(st.lists(st.tuples(st.booleans(), st.integers(0, 15)), max_size=200))
def test_allocator_never_duplicates(ops):
    a = BlockAllocator(16)
    held = []
    for alloc, k in ops:
        if alloc and a.num_free:
            held.append(a.allocate())
        elif held:
            a.free([held.pop(k % len(held))])
        assert a.num_free + a.num_used == 16 and len(set(held)) == len(held)
    a.free(held)
    assert a.num_free == 16


def full_groups(layers=2, window=None):
    return group_layers([PagedCacheSpec(2, 16, window)] * layers)


def test_groups_collect_layers_with_equal_needs():
    specs = [PagedCacheSpec(2, 16), PagedCacheSpec(2, 16, 8), None, PagedCacheSpec(2, 16), StateCacheSpec((4,)),
             PagedCacheSpec(2, 16, 8)]
    groups = group_layers(specs)
    assert [(g.layers, g.paged) for g in groups] == [((0, 3), True), ((1, 5), True), ((4,), False)]


def test_tables_slots_and_lengths():
    m = CacheManager(full_groups(), num_blocks=8, block_size=4, max_seqs=3)
    m.add_sequence("x")
    lay = m.append(["x"], [6])
    table = list(m.table(0, "x"))
    row = m.slot_of["x"]
    assert len(table) == 2 and lay.starts == [0] and m.lengths["x"] == 6
    assert lay.slots[0] == [table[p // 4] * 4 + p % 4 for p in range(6)]
    assert lay.table_updates[0] == [(row, 0, table[0]), (row, 1, table[1])]  # what the device copy is told
    lay = m.append(["x"], [3])  # crosses into a third page
    assert lay.starts == [6] and len(m.table(0, "x")) == 3 and m.table(0, "x")[:2] == table
    assert lay.table_updates[0] == [(row, 2, m.table(0, "x")[2])]
    assert m.append(["x"], [1]).table_updates[0] == []
    assert m.extra_blocks_needed("x", 2) == 0 and m.extra_blocks_needed("x", 3) == 1
    with pytest.raises(ValueError):
        m.add_sequence("x")
    m.free_sequence("x")
    assert m.num_free_blocks == 8 and m.num_free_slots == 3
    with pytest.raises(KeyError):
        m.free_sequence("x")


def test_append_is_atomic():
    # needing 3 of 2 pages raises and changes nothing (tests/test_paged.py:115-121)
    m = CacheManager(full_groups(), num_blocks=2, block_size=4, max_seqs=2)
    m.add_sequence(0)
    m.add_sequence(1)
    assert not m.can_append([0, 1], [4, 8]) and m.can_append([0, 1], [4, 4]) and m.can_append([1], [8])
    with pytest.raises(OutOfBlocks):
        m.append([0, 1], [4, 8])
    assert m.num_free_blocks == 2 and m.lengths == {0: 0, 1: 0}
    m.check_invariants()
    with pytest.raises(ValueError):
        m.append([0, 0], [1, 1])
    with pytest.raises(ValueError):
        m.append([0], [0])


def test_state_slots_are_unique_and_fresh_once():
    m = CacheManager(group_layers([StateCacheSpec((3,))]), num_blocks=1, block_size=4, max_seqs=2)
    a, b = m.add_sequence("a"), m.add_sequence("b")
    assert a != b
    with pytest.raises(OutOfBlocks):
        m.add_sequence("c")
    assert m.append(["a"], [2]).fresh_slots == [a]
    assert m.append(["a", "b"], [1, 1]).fresh_slots == [b]
    m.free_sequence("a")
    c = m.add_sequence("c")
    assert c == a and m.append(["c"], [1]).fresh_slots == [c]  # a slot that changes hands is cleared again


def test_window_pages_come_back_when_out_of_reach():
    m = CacheManager(group_layers([PagedCacheSpec(1, 16), PagedCacheSpec(1, 16, 6)]), num_blocks=8, block_size=4,
                     max_seqs=1)
    m.add_sequence("w")
    m.append(["w"], [13])
    assert m.release_passed(["w"]) == 2  # next query (13) sees keys >= 8: pages 0 and 1 are dead
    full, win = m.tables[0]["w"], m.tables[1]["w"]
    assert all(b >= 0 for b in full) and win[:2] == [-1, -1] and all(b >= 0 for b in win[2:])
    m.check_invariants()
    m.append(["w"], [1])
    assert m.release_passed(["w"]) == 0  # keys >= 9: page 2 (8..11) still in reach
    m.append(["w"], [6])  # length 20: keys >= 15
    assert m.release_passed(["w"]) == 1
    m.free_sequence("w")
    assert all(a.num_free == 8 for a in m.allocators.values())


def test_window_release_never_takes_a_reachable_key():
    bs, window = 4, 7
    m = CacheManager(group_layers([PagedCacheSpec(1, 16, window)]), num_blocks=64, block_size=bs, max_seqs=1)
    m.add_sequence(0)
    length = 0
    for n in [5, 1, 1, 9, 2, 1, 1, 1, 12, 1]:
        m.append([0], [n])
        table = m.table(0, 0)
        for p in range(length, length + n):  # every key a query of this step sees must still be held
            for j in range(max(0, p - window + 1), p + 1):
                assert table[j // bs] >= 0, (p, j)
        length += n
        m.release_passed([0])
        m.check_invariants()


@settings(max_examples=60, deadline=None)
@given(st.lists(st.tuples(st.integers(0, 3), st.integers(0, 5), st.integers(1, 30)), max_size=120),
       st.sampled_from([None, 5]))
def test_random_requests_keep_the_books(ops, window):
    m = CacheManager(group_layers([PagedCacheSpec(2, 16), PagedCacheSpec(2, 16, window)]), num_blocks=24,
                     block_size=4, max_seqs=4)
    for op, seq, n in ops:
        if op == 0 and not m.has_sequence(seq) and m.num_free_slots:
            m.add_sequence(seq)
        elif op == 1 and m.has_sequence(seq):
            m.free_sequence(seq)
        elif m.has_sequence(seq):
            before = (m.num_free_blocks, dict(m.lengths))
            try:
                m.append([seq], [n])
                m.release_passed([seq])
            except OutOfBlocks:
                assert (m.num_free_blocks, m.lengths) == before
        m.check_invariants()
        held = sum(a.num_used for a in m.allocators.values())
        assert held <= 2 * sum(m.blocks_for(length) for length in m.lengths.values())
        # wasted slots stay below one page per request and group (tests/test_paged.py:124-130)
        g0 = m.allocators[0].num_used * 4 - sum(m.lengths.values())
        assert 0 <= g0 < 4 * max(1, len(m.lengths)) or not m.lengths
    for seq in list(m.lengths):
        m.free_sequence(seq)
    assert all(a.num_free == 24 for a in m.allocators.values()) and m.num_free_slots == 4


def test_fragmentation_and_need_count_every_group():
    """One group keeps every key, one a window of 6: after 22 tokens in pages of 4 the first holds 6 pages
    (24 slots, 22 used), the second 2 pages after giving 4 back (8 slots, 6 of them live keys 16..21)."""
    m = CacheManager(group_layers([PagedCacheSpec(1, 16), PagedCacheSpec(1, 16, 6)]), num_blocks=16, block_size=4, max_seqs=2)
    m.add_sequence("r")
    m.append(["r"], [22])
    assert m.release_passed(["r"]) == 4
    assert [a.num_used for a in m.allocators.values()] == [6, 2]
    assert abs(m.internal_fragmentation() - (1 - (22 + 6) / (24 + 8))) < 1e-9
    assert m.extra_blocks_needed("r", 2) == 0 and m.extra_blocks_needed("r", 3) == 1 and m.extra_blocks_needed("r", 11) == 3
    m.free_sequence("r")
    assert m.internal_fragmentation() == 0.0


def test_sequence_lengths_give_table_lengths():
    # N sequences of 1..30 tokens with pages of 4 (tests/test_paged.py:56-68)
    m = CacheManager(full_groups(), num_blocks=64, block_size=4, max_seqs=8)
    for i, n in enumerate([1, 4, 5, 30, 17, 8]):
        m.add_sequence(i)
        m.append([i], [n])
        assert len(m.tables[0][i]) == m.blocks_for(n) == -(-n // 4)
    assert 0 < m.utilization() < 1 and 0 <= m.internal_fragmentation() < 1
    for i in range(6):
        m.free_sequence(i)
    assert m.num_free_blocks == 64


# ------------------------------------------------------------------ what a request costs, group by group
def test_pages_are_counted_per_group_and_pools_have_sizes_of_their_own():
    from llmserve.cache.manager import window_pages
    from llmserve.parts.spec import StateCacheSpec

    full, windowed, state = PagedCacheSpec(2, 16), PagedCacheSpec(2, 16, window=6), StateCacheSpec((5,), "float32")
    groups = group_layers([full, windowed, state, full])
    ids = {g.spec: g.group_id for g in groups}
    m = CacheManager(groups, {ids[full]: 10, ids[windowed]: 4}, block_size=4, max_seqs=3)
    assert m.capacity() == {ids[full]: 10, ids[windowed]: 4} and m.num_blocks == 4
    # 30 tokens: 8 pages where every key stays; with a window of 6 and portions of up to 4 tokens no more than
    # ceil((5 + 4) / 4) + 1 = 4; the state group costs no pages and is not named
    assert window_pages(6, 4, 4) == 4
    assert m.pages_for(30, step_tokens=4) == {ids[full]: 8, ids[windowed]: 4}
    assert m.pages_for(30) == {ids[full]: 8, ids[windowed]: 8} and m.pages_for(3, step_tokens=4) == {ids[full]: 1, ids[windowed]: 1}
    m.add_sequence("a")
    for _ in range(7):  # 28 tokens in portions of 4: the windowed group never holds more than its 4 pages
        m.append(["a"], [4])
        m.release_passed(["a"])
        assert m.allocators[ids[windowed]].num_used <= 4
        m.check_invariants()
    assert m.free_pages() == {ids[full]: 3, ids[windowed]: 2}
    assert m.pages_owed("a", 9) == {ids[full]: 3, ids[windowed]: 3}
    # many more tokens, in portions of 4: the windowed group is owed what brings the request to its most there
    assert m.pages_owed("a", 90, step_tokens=4) == {ids[full]: 23, ids[windowed]: 4 - m.allocators[ids[windowed]].num_used}
    assert not m.can_append(["a"], [9])  # the windowed group has 2
    with pytest.raises(OutOfBlocks, match=f"group {ids[windowed]}"):
        m.append(["a"], [9])
    m.free_sequence("a")
    assert m.free_pages() == m.capacity()
    with pytest.raises(ValueError, match="every paged group"):
        CacheManager(groups, {ids[full]: 10}, 4, 3)


def test_a_model_of_fixed_size_state_alone_has_no_pages_to_run_out_of():
    from llmserve.parts.spec import StateCacheSpec

    m = CacheManager(group_layers([StateCacheSpec((8,), "float32")] * 3), 1, block_size=16, max_seqs=2)
    assert m.capacity() == {} and m.pages_for(10_000, 64) == {} and m.free_pages() == {}
    m.add_sequence(0)
    assert m.pages_owed(0, 5000) == {} and m.can_append([0], [5000])
    layout = m.append([0], [5000])
    assert layout.slots == {} and m.lengths[0] == 5000 and m.utilization() == 0.0
    m.add_sequence(1)
    with pytest.raises(OutOfBlocks, match="state slots"):
        m.add_sequence(2)


def test_pools_are_sized_by_what_each_group_needs():
    from llmserve.cache.storage import page_bytes_of, pool_sizes_for_budget, state_bytes
    from llmserve.parts.spec import StateCacheSpec

    full, windowed, state = PagedCacheSpec(4, 64), PagedCacheSpec(4, 64, window=128), StateCacheSpec((1000,), "float32")
    groups = group_layers([full] * 30 + [windowed] * 2 + [state])
    by_spec = {g.spec: g for g in groups}
    fixed = state_bytes(groups, max_seqs=8)
    assert fixed == 8 * 1000 * 4
    budget = fixed + 50_000_000
    sizes = pool_sizes_for_budget(groups, 16, 2, budget, max_seqs=8, longest=4096, step_tokens=512)
    f, w = sizes[by_spec[full].group_id], sizes[by_spec[windowed].group_id]
    # both groups hold the same number of longest requests: 256 pages each in the full group, 41 in the windowed
    assert abs(f / 256 - w / 41) < 0.05 and w < f / 5
    spent = f * page_bytes_of(by_spec[full], 16, 2) + w * page_bytes_of(by_spec[windowed], 16, 2)
    assert 0.9 * 50_000_000 < spent <= 50_000_000
    # never more than all slots could fill; the state alone may already be too much
    roomy = pool_sizes_for_budget(groups, 16, 2, 10**12, max_seqs=8, longest=4096, step_tokens=512)
    assert roomy == {by_spec[full].group_id: 8 * 256, by_spec[windowed].group_id: 8 * 41}
    with pytest.raises(ValueError, match="fixed-size state"):
        pool_sizes_for_budget(groups, 16, 2, fixed - 1, max_seqs=8, longest=4096, step_tokens=512)
    assert pool_sizes_for_budget(group_layers([state]), 16, 2, budget, 8, 4096, 512) == {}
