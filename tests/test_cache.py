"""The cache's bookkeeping on the host: no slot or page lost, held twice or freed twice."""
import random

import pytest
import torch

from braidinfer_amd.cache import CacheNeed, PagePool, SequenceCache, SlotAllocator, StateNeed
from braidinfer_amd.errors import CacheError


def test_pool_gives_every_page_once_then_fails():
    # reference behaviour: alloc all, then exhaustion is an error; a freed page comes back
    # first (LIFO, paged_kv.rs:1126-1180)
    pool = PagePool(5)
    got = pool.alloc(5)
    assert sorted(got) == [0, 1, 2, 3, 4] and pool.free_count == 0
    with pytest.raises(CacheError, match="out of cache pages"):
        pool.alloc(1)
    pool.free([got[2]])
    assert pool.alloc(1) == [got[2]]


def test_pool_alloc_is_all_or_nothing():
    pool = PagePool(4)
    pool.alloc(3)
    with pytest.raises(CacheError):
        pool.alloc(2)
    assert pool.free_count == 1


def test_pool_rejects_double_and_foreign_frees():
    pool = PagePool(3)
    a = pool.alloc(2)
    pool.free([a[0]])
    with pytest.raises(CacheError, match="twice"):
        pool.free([a[0]])
    with pytest.raises(CacheError, match="outside"):
        pool.free([7])
    with pytest.raises(CacheError, match="twice"):
        pool.free([a[1], a[1]])
    assert pool.held_count == 1          # the failed frees changed nothing


def test_slots():
    s = SlotAllocator(2)
    a, b = s.alloc(), s.alloc()
    assert {a, b} == {0, 1}
    with pytest.raises(CacheError, match="out of sequence slots"):
        s.alloc()
    s.free(a)
    with pytest.raises(CacheError, match="twice"):
        s.free(a)
    with pytest.raises(CacheError, match="not live"):
        s.check_live(a)
    assert s.alloc() == a               # used again


def _cache(window=None, max_tokens=64 * 6, **kw):
    needs = {0: CacheNeed(2, 16, window), 1: CacheNeed(2, 16, window), 2: CacheNeed(2, 16, None)}
    return SequenceCache(needs, {}, max_tokens=max_tokens, dtype=None, device="cpu", **kw)


def test_groups_gather_units_with_equal_needs():
    c = _cache(window=100)
    assert [g.unit_ids for g in c.groups] == [[0, 1], [2]]
    assert c.unit_group(0) is c.unit_group(1) and c.unit_group(2) is not c.unit_group(0)
    c2 = _cache(window=None)
    assert [g.unit_ids for g in c2.groups] == [[0, 1, 2]]


def test_reserve_grows_pages_and_tables_and_commit_sets_lengths():
    c = _cache()
    s = c.alloc_slot()
    c.reserve([s], [70])
    g = c.groups[0]
    assert len(g.pages[s]) == 2 and list(g.table_cpu[s, :2]) == g.pages[s] and g.table_cpu[s, 2] == -1
    assert c.length(s) == 0
    c.commit([s], [70])
    assert c.length(s) == 70
    c.reserve([s], [58])
    assert len(g.pages[s]) == 2          # 128 tokens still fit two pages
    c.commit([s], [58])
    c.reserve([s], [1])
    assert len(g.pages[s]) == 3


def test_reserve_is_atomic_over_the_batch():
    c = _cache(max_tokens=64 * 3)
    a, b = c.alloc_slot(), c.alloc_slot()
    with pytest.raises(CacheError, match="out of cache pages"):
        c.reserve([a, b], [100, 100])
    assert all(g.pool.held_count == 0 for g in c.groups) and c.length(a) == 0
    c.reserve([a, b], [100, 60])
    assert c.groups[0].pool.held_count == 3
    with pytest.raises(CacheError, match="twice"):
        c.reserve([a, a], [1, 1])


def test_free_slot_returns_everything_and_slots_are_used_again():
    c = _cache()
    a = c.alloc_slot()
    c.reserve([a], [200]); c.commit([a], [200])
    held = c.groups[0].pool.held_count
    assert held == 4
    c.free_slot(a)
    assert c.groups[0].pool.held_count == 0 and torch.all(c.groups[0].table_cpu == -1)
    with pytest.raises(CacheError, match="twice"):
        c.free_slot(a)
    with pytest.raises(CacheError, match="not live"):
        c.reserve([a], [1])
    b = c.alloc_slot()
    assert b == a and c.length(b) == 0


def test_window_group_returns_pages_behind_the_window():
    c = _cache(window=70, max_tokens=64 * 8)
    s = c.alloc_slot()
    gw, gf = c.groups
    c.reserve([s], [300]); c.commit([s], [300])
    # the next query sits at 300 and sees keys 231..300: pages 0..2 (tokens < 192) are dead
    assert gw.first_page[s] == 3 and gw.pages[s][:3] == [-1, -1, -1] and gw.pool.held_count == 2
    assert gf.pool.held_count == 5
    assert list(gw.table_cpu[s, :3]) == [-1, -1, -1]
    for _ in range(100):
        c.reserve([s], [1]); c.commit([s], [1])
    assert c.length(s) == 400 and gw.pool.held_count <= 3
    c.free_slot(s)
    assert gw.pool.held_count == 0 and gf.pool.held_count == 0


def test_longest_sequence_is_enforced():
    c = _cache(max_tokens=64 * 8, max_seq_len=128)
    s = c.alloc_slot()
    with pytest.raises(CacheError, match="longest"):
        c.reserve([s], [129])
    c.reserve([s], [128])


def test_state_area_is_zeroed_for_a_new_owner():
    c = SequenceCache({}, {"m": StateNeed((3, 2), torch.float32), "n": StateNeed((5,), torch.int32)},
                      max_tokens=128, dtype=None, device="cpu")
    a = c.alloc_slot()
    c.state("m")[a] += 7.0
    c.state("n")[a] += 3
    assert c.state("m").shape == (2, 3, 2) and float(c.state("m")[a].sum()) == 42.0
    c.free_slot(a)
    b = c.alloc_slot()
    assert b == a and float(c.state("m")[b].abs().sum()) == 0.0 and int(c.state("n")[b].sum()) == 0
    assert c.state("absent") is None


def test_random_walk_never_loses_or_doubles_a_page():
    rng = random.Random(3)
    c = _cache(window=90, max_tokens=64 * 40)
    live = {}
    for _ in range(600):
        op = rng.random()
        if op < 0.25 and c.slots.free_count:
            live[c.alloc_slot()] = 0
        elif op < 0.45 and live:
            s = rng.choice(list(live)); c.free_slot(s); del live[s]
        elif live:
            pick = rng.sample(list(live), rng.randint(1, len(live)))
            new = [rng.choice([1, 1, 1, 17, 64, 130]) for _ in pick]
            try:
                c.reserve(pick, new)
            except CacheError:
                continue
            c.commit(pick, new)
            for s, n in zip(pick, new):
                live[s] += n
        for g in c.groups:
            held = [p for s in range(c.n_slots) for p in g.pages[s] if p >= 0]
            assert len(held) == len(set(held)) == g.pool.held_count          # none held twice, none lost
            assert sorted(held + g.pool._free) == list(range(g.pool.n_pages))
        for s, n in live.items():
            assert c.length(s) == n
            for g in c.groups:
                lo = 0 if g.need.window is None else max(0, n - g.need.window + 1) // 64
                assert all(p >= 0 for p in g.pages[s][lo:-(-n // 64)])        # every visible page is there
    for s in list(live):
        c.free_slot(s)
    assert all(g.pool.held_count == 0 for g in c.groups)


def test_a_need_with_a_rule_of_its_own_gives_back_what_the_rule_says():
    """`CacheNeed.live_from`: here chunks of 128 tokens, of which only the running one stays visible (the rule
    of a mixer that attends within chunks): when a sequence enters a new chunk, the pages of the chunk before
    go back; a group with the window's rule beside it is untouched by that."""
    chunk = lambda n: (n // 128) * 128
    needs = {0: CacheNeed(2, 16, live_from=chunk), 1: CacheNeed(2, 16, live_from=chunk), 2: CacheNeed(2, 16, 100)}
    c = SequenceCache(needs, {}, max_tokens=64 * 12, dtype=None)
    assert len(c.groups) == 2 and c.groups[0].unit_ids == [0, 1]
    assert needs[0].first_live(127) == 0 and needs[0].first_live(128) == 128 and needs[0].first_live(300) == 256
    assert CacheNeed(2, 16, 100).first_live(150) == 51 and CacheNeed(2, 16).first_live(150) == 0
    gc, gw = c.groups
    s = c.alloc_slot()
    for n in (100, 27, 1, 127, 130):                                          # lengths 100, 127, 128, 255, 385
        c.reserve([s], [n]); c.commit([s], [n])
        first = chunk(c.lengths[s]) // 64
        assert gc.pool.held_count == len(gc.pages[s]) - first and gc.first_page[s] == first
        assert all(p == -1 for p in gc.pages[s][:first]) and all(p >= 0 for p in gc.pages[s][first:])
        assert (gc.table_cpu[s, :first] == -1).all()
    assert gw.pool.held_count == 3                                            # 385 tokens, the last 100: pages 4 to 6
    c.free_slot(s)
    assert gc.pool.held_count == 0 and gw.pool.held_count == 0
