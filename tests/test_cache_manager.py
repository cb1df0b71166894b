"""The cache manager (host code, no GPU): pages, block tables, windows, state
slots; no page lost, held twice or freed twice, under random orders of requests."""
import random

import pytest

from lyapunov_engine_amd.cache import CacheError, CacheManager, GroupConfig


def test_reference_vector_100_pages_32_tokens():
    # tests/test_block_manager.py:15-36 of the reference: 100 pages of 16, 32 tokens -> 2 pages -> free -> 100
    m = CacheManager([GroupConfig(100, 16)], 8)
    assert m.num_free_pages() == 100
    m.add(0)
    assert m.can_extend(0, 32)
    m.extend(0, 32)
    assert m.table(0) == [0, 1] and m.num_free_pages() == 98 and m.capacity(0) == 32 and m.length(0) == 0
    m.commit(0, 32)
    assert m.length(0) == 32
    m.free(0)
    assert m.num_free_pages() == 100 and m.num_requests() == 0
    m.free(0)  # unknown request: a no-op (block_manager.cpp:83-86)
    m.check()


def test_growth_by_any_number_of_tokens_and_fifo_reuse():
    m = CacheManager([GroupConfig(6, 4)], 4)
    m.add(1), m.add(2)
    m.extend(1, 5)                      # 2 pages
    m.extend(2, 1)                      # 1 page
    assert m.table(1) == [0, 1] and m.table(2) == [2]
    m.extend(1, 8)                      # still 2 pages: nothing new (the reference grows only when total % bs == 1)
    assert m.table(1) == [0, 1]
    m.extend(1, 9)
    assert m.table(1) == [0, 1, 3]
    m.free(1)                           # pages 0, 1, 3 go to the back of the queue: 4, 5, 0, 1, 3
    m.extend(2, 16)
    assert m.table(2) == [2, 4, 5, 0]   # first in, first out: the order of reuse is fixed
    assert not m.can_extend(2, 25) and m.can_extend(2, 24)
    with pytest.raises(CacheError, match="out of pages"):
        m.extend(2, 25)
    assert m.table(2) == [2, 4, 5, 0]   # a failed extend changes nothing
    assert m.max_length(2) == 24
    m.check()


def test_pages_for_several_requests_all_or_none():
    import numpy as np

    m = CacheManager([GroupConfig(6, 4), GroupConfig(5, 4)], 4)
    for i in (1, 2, 3):
        m.add(i)
        m.extend(i, 4)                  # one page each in both groups: 3 free in the first, 2 in the second
    ids = np.array([1, 2, 3], dtype=np.int64)
    assert m.reserve(ids, np.array([4, 3, 1], dtype=np.int32)) and m.num_free_pages(0) == 3   # held already
    assert not m.reserve(ids, np.array([5, 5, 5], dtype=np.int32))     # the second group has two pages only
    assert m.num_free_pages(0) == 3 and m.num_free_pages(1) == 2 and m.capacity(1) == 4
    assert m.reserve(ids, np.array([5, 4, 8], dtype=np.int32))
    assert m.capacity(1) == 5 and m.capacity(2) == 4 and m.capacity(3) == 8
    assert m.num_free_pages(0) == 1 and m.num_free_pages(1) == 0
    assert len(m.table(1)) == 2 and len(m.table(2)) == 1 and len(m.table(3, 1)) == 2
    m.check()
    for i in (1, 2, 3):
        m.free(i)
    assert m.num_free_pages(0) == 6 and m.num_free_pages(1) == 5
    m.check()


def test_errors():
    m = CacheManager([GroupConfig(4, 4)], 2)
    m.add(7)
    with pytest.raises(CacheError, match="already live"):
        m.add(7)
    m.add(8)
    with pytest.raises(CacheError, match="no free state slot"):
        m.add(9)
    assert not m.can_extend(9, 1)       # an unknown request also needs a slot
    m.extend(7, 4)
    with pytest.raises(CacheError, match="beyond the pages"):
        m.commit(7, 5)
    m.commit(7, 4)
    with pytest.raises(CacheError, match="shrink"):
        m.commit(7, 3)
    with pytest.raises(CacheError):
        m.length(99)
    with pytest.raises(CacheError):
        CacheManager([GroupConfig(0, 4)], 2)


def test_state_slots_are_given_back_and_reused():
    m = CacheManager([GroupConfig(8, 4)], 3)
    assert [m.add(i) for i in range(3)] == [0, 1, 2]
    m.free(1)
    assert m.add(5) == 1 and m.state_slot(5) == 1 and m.num_free_slots() == 0
    m.check()


def test_window_group_gives_pages_back_as_the_window_passes():
    # group 0 keeps everything; group 1 sees a window of 6 tokens, pages of 4
    m = CacheManager([GroupConfig(32, 4, 0), GroupConfig(5, 4, 6)], 2)
    m.add(0)
    held = []
    length = 0
    for step in range(40):
        n = 1 if step else 7            # a prompt of 7, then one token at a time
        m.extend(0, length + n)
        length += n
        m.commit(0, length)
        t = m.table(0, 1)
        # the next token, at position `length`, sees keys > length - 6: those pages must be there
        for pos in range(max(0, length - 6 + 1), length):
            assert t[pos // 4] >= 0, (length, pos, t)
        # pages wholly out of reach are gone
        for i, p in enumerate(t):
            if (i + 1) * 4 <= length - 6 + 1:
                assert p == -1, (length, i, t)
        held.append(sum(1 for p in t if p >= 0))
        m.check()
    assert max(held) <= 3               # never more than ceil((6 + 1) / 4) + 1 pages
    assert len(m.table(0, 0)) == -(-length // 4) and all(p >= 0 for p in m.table(0, 0))
    assert m.counters()["window_returns"] > 0
    # the window group has 5 pages only, yet the request grew to 46 tokens
    assert length == 46
    m.free(0)
    assert m.num_free_pages(0) == 32 and m.num_free_pages(1) == 5


def test_pages_given_back_by_a_window_are_taken_by_another_request():
    m = CacheManager([GroupConfig(4, 4, 4)], 2)
    m.add(0), m.add(1)
    m.extend(0, 8), m.commit(0, 8)      # pages 0, 1; first needed key 5 -> page 0 is returned
    assert m.table(0) == [-1, 1]
    m.extend(1, 12)                     # takes 2, 3, 0
    assert m.table(1) == [2, 3, 0]
    m.check()


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_keep_every_invariant(seed):
    rng = random.Random(seed)
    groups = [GroupConfig(rng.randint(8, 40), rng.choice([1, 2, 4, 16]), 0),
              GroupConfig(rng.randint(6, 20), rng.choice([2, 4, 8]), rng.choice([3, 8, 17]))]
    slots = rng.randint(2, 5)
    m = CacheManager(groups, slots)
    live, next_id = {}, 0
    for _ in range(600):
        op = rng.random()
        if op < 0.25 and len(live) < slots:
            m.add(next_id)
            live[next_id] = 0
            next_id += 1
        elif op < 0.8 and live:
            rid = rng.choice(list(live))
            new_len = live[rid] + rng.randint(1, 9)
            if m.can_extend(rid, new_len):
                before = [m.num_free_pages(g) for g in range(2)]
                m.extend(rid, new_len)
                assert all(m.num_free_pages(g) <= before[g] for g in range(2))
                m.commit(rid, new_len)
                live[rid] = new_len
            else:
                with pytest.raises(CacheError):
                    m.extend(rid, new_len)
        elif live:
            rid = rng.choice(list(live))
            m.free(rid)
            del live[rid]
            if rng.random() < 0.3:
                m.free(rid)             # twice: must not put pages in the free list twice
        m.check()
        # no page in two live tables
        for g in range(2):
            seen = [p for rid in live for p in m.table(rid, g) if p >= 0]
            assert len(seen) == len(set(seen))
            assert len(seen) + m.num_free_pages(g) == groups[g].num_pages
            assert all(m.ref_count(g, p) == 1 for p in seen)
        assert m.num_requests() == len(live) and m.num_free_slots() == slots - len(live)
    for rid in list(live):
        m.free(rid)
    assert [m.num_free_pages(g) for g in range(2)] == [g.num_pages for g in groups]
    m.check()
    c = m.counters()
    assert c["pages_taken"] == c["pages_returned"] and c["high_water"] > 0
    m.reset()
    assert m.num_free_slots() == slots


def test_tables_of_a_step_are_checked_and_filled():
    import numpy as np

    m = CacheManager([GroupConfig(8, 4), GroupConfig(8, 4, window=4)], 4)
    m.add(7), m.add(9)
    m.extend(7, 12)                      # pages 0, 1, 2
    m.commit(7, 8)                       # the window group has given its first page back
    m.extend(9, 3)                       # page 3
    ids = np.array([7, 9], dtype=np.int64)
    start, count = np.array([8, 0], dtype=np.int32), np.array([3, 2], dtype=np.int32)

    def tables(g, width=4, ids=ids, start=start, count=count):
        bt = np.full((len(ids), width), 99, dtype=np.int32)
        slot_map, slots = np.full(int(count.sum()), 99, dtype=np.int32), np.full(len(ids), 99, dtype=np.int32)
        m.step_tables(ids, start, count, g, bt, slot_map, slots)
        return bt.tolist(), slot_map.tolist(), slots.tolist()

    bt, slot_map, slots = tables(0)
    assert bt == [[0, 1, 2, -1], [3, -1, -1, -1]]                 # -1 past a table's end
    assert slot_map == [2 * 4 + 0, 2 * 4 + 1, 2 * 4 + 2, 3 * 4 + 0, 3 * 4 + 1]
    assert slots == [m.state_slot(7), m.state_slot(9)]
    bt, slot_map, _ = tables(1, width=3)
    assert bt == [[-1, 1, 2], [3, -1, -1]] and slot_map[:3] == [8, 9, 10]   # a page the window has passed stays -1

    one = lambda v, t: np.array([v], dtype=t)
    for kw, words in [
        (dict(ids=one(5, np.int64), start=one(0, np.int32), count=one(1, np.int32)), "request 5 is not known"),
        (dict(ids=one(7, np.int64), start=one(5, np.int32), count=one(1, np.int32)), "continues at 5 but its cache holds 8"),
        (dict(ids=one(7, np.int64), start=one(8, np.int32), count=one(5, np.int32)), "has pages for 12 tokens, the step needs 13"),
        (dict(ids=one(7, np.int64), start=one(8, np.int32), count=one(0, np.int32)), "brings no tokens"),
        (dict(width=2), "row of 2 entries for 3 pages"),
    ]:
        with pytest.raises(CacheError, match=words):
            tables(0, **kw)
    m.check()
