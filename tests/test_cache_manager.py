"""Page allocator, page groups, windows and state slots: no page lost, held twice or freed twice."""
import random

import pytest
import torch

from velox_amd.cache import NULL_PAGE, CacheManager, PoolExhausted, PageAllocator
from velox_amd.parts import StateNeed, kv_pages


def test_allocator_order_and_errors():
    a = PageAllocator(6)
    assert [a.take() for _ in range(3)] == [1, 2, 3]  # page 0 is never handed out
    a.drop(2)
    assert a.take() == 2  # the page freed last is used again first
    assert a.take_many(2) == [4, 5]
    with pytest.raises(PoolExhausted):
        a.take()
    with pytest.raises(PoolExhausted):
        a.take_many(1)
    a.drop(4)
    with pytest.raises(RuntimeError):
        a.drop(4)  # freed twice
    with pytest.raises(RuntimeError):
        a.share(4)  # free page
    a.share(1)
    assert a.drop(1) == 1 and a.num_free == 1
    assert a.drop(NULL_PAGE) == 1  # the reserved page stays
    with pytest.raises(IndexError):
        a.drop(6)
    with pytest.raises(ValueError):
        PageAllocator(1)
    a.verify()


@pytest.mark.parametrize("num_pages", [2, 3, 4, 5, 17, 64, 1000, 7201])
def test_scattered_first_hand_outs(num_pages):
    """``scatter=True``: every page is still handed out exactly once, never page 0, freed pages come back most recent
    first, the order is the same every time, and pages handed out 256 hand-outs apart (the same place of two sequences
    filled one after the other) lie at no regular distance."""
    a = PageAllocator(num_pages, scatter=True)
    order = a.take_many(num_pages - 1)
    assert sorted(order) == list(range(1, num_pages))
    with pytest.raises(PoolExhausted):
        a.take()
    if num_pages > 2:
        a.drop(order[0])
        a.drop(order[-1])
        assert a.take() == order[-1] and a.take() == order[0]
    a.verify()
    assert PageAllocator(num_pages, scatter=True).take_many(num_pages - 1) == order
    if num_pages >= 1000:
        far = {(order[i + 256] - order[i]) % (num_pages - 1) for i in range(len(order) - 256)}
        assert len(far) > (len(order) - 256) // 2
    assert PageAllocator(num_pages).take_many(num_pages - 1) == list(range(1, num_pages))


def _manager(needs, pages=9, page=4, seqs=4, max_len=None):
    return CacheManager(needs, page, pages, seqs, torch.float32, "cpu", max_model_len=max_len)


def test_growth_and_release():
    need = kv_pages(2, 16)
    m = _manager([need, need, need])
    assert len(m.groups) == 1 and m.groups[0].tensors["k"].shape == (3, 9, 2, 4, 16) and m.groups[0].tensors["v"].shape == (3, 9, 2, 16, 4)
    assert m.max_model_len == 32
    s = m.new_sequence()
    assert m.append(s, 0, 5) and s.tables[0] == [1, 2]
    assert m.append(s, 5, 3) and s.tables[0] == [1, 2]  # 8 tokens still fit two pages
    assert m.append(s, 8, 1) and s.tables[0] == [1, 2, 3]
    assert m.slot_for(s, 0, 6) == 2 * 4 + 2
    t = m.new_sequence()
    assert not m.append(t, 0, 21) and t.tables[0] == []  # all or nothing
    assert m.append(t, 0, 20) and m.num_free_pages() == 0
    assert not m.can_append(s, 9, 4) and m.can_append(s, 9, 3)
    assert not m.append(s, 9, 100)  # beyond max_model_len
    m.assert_consistent([s, t])
    m.free_sequence(t)
    assert m.num_free_pages() == 5
    u = m.new_sequence()
    assert m.append(u, 0, 1) and u.tables[0] == [8]  # the page freed last is handed out first
    m.free_sequence(s)
    m.free_sequence(u)
    m.assert_consistent([])
    assert m.num_used_pages() == 0 and m.state.num_free == 4


def test_groups_by_need_and_window_release():
    full = kv_pages(2, 16)
    windowed = kv_pages(2, 16, window=6)
    m = _manager([full, windowed, full, windowed, None], pages=12)
    assert len(m.groups) == 2 and m.entry_group[0] == (0, 0) and m.entry_group[2] == (0, 1) and m.entry_group[3] == (1, 1)
    s = m.new_sequence()
    assert m.append(s, 0, 10)
    assert s.tables == [[1, 2, 3], [1, 2, 3]]  # each group has pages of its own
    assert m.release_behind_window(s, 10) == 1  # a query at 10 reads keys 5..: page 0 (keys 0..3) goes back
    assert s.tables[1] == [NULL_PAGE, 2, 3] and s.tables[0] == [1, 2, 3]
    assert m.groups[1].allocator.num_free == 9 and m.groups[0].allocator.num_free == 8
    assert m.append(s, 10, 7)  # 17 tokens: 5 entries
    assert s.tables[1][3] == 1  # the page given back is used again, by the same request
    assert m.release_behind_window(s, 17) == 2  # keys 12.. are needed: pages 1 and 2 go back
    assert m.release_behind_window(s, 17) == 0
    m.assert_consistent([s])
    m.free_sequence(s)
    m.assert_consistent([])
    assert all(g.allocator.num_used == 0 for g in m.groups)


def test_state_slots_are_zeroed_on_take():
    need = StateNeed((("sum", (3,), torch.float32), ("count", (), None)))
    m = _manager([kv_pages(1, 16), need], seqs=2)
    a, b = m.new_sequence(), m.new_sequence()
    assert m.new_sequence() is None and {a.slot, b.slot} == {0, 1}
    view = m.view(1, [None])
    assert view.tensors["sum"].shape == (3, 3) and view.tensors["count"].shape == (3,)  # one spare row for padding
    view.tensors["sum"][a.slot] = 7.0
    m.free_sequence(a)
    with pytest.raises(RuntimeError):
        m.state.release(a.slot if a.slot >= 0 else 0 if b.slot != 0 else 1)
    c = m.new_sequence()
    assert float(view.tensors["sum"][c.slot].abs().sum()) == 0.0
    m.free_sequence(b)
    m.free_sequence(c)
    m.assert_consistent([])


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_of_requests(seed):
    rng = random.Random(seed)
    windowed = seed % 2 == 1
    needs = [kv_pages(1, 16), kv_pages(1, 16, window=9) if windowed else kv_pages(1, 16)]
    m = _manager(needs, pages=14, page=4, seqs=5)
    live = {}
    for step in range(600):
        action = rng.random()
        if action < 0.25 and len(live) < 5:
            seq = m.new_sequence()
            assert seq is not None
            live[step] = [seq, 0]
        elif action < 0.85 and live:
            key = rng.choice(list(live))
            seq, computed = live[key]
            n = rng.choice([1, 1, 1, 2, 5, 7, 13])
            before = [list(t) for t in seq.tables]
            if m.append(seq, computed, n):
                live[key][1] = computed + n
                m.release_behind_window(seq, computed + n)
            else:
                assert [list(t) for t in seq.tables] == before  # a refused growth changes nothing
        elif live:
            key = rng.choice(list(live))
            m.free_sequence(live.pop(key)[0])
        m.assert_consistent([s for s, _ in live.values()])
        for seq, computed in live.values():
            for g, group in enumerate(m.groups):
                first = group.first_needed_page(computed)
                for index in range(first, group.table_entries_for(computed)):
                    assert seq.tables[g][index] != NULL_PAGE  # every page a query may read is held
    for seq, _ in live.values():
        m.free_sequence(seq)
    m.assert_consistent([])
    assert m.num_used_pages() == 0 and m.state.num_free == 5


def test_pool_size_from_free_memory():
    """Reference ``src/paged_kv_cache.py:183-194``: (free bytes x utilisation - reserve) / bytes per page, rounded down."""
    from velox_amd.cache.manager import pages_that_fit

    per_page = 2 * 16 * 4 * 128 * 2 * 28  # keys and values, 16 tokens, 4 KV heads of 128, bfloat16, 28 layers
    assert pages_that_fit(per_page, 100 << 30, 0.9, 512 << 20) == (int((100 << 30) * 0.9) - (512 << 20)) // per_page
    assert pages_that_fit(per_page, 10 * per_page + 1000, 1.0, 1000) == 10
    with pytest.raises(RuntimeError, match="not enough free GPU memory"):
        pages_that_fit(per_page, 1 << 20, 0.5, 1 << 20)
    with pytest.raises(RuntimeError, match="even one cache page"):
        pages_that_fit(per_page, per_page + 10, 1.0, 0)
    m = CacheManager([kv_pages(4, 128)] * 28, 16, 2, 4, torch.bfloat16, "cpu", allocate_tensors=False)
    assert m.bytes_per_page() == per_page
