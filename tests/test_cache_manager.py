"""The cache manager: no page lost, held twice or freed twice, under random orders of
requests; groups with a window give pages back; state slots."""
import random

import pytest
import torch

from zinfer_amd import CacheFull, StepError, ZinferError
from zinfer_amd.cache import NO_PAGE, CacheManager, PageAllocator
from zinfer_amd.parts import KVNeed, StateNeed


def test_page_allocator_lifo_and_errors():
    a = PageAllocator(4)
    p = a.alloc(3)
    assert len(set(p)) == 3 and a.num_free == 1
    with pytest.raises(CacheFull):
        a.alloc(2)
    assert a.num_free == 1                      # all or nothing
    a.free([p[1]])
    assert a.alloc(1) == [p[1]]                 # the page given back is the next handed out
    with pytest.raises(ZinferError):
        a.free([3] if 3 not in p else [99])
    a.free(p)
    with pytest.raises(ZinferError):
        a.free([p[0]])                          # freed twice
    a.check()


def _manager(window=None, num_pages=12, page_size=4, max_requests=3, state=False):
    needs = [KVNeed(2, 8), KVNeed(2, 8, window), KVNeed(2, 8)]
    reads = [None, None, None]
    if state:
        needs.append(StateNeed((5,)))
        reads.append(None)
    return CacheManager(needs, reads, page_size, num_pages, max_requests, torch.float32, "cpu")


def test_groups_by_need_and_shared_cache():
    m = _manager(window=6)
    assert len(m.groups) == 2                   # layers 0 and 2 share a need, layer 1 has its own
    assert m.groups[0].runs == [0, 2] and m.groups[1].runs == [1]
    assert m.view(0).group == 0 and m.view(2).group == 0 and m.view(1).group == 1
    m2 = CacheManager([KVNeed(1, 4), None], [None, 0], 4, 4, 2, torch.float32, "cpu")
    v0, v1 = m2.view(0), m2.view(1)
    assert v1.k_pool.data_ptr() == v0.k_pool.data_ptr() and v0.writes and not v1.writes


def test_reserve_commit_release():
    m = _manager(num_pages=5)
    m.add_request("a")
    m.reserve("a", 9)                           # 3 pages of 4
    assert m.num_free_pages() == [2]
    m.commit("a", 9)
    m.reserve("a", 12)                          # still 3 pages
    assert m.num_free_pages() == [2]
    with pytest.raises(CacheFull):
        m.reserve("a", 21)                      # 6 pages > 5
    assert m.num_free_pages() == [2]
    assert not m.can_reserve([("a", 12), ("b", 9)]) and m.can_reserve([("a", 12), ("b", 8)])
    with pytest.raises(StepError):
        m.reserve("a", 3)
    m.release("a")
    assert m.num_free_pages() == [5]
    with pytest.raises(StepError):
        m.release("a")
    m.check()


def test_window_gives_pages_back():
    m = _manager(window=6, num_pages=6)
    m.add_request("a")
    length = 0
    for new_len in (3, 10, 11, 19, 20, 24):
        m.reserve("a", new_len)
        m.commit("a", new_len)
        length = new_len
        full, win = m.table(0, "a"), m.table(1, "a")
        assert all(p != NO_PAGE for p in full)
        first = max(0, length - 6 + 1) // 4     # first page a later query can still read
        assert all(p == NO_PAGE for p in win[:first]) and all(p != NO_PAGE for p in win[first:])
        m.check()
    assert m.groups[1].pages.num_held <= 3      # ceil(window / page) + 1
    assert m.groups[0].pages.num_held == 6
    m.release("a")
    m.check()


def test_state_slots():
    m = _manager(state=True, max_requests=2)
    m.add_request("a"); m.add_request("b")
    assert {m.state_slot("a"), m.state_slot("b")} == {0, 1}
    m.state_pools[3][m.state_slot("a")] = 7.0
    with pytest.raises(CacheFull):
        m.add_request("c")
    slot = m.state_slot("a")
    m.release("a")
    m.add_request("c")
    assert m.state_slot("c") == slot and float(m.state_pools[3][slot].abs().sum()) == 0.0
    assert m.view(3).state is m.state_pools[3] and m.view(3).group == -1
    m.check()


@pytest.mark.parametrize("seed", range(6))
@pytest.mark.parametrize("window", [None, 7])
def test_random_orders_lose_nothing(seed, window):
    rnd = random.Random(seed)
    m = _manager(window=window, num_pages=10, page_size=4, max_requests=4)
    lengths = {}
    next_id = 0
    for _ in range(400):
        op = rnd.random()
        if op < 0.25 and len(lengths) < 4:
            rid = f"r{next_id}"; next_id += 1
            m.add_request(rid)
            lengths[rid] = 0
        elif op < 0.85 and lengths:
            rid = rnd.choice(sorted(lengths))
            new_len = lengths[rid] + rnd.choice((1, 1, 1, 2, 5, 13))
            if m.can_reserve([(rid, new_len)]):
                m.reserve(rid, new_len)
                m.commit(rid, new_len)
                lengths[rid] = new_len
            else:
                with pytest.raises(CacheFull):
                    m.reserve(rid, new_len)
        elif lengths:
            rid = rnd.choice(sorted(lengths))
            m.release(rid)
            del lengths[rid]
        m.check()
        for rid, n in lengths.items():
            assert m.length(rid) == n
            assert len([p for p in m.table(0, rid) if p != NO_PAGE]) == (n + 3) // 4
    for rid in list(lengths):
        m.release(rid)
    m.check()
    assert all(g.pages.num_free == g.pages.num_pages for g in m.groups)
