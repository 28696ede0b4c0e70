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


@pytest.mark.parametrize("seed", range(6))
def test_native_bookkeeping_follows_the_plain_model(seed):
    """The native core against a plain model in lists and dicts, call by call under a random
    order of calls (requests that come, grow in portions, are cut back, end; two groups, one
    with a window; few pages, so that they run out and are used again): the same block tables
    page for page, the same free pages and slots, the same answers to what is missing and
    what fits, the same refusals; and the step tables the core packs are the tables' pages."""
    import numpy as np
    from plain_cache import Full, Misuse, PlainCache
    rng = random.Random(100 + seed)
    ps, num_pages, max_requests = rng.choice([2, 4, 16]), rng.choice([6, 9, 14]), 3
    window = rng.choice([3, 7, 20])
    needs = [KVNeed(1, 4), KVNeed(1, 4, window)]
    m = CacheManager(needs, [None, None], ps, num_pages, max_requests, torch.float32, "cpu")
    plain = PlainCache([None, window], ps, num_pages, max_requests)
    names = ["a", "b", "c", "d", "e"]
    packed = 0
    for _ in range(600):
        rid = rng.choice(names)
        live = m.has_request(rid)
        assert live == (rid in plain.requests)
        op = rng.choice(["add", "grow", "grow", "grow", "trim", "release", "ask"])
        new_len = (m.length(rid) if live else 0) + rng.randint(0, 3 * ps)
        assert m.pages_missing(rid, new_len) == plain.pages_missing(rid, new_len)
        other = rng.choice(names)
        wanted = [(rid, new_len), (other, rng.randint(1, 4 * ps) +
                                   (m.length(other) if m.has_request(other) else 0))]
        assert m.can_reserve(wanted) == plain.can_reserve(wanted)
        outcome = []
        for cache, full, misuse in ((m, CacheFull, StepError), (plain, Full, (Misuse, KeyError))):
            try:
                if op == "add":
                    cache.add_request(rid)
                elif op == "grow":
                    cache.reserve(rid, new_len)
                elif op == "trim":
                    cache.trim(rid)
                elif op == "release":
                    cache.release(rid)
                outcome.append("ok")
            except full:
                outcome.append("full")
            except misuse:
                outcome.append("misuse")
        assert outcome[0] == outcome[1], (op, rid, outcome)
        if op == "grow" and outcome[0] == "ok" and rng.random() < 0.8:
            m.commit(rid, new_len)
            plain.commit(rid, new_len)
        for r, rec in plain.requests.items():
            assert m.length(r) == rec["length"] and m.state_slot(r) == rec["slot"]
            for g in range(2):
                assert m.table(g, r) == rec["tables"][g], (op, rid, r, g)
        assert m.num_free_pages() == [len(p.free_list) for p in plain.pools]
        assert m.num_free_slots() == len(plain.slots.free_list)
        assert [g.pages.handed_out for g in m.groups] == [p.handed_out for p in plain.pools]
        m.check()
        # a step of the live requests that hold something: one more token each
        step = [r for r in plain.requests if plain.requests[r]["length"] > 0]
        if step and all(m.pages_missing(r, m.length(r) + 1) == [0, 0] for r in step):
            for g in range(2):
                starts = [m.length(r) - 1 for r in step]       # the last token held, again
                width = max(len(plain.requests[r]["tables"][g]) for r in step) + 1
                table = np.empty((len(step), width), dtype=np.int32)
                slots = np.empty((len(step),), dtype=np.int32)
                m.pack_step(g, step, starts, [1] * len(step), width, table, slots)
                packed += 1
                for i, r in enumerate(step):
                    t = plain.requests[r]["tables"][g]
                    assert list(table[i]) == t + [NO_PAGE] * (width - len(t))
                    assert slots[i] == t[starts[i] // ps] * ps + starts[i] % ps
    assert packed > 20
    # several tokens of a request in one step, and a token whose page is not held
    for r, rec in plain.requests.items():
        n, t = rec["length"], rec["tables"][0]
        if n < 2:
            continue
        table = np.empty((1, len(t)), dtype=np.int32)
        slots = np.empty((n - 1,), dtype=np.int32)
        m.pack_step(0, [r], [1], [n - 1], len(t), table, slots)
        assert list(slots) == [t[p // ps] * ps + p % ps for p in range(1, n)]
        if plain._first_needed(1, n) > 0:       # the window has passed the first page
            with pytest.raises(StepError, match="not held"):
                m.pack_step(1, [r], [0], [n], len(rec["tables"][1]),
                            np.empty((1, len(rec["tables"][1])), dtype=np.int32),
                            np.empty((n,), dtype=np.int32))
