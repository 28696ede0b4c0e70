"""The cache manager: keys and values in pages with a block table for each request, one pool
for each group of layers with the same need, and slots for per-request state of fixed size.

The reference keeps one contiguous buffer per request and layer, sized at creation
(`src/model/runtime/optimized_kv_cache/cache.zig:21-107,350-404`), and recycles it with
``reset()`` (`:109-111`); its ``error.CacheFull`` (`:96`) is kept as the error of a pool
that has run out.  Paging, groups and slots are this engine's own.

Layout of a group's pool, per run of a layer: keys ``[num_pages, n_kv_heads, page_size,
head_dim]`` and values ``[num_pages, n_kv_heads, value width, page_size]`` (the positions of a
page contiguous, as the attention kernels' second matrix product reads them; the value
width is the key's unless the need says otherwise, and so is the dtype); token ``p`` of
a request lies in page ``table[p // page_size]`` at row ``p % page_size``.  The manager only
hands out pages; the layout inside a page belongs to the kernels.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from ..errors import CacheFull, StepError
from ..parts.base import KVNeed, StateNeed
from .pages import PageAllocator

NO_PAGE = -1


@dataclass
class LayerCacheView:
    """What a mixer gets for one run of its layer."""
    group: int                       # index of the KV group (-1: none)
    page_size: int
    k_pool: Optional[torch.Tensor]   # [num_pages, n_kv * page_size * key width] or None
    v_pool: Optional[torch.Tensor]   # [num_pages, n_kv * page_size * value width] or None
    writes: bool                     # False: the run only reads another run's cache
    state: Optional[torch.Tensor]    # [max_requests, *shape] for a StateNeed


class KVGroup:
    def __init__(self, need: KVNeed, runs: List[int], page_size: int, num_pages: int,
                 dtype: torch.dtype, device):
        self.need = need
        self.runs = runs                     # schedule positions that own a cache here
        self.page_size = page_size
        self.pages = PageAllocator(num_pages)
        self.tables: Dict[object, List[int]] = {}
        # a need may bring its own dtype and a value row of another width than a key's
        dtype = need.dtype or dtype
        self.k = torch.zeros((len(runs), num_pages, need.n_kv_heads * page_size * need.key_width),
                             dtype=dtype, device=device)
        self.v = torch.zeros((len(runs), num_pages, need.n_kv_heads * page_size * need.value_width),
                             dtype=dtype, device=device)

    def first_needed_page(self, length: int) -> int:
        """Logical index of the first page a query at position >= ``length`` can still read."""
        if self.need.window is None:
            return 0
        return max(0, length - self.need.window + 1) // self.page_size

    def pages_missing(self, rid, length: int, new_len: int) -> int:
        table = self.tables[rid]
        last = (new_len + self.page_size - 1) // self.page_size
        if self.need.window is None:       # no holes: every page up to len(table) is held
            return max(0, last - len(table))
        first = self.first_needed_page(length)
        return sum(1 for i in range(first, last) if i >= len(table) or table[i] == NO_PAGE)


class CacheManager:
    """``needs[pos]`` is the cache need of schedule position ``pos`` (None: no cache of its
    own); ``reads[pos]`` names the position whose cache a run reads instead."""

    def __init__(self, needs: Sequence[object], reads: Sequence[Optional[int]], page_size: int,
                 num_pages: int, max_requests: int, kv_dtype: torch.dtype, device,
                 poison_freed: bool = False):
        if page_size < 1:
            raise ValueError("page_size must be at least 1")
        self.page_size = page_size
        self.max_requests = max_requests
        self.device = device
        self.poison_freed = poison_freed
        self.groups: List[KVGroup] = []
        by_need: Dict[KVNeed, List[int]] = {}
        self.state_pools: Dict[int, torch.Tensor] = {}
        for pos, need in enumerate(needs):
            if isinstance(need, KVNeed):
                by_need.setdefault(need, []).append(pos)
            elif isinstance(need, StateNeed):
                self.state_pools[pos] = torch.zeros((max_requests,) + tuple(need.shape),
                                                    dtype=need.dtype, device=device)
            elif need is not None:
                raise StepError(f"unknown cache need {need!r}")
        self._where: Dict[int, Tuple[int, int]] = {}     # schedule position -> (group, run)
        for need, runs in by_need.items():
            g = len(self.groups)
            self.groups.append(KVGroup(need, runs, page_size, num_pages, kv_dtype, device))
            for i, pos in enumerate(runs):
                self._where[pos] = (g, i)
        self._reads = list(reads)
        self._slots = PageAllocator(max_requests)        # state slots, same bookkeeping
        self.requests: Dict[object, dict] = {}

    # ------------------------------------------------------------------ views
    def view(self, pos: int) -> LayerCacheView:
        src = self._reads[pos] if self._reads[pos] is not None else pos
        state = self.state_pools.get(src)
        if src in self._where:
            g, i = self._where[src]
            grp = self.groups[g]
            return LayerCacheView(g, self.page_size, grp.k[i], grp.v[i], src == pos, state)
        return LayerCacheView(-1, self.page_size, None, None, src == pos, state)

    # ------------------------------------------------------------------ requests
    def has_request(self, rid) -> bool:
        return rid in self.requests

    def length(self, rid) -> int:
        return self.requests[rid]["length"]

    def state_slot(self, rid) -> int:
        return self.requests[rid]["slot"]

    def add_request(self, rid) -> None:
        if rid in self.requests:
            raise StepError(f"request {rid!r} is already live")
        if self._slots.num_free == 0:
            raise CacheFull(f"CacheFull: all {self.max_requests} request slots are in use")
        slot = self._slots.alloc(1)[0]
        for pool in self.state_pools.values():
            pool[slot].zero_()
        self.requests[rid] = {"length": 0, "slot": slot}
        for grp in self.groups:
            grp.tables[rid] = []

    def pages_missing(self, rid, new_len: int) -> List[int]:
        """Pages each group would have to hand out for ``rid`` (live or not yet) to hold
        ``new_len`` tokens."""
        if rid in self.requests:
            length = self.requests[rid]["length"]
            return [grp.pages_missing(rid, length, new_len) for grp in self.groups]
        last = (new_len + self.page_size - 1) // self.page_size
        return [last - grp.first_needed_page(0) for grp in self.groups]

    def can_reserve(self, wanted: Sequence[Tuple[object, int]]) -> bool:
        """Whether all ``(request, new_len)`` of a step fit together."""
        total = [0] * len(self.groups)
        new = 0
        for rid, new_len in wanted:
            if rid not in self.requests:
                new += 1
            for g, n in enumerate(self.pages_missing(rid, new_len)):
                total[g] += n
        return new <= self._slots.num_free and \
            all(t <= grp.pages.num_free for t, grp in zip(total, self.groups))

    def reserve(self, rid, new_len: int) -> None:
        """Pages for positions up to ``new_len`` (all groups or none)."""
        req = self.requests[rid]
        if new_len < req["length"]:
            raise StepError(f"request {rid!r} holds {req['length']} tokens, cannot shrink to "
                            f"{new_len}")
        missing = self.pages_missing(rid, new_len)
        for n, grp in zip(missing, self.groups):
            if n > grp.pages.num_free:
                raise CacheFull(f"CacheFull: request {rid!r} needs {n} more pages of "
                                f"{self.page_size} tokens, {grp.pages.num_free} of "
                                f"{grp.pages.num_pages} free")
        for grp in self.groups:
            table = grp.tables[rid]
            last = (new_len + self.page_size - 1) // self.page_size
            first = grp.first_needed_page(req["length"])
            while len(table) < last:
                table.append(NO_PAGE)
            for i in range(first, last):
                if table[i] == NO_PAGE:
                    table[i] = grp.pages.alloc(1)[0]

    def commit(self, rid, new_len: int) -> None:
        """The request now holds ``new_len`` tokens; pages a window has passed go back."""
        req = self.requests[rid]
        req["length"] = new_len
        for grp in self.groups:
            if grp.need.window is None:
                continue
            table = grp.tables[rid]
            first = grp.first_needed_page(new_len)
            gone = [i for i in range(min(first, len(table))) if table[i] != NO_PAGE]
            self._give_back(grp, [table[i] for i in gone])
            for i in gone:
                table[i] = NO_PAGE

    def trim(self, rid) -> None:
        """Gives back the pages reserved beyond the tokens the request holds (a step that
        reserved them did not run)."""
        req = self.requests[rid]
        keep = (req["length"] + self.page_size - 1) // self.page_size
        for grp in self.groups:
            table = grp.tables[rid]
            self._give_back(grp, [p for p in table[keep:] if p != NO_PAGE])
            del table[keep:]

    def pages_at_most(self, n_tokens: int, portion: int) -> List[int]:
        """Upper bound, per group, of the pages a request of ``n_tokens`` tokens holds at any
        one time when it runs in portions of at most ``portion`` tokens: a group with a window
        keeps only the window and the portion being written."""
        out = []
        for grp in self.groups:
            n = n_tokens
            if grp.need.window is not None:
                n = min(n, grp.need.window + portion + self.page_size)
            out.append((n + self.page_size - 1) // self.page_size)
        return out

    def num_pages(self) -> List[int]:
        return [g.pages.num_pages for g in self.groups]

    def release(self, rid) -> None:
        """Everything the request holds goes back: pages of every group and the state slot."""
        req = self.requests.pop(rid, None)
        if req is None:
            raise StepError(f"request {rid!r} is not live")
        for grp in self.groups:
            table = grp.tables.pop(rid)
            self._give_back(grp, [p for p in table if p != NO_PAGE])
        self._slots.free([req["slot"]])

    def _give_back(self, grp: KVGroup, pages: List[int]) -> None:
        if not pages:
            return
        if self.poison_freed:
            if grp.k.is_cuda:
                from .. import ops
                idx = torch.tensor(pages, dtype=torch.int32, device=self.device)
                ops.poison_pages(grp.k, idx)
                ops.poison_pages(grp.v, idx)
            else:
                idx = torch.tensor(pages, dtype=torch.long, device=self.device)
                grp.k[:, idx] = float("nan")
                grp.v[:, idx] = float("nan")
        grp.pages.free(reversed(pages))

    def table(self, group: int, rid) -> List[int]:
        return self.groups[group].tables[rid]

    # ------------------------------------------------------------------ accounting
    def num_free_slots(self) -> int:
        return self._slots.num_free

    def num_free_pages(self) -> List[int]:
        return [g.pages.num_free for g in self.groups]

    def kv_bytes(self) -> int:
        return sum(g.k.numel() * g.k.element_size() + g.v.numel() * g.v.element_size()
                   for g in self.groups)

    def check(self) -> None:
        """No page lost, none held twice: the pages in all tables are exactly the held ones."""
        for grp in self.groups:
            grp.pages.check()
            held = [p for t in grp.tables.values() for p in t if p != NO_PAGE]
            assert len(held) == len(set(held)), "a page is in two tables"
            assert len(held) == grp.pages.num_held, "held pages and tables disagree"
        self._slots.check()
        slots = [r["slot"] for r in self.requests.values()]
        assert len(slots) == len(set(slots)) == self._slots.num_held
