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

import ctypes
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..errors import StepError
from ..parts.base import KVNeed, StateNeed
from .pages import PoolCounts, core_lib, raise_for

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


class _GroupPages(PoolCounts):
    """The counts of one group's pool of pages (or, group -1, of the request slots)."""

    def __init__(self, manager: "CacheManager", group: int):
        self._manager, self._group = manager, group

    def _counts(self):
        lib, h = self._manager._lib, self._manager._core
        what = (ctypes.c_int * 4)()
        handed = ctypes.c_longlong()
        if self._group < 0:
            lib.zc_slot_counts(h, what)
        else:
            lib.zc_group_counts(h, self._group, what, ctypes.byref(handed))
        return what[0], what[1], what[2], what[3], handed.value


class KVGroup:
    """The pools of one group of layers with the same need; which of their pages are free and
    which request holds which is the native core's to know (``pages``: its counts)."""

    def __init__(self, need: KVNeed, runs: List[int], page_size: int, num_pages: int,
                 dtype: torch.dtype, device, pages: PoolCounts):
        self.need = need
        self.runs = runs                     # schedule positions that own a cache here
        self.page_size = page_size
        self.pages = pages
        # a need may bring its own dtype and a value row of another width than a key's
        dtype = need.dtype or dtype
        self.k = torch.zeros((len(runs), num_pages, need.n_kv_heads * page_size * need.key_width),
                             dtype=dtype, device=device)
        self.v = torch.zeros((len(runs), num_pages, need.n_kv_heads * page_size * need.value_width),
                             dtype=dtype, device=device)


class CacheManager:
    """``needs[pos]`` is the cache need of schedule position ``pos`` (None: no cache of its
    own); ``reads[pos]`` names the position whose cache a run reads instead.  The pools are
    tensors of this class; which pages are free, the block tables and the slots are kept by
    the native core, where a request goes by a number that this class gives it."""

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
        self._lib = core_lib()
        windows = [-1 if need.window is None else int(need.window) for need in by_need]
        self._core = ctypes.c_void_p(self._lib.zc_create(
            len(windows), (ctypes.c_int * max(len(windows), 1))(*windows), int(page_size),
            int(num_pages), int(max_requests)))
        if not self._core:
            raise ValueError(f"a cache of {num_pages} pages of {page_size} tokens for "
                             f"{max_requests} requests cannot be made")
        self._where: Dict[int, Tuple[int, int]] = {}     # schedule position -> (group, run)
        for need, runs in by_need.items():
            g = len(self.groups)
            self.groups.append(KVGroup(need, runs, page_size, num_pages, kv_dtype, device,
                                       _GroupPages(self, g)))
            for i, pos in enumerate(runs):
                self._where[pos] = (g, i)
        self._reads = list(reads)
        self._slots = _GroupPages(self, -1)              # state slots, same bookkeeping
        self.requests: Dict[object, int] = {}            # live request -> its number in the core
        self._names: Dict[int, object] = {}
        self._next_number = 0

    def __del__(self):
        core, self._core = getattr(self, "_core", None), None
        if core:
            self._lib.zc_destroy(core)

    def _number(self, rid) -> int:
        try:
            return self.requests[rid]
        except KeyError:
            raise StepError(f"request {rid!r} is not live") from None

    def _raise(self, code: int) -> None:
        """The core's error with the request's own name in place of its number."""
        if code == 0:
            return
        try:
            raise_for(code, StepError)
        except Exception as e:  # noqa: BLE001 - re-raised with the name put in
            text = str(e)
            for number, rid in self._names.items():
                text = text.replace(f"request #{number} ", f"request {rid!r} ")
            raise type(e)(text) from None

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
        out = ctypes.c_int()
        self._raise(self._lib.zc_length(self._core, self._number(rid), ctypes.byref(out)))
        return out.value

    def state_slot(self, rid) -> int:
        out = ctypes.c_int()
        self._raise(self._lib.zc_state_slot(self._core, self._number(rid), ctypes.byref(out)))
        return out.value

    def add_request(self, rid) -> None:
        if rid in self.requests:
            raise StepError(f"request {rid!r} is already live")
        number, slot = self._next_number, ctypes.c_int()
        self._raise(self._lib.zc_add_request(self._core, number, ctypes.byref(slot)))
        self._next_number += 1
        self.requests[rid] = number
        self._names[number] = rid
        for pool in self.state_pools.values():
            pool[slot.value].zero_()

    def _number_or_new(self, rid) -> int:
        return self.requests.get(rid, -1)        # no request has the number -1: "not yet live"

    def pages_missing(self, rid, new_len: int) -> List[int]:
        """Pages each group would have to hand out for ``rid`` (live or not yet) to hold
        ``new_len`` tokens."""
        out = (ctypes.c_int * max(len(self.groups), 1))()
        self._lib.zc_pages_missing(self._core, self._number_or_new(rid), int(new_len), out)
        return list(out[:len(self.groups)])

    def can_reserve(self, wanted: Sequence[Tuple[object, int]]) -> bool:
        """Whether all ``(request, new_len)`` of a step fit together."""
        n = len(wanted)
        rids = (ctypes.c_longlong * max(n, 1))(*[self._number_or_new(r) for r, _ in wanted])
        lens = (ctypes.c_int * max(n, 1))(*[int(l) for _, l in wanted])
        return bool(self._lib.zc_can_reserve(self._core, n, rids, lens))

    def reserve(self, rid, new_len: int) -> None:
        """Pages for positions up to ``new_len`` (all groups or none)."""
        self._raise(self._lib.zc_reserve(self._core, self._number(rid), int(new_len)))

    def commit(self, rid, new_len: int) -> None:
        """The request now holds ``new_len`` tokens; pages a window has passed go back."""
        self._raise(self._lib.zc_commit(self._core, self._number(rid), int(new_len)))
        self._poison_freed()

    def trim(self, rid) -> None:
        """Gives back the pages reserved beyond the tokens the request holds (a step that
        reserved them did not run)."""
        self._raise(self._lib.zc_trim(self._core, self._number(rid)))
        self._poison_freed()

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
        number = self._number(rid)
        self._raise(self._lib.zc_release(self._core, number))
        del self.requests[rid]
        del self._names[number]
        self._poison_freed()

    def _poison_freed(self) -> None:
        """(debugging) What the last call gave back is overwritten with NaN, so that a kernel
        that reads a page it does not hold shows."""
        if not self.poison_freed:
            return
        for g, grp in enumerate(self.groups):
            cap = grp.pages.num_pages
            out = (ctypes.c_int * max(cap, 1))()
            n = self._lib.zc_last_freed(self._core, g, out, cap)
            if n == 0:
                continue
            pages = list(out[:n])
            if grp.k.is_cuda:
                from .. import ops
                idx = torch.tensor(pages, dtype=torch.int32, device=self.device)
                ops.poison_pages(grp.k, idx)
                ops.poison_pages(grp.v, idx)
            else:
                idx = torch.tensor(pages, dtype=torch.long, device=self.device)
                grp.k[:, idx] = float("nan")
                grp.v[:, idx] = float("nan")

    def table(self, group: int, rid) -> List[int]:
        """A copy of the request's block table in a group."""
        number = self._number(rid)
        cap = self.groups[group].pages.num_pages + 1
        while True:
            out = (ctypes.c_int * cap)()
            n = self._lib.zc_table(self._core, group, number, out, cap)
            if n <= cap:
                return list(out[:n])
            cap = n

    def set_table_entry(self, group: int, rid, index: int, page: int) -> None:
        """(debugging) Plants ``page`` in a block table, whatever the pool says: what the
        device-side check of a step's tables is tested with."""
        self._raise(self._lib.zc_set_table_entry(self._core, group, self._number(rid),
                                                 int(index), int(page)))

    def pack_step(self, group: int, rids: Sequence[object], starts: Sequence[int],
                  q_lens: Sequence[int], max_pages: int, table_out: np.ndarray,
                  slots_out: np.ndarray) -> None:
        """A step's block tables ``table_out`` [n, max_pages] (``NO_PAGE`` where a request has
        none) and slot mapping ``slots_out`` [sum of q_lens] (page * page_size + row of every
        token's own key and value) of one group, written into int32 arrays of the caller's."""
        n = len(rids)
        if table_out.dtype != np.int32 or slots_out.dtype != np.int32 \
                or not table_out.flags.c_contiguous or not slots_out.flags.c_contiguous \
                or table_out.size != n * max_pages or slots_out.size != sum(q_lens):
            raise StepError("pack_step: int32 arrays [n, max_pages] and [tokens] are needed")
        numbers = (ctypes.c_longlong * max(n, 1))(*[self._number(r) for r in rids])
        s = (ctypes.c_int * max(n, 1))(*[int(x) for x in starts])
        q = (ctypes.c_int * max(n, 1))(*[int(x) for x in q_lens])
        self._raise(self._lib.zc_pack_group(
            self._core, group, n, numbers, s, q, int(max_pages),
            table_out.ctypes.data_as(ctypes.POINTER(ctypes.c_int)),
            slots_out.ctypes.data_as(ctypes.POINTER(ctypes.c_int))))

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
        code = self._lib.zc_check(self._core)
        assert code == 0, self._lib.zc_last_error().decode()
