"""A plain model of the cache manager's bookkeeping, in lists and dicts: what the native core
(`zinfer_amd/csrc/host/cache_core.cpp`) is compared with under random orders of calls.  No
tensors, no device; it shares no code with the product path."""
from typing import Dict, List, Optional, Sequence, Tuple

NO_PAGE = -1


class Full(Exception):
    pass


class Misuse(Exception):
    pass


class PlainPool:
    def __init__(self, n: int):
        self.n = n
        self.free_list = list(range(n - 1, -1, -1))       # page 0 is handed out first
        self.held = [False] * n
        self.handed_out = 0

    def take(self) -> int:
        p = self.free_list.pop()
        self.held[p] = True
        self.handed_out += 1
        return p

    def give(self, p: int) -> None:
        if not (0 <= p < self.n) or not self.held[p]:
            raise Misuse(f"page {p} freed but not held")
        self.held[p] = False
        self.free_list.append(p)


class PlainCache:
    """``windows[g]``: the window of group g (None: every key is kept)."""

    def __init__(self, windows: Sequence[Optional[int]], page_size: int, num_pages: int,
                 max_requests: int):
        self.windows = list(windows)
        self.ps = page_size
        self.pools = [PlainPool(num_pages) for _ in windows]
        self.slots = PlainPool(max_requests)
        self.requests: Dict[object, dict] = {}

    def _pages_for(self, tokens: int) -> int:
        return (tokens + self.ps - 1) // self.ps

    def _first_needed(self, g: int, length: int) -> int:
        w = self.windows[g]
        return 0 if w is None else max(0, length - w + 1) // self.ps

    def _missing(self, g: int, table: List[int], length: int, new_len: int) -> int:
        last = self._pages_for(new_len)
        return sum(1 for i in range(self._first_needed(g, length), last)
                   if i >= len(table) or table[i] == NO_PAGE)

    def pages_missing(self, rid, new_len: int) -> List[int]:
        if rid in self.requests:
            r = self.requests[rid]
            return [self._missing(g, r["tables"][g], r["length"], new_len)
                    for g in range(len(self.pools))]
        return [self._pages_for(new_len) - self._first_needed(g, 0) for g in range(len(self.pools))]

    def can_reserve(self, wanted: Sequence[Tuple[object, int]]) -> bool:
        total = [0] * len(self.pools)
        new = 0
        for rid, new_len in wanted:
            new += rid not in self.requests
            for g, n in enumerate(self.pages_missing(rid, new_len)):
                total[g] += n
        return new <= len(self.slots.free_list) and \
            all(t <= len(p.free_list) for t, p in zip(total, self.pools))

    def add_request(self, rid) -> None:
        if rid in self.requests:
            raise Misuse("already live")
        if not self.slots.free_list:
            raise Full("no slot")
        self.requests[rid] = {"length": 0, "slot": self.slots.take(),
                              "tables": [[] for _ in self.pools]}

    def reserve(self, rid, new_len: int) -> None:
        r = self.requests[rid]
        if new_len < r["length"]:
            raise Misuse("cannot shrink")
        missing = self.pages_missing(rid, new_len)
        if any(n > len(p.free_list) for n, p in zip(missing, self.pools)):
            raise Full("no pages")
        last = self._pages_for(new_len)
        for g, pool in enumerate(self.pools):
            table = r["tables"][g]
            table.extend([NO_PAGE] * (last - len(table)))
            for i in range(self._first_needed(g, r["length"]), last):
                if table[i] == NO_PAGE:
                    table[i] = pool.take()

    def _give_back(self, g: int, pages: List[int]) -> None:
        for p in reversed(pages):      # the first of them is handed out next
            self.pools[g].give(p)

    def commit(self, rid, new_len: int) -> None:
        r = self.requests[rid]
        r["length"] = new_len
        for g, w in enumerate(self.windows):
            if w is None:
                continue
            table = r["tables"][g]
            gone = [i for i in range(min(self._first_needed(g, new_len), len(table)))
                    if table[i] != NO_PAGE]
            self._give_back(g, [table[i] for i in gone])
            for i in gone:
                table[i] = NO_PAGE

    def trim(self, rid) -> None:
        r = self.requests[rid]
        keep = self._pages_for(r["length"])
        for g in range(len(self.pools)):
            table = r["tables"][g]
            self._give_back(g, [p for p in table[keep:] if p != NO_PAGE])
            del table[keep:]

    def release(self, rid) -> None:
        r = self.requests.pop(rid)
        for g in range(len(self.pools)):
            self._give_back(g, [p for p in r["tables"][g] if p != NO_PAGE])
        self.slots.give(r["slot"])
