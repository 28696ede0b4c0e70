"""Page and slot bookkeeping of the cache: which pages are free, which are held.  The
bookkeeping itself is native host code (``csrc/host/cache_core.cpp``, loaded through
``ctypes``); it never touches a device."""
from __future__ import annotations

import ctypes
from typing import List

from ..errors import CacheFull, ZinferError

_lib = None


def core_lib() -> ctypes.CDLL:
    """The native library of the cache's bookkeeping, built at its first use."""
    global _lib
    if _lib is None:
        from ..ops import build
        lib = build.load("cache_core")
        vp, i32, i64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_longlong
        pi32, pi64 = ctypes.POINTER(i32), ctypes.POINTER(i64)
        lib.zc_last_error.restype = ctypes.c_char_p
        for name, restype, argtypes in (
                ("zc_create", vp, (i32, pi32, i32, i32, i32)), ("zc_destroy", None, (vp,)),
                ("zc_has_request", i32, (vp, i64)), ("zc_length", i32, (vp, i64, pi32)),
                ("zc_state_slot", i32, (vp, i64, pi32)), ("zc_add_request", i32, (vp, i64, pi32)),
                ("zc_pages_missing", None, (vp, i64, i32, pi32)),
                ("zc_can_reserve", i32, (vp, i32, pi64, pi32)), ("zc_reserve", i32, (vp, i64, i32)),
                ("zc_commit", i32, (vp, i64, i32)), ("zc_trim", i32, (vp, i64)),
                ("zc_release", i32, (vp, i64)), ("zc_last_freed", i32, (vp, i32, pi32, i32)),
                ("zc_table", i32, (vp, i32, i64, pi32, i32)),
                ("zc_set_table_entry", i32, (vp, i32, i64, i32, i32)),
                ("zc_pack_group", i32, (vp, i32, i32, pi64, pi32, pi32, i32, pi32, pi32)),
                ("zc_group_counts", None, (vp, i32, pi32, pi64)),
                ("zc_slot_counts", None, (vp, pi32)), ("zc_check", i32, (vp,)),
                ("zp_create", vp, (i32,)), ("zp_destroy", None, (vp,)),
                ("zp_alloc", i32, (vp, i32, pi32)), ("zp_free", i32, (vp, pi32, i32)),
                ("zp_counts", None, (vp, pi32, pi64)), ("zp_check", i32, (vp,))):
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = restype, argtypes
        _lib = lib
    return _lib


def raise_for(code: int, error=ZinferError) -> None:
    """The exception for a call's return code: 1 a pool that has run out, 2 a call that does
    not fit the state (``error``)."""
    if code == 0:
        return
    text = core_lib().zc_last_error().decode()
    raise (CacheFull if code == 1 else error)(text)


class PoolCounts:
    """What a pool of pages (or slots) counts: ``_counts()`` gives free, held, all, the most
    ever held at once, and the pages handed out over the pool's life."""

    def _counts(self):
        raise NotImplementedError

    @property
    def num_free(self) -> int:
        return self._counts()[0]

    @property
    def num_held(self) -> int:
        return self._counts()[1]

    @property
    def num_pages(self) -> int:
        return self._counts()[2]

    @property
    def high_water(self) -> int:
        return self._counts()[3]

    @property
    def handed_out(self) -> int:
        return self._counts()[4]


class PageAllocator(PoolCounts):
    """Pages 0..num_pages-1 with a last-in-first-out free list, so that a page given back is
    the next one handed out (reuse happens early, which is what tests with few pages need).
    Handing out is all-or-nothing; a page is never held twice nor freed twice."""

    def __init__(self, num_pages: int):
        if num_pages < 0:
            raise ValueError("num_pages must not be negative")
        self._lib = core_lib()
        self._h = ctypes.c_void_p(self._lib.zp_create(int(num_pages)))

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.zp_destroy(h)

    def _counts(self):
        what = (ctypes.c_int * 4)()
        handed = ctypes.c_longlong()
        self._lib.zp_counts(self._h, what, ctypes.byref(handed))
        return what[0], what[1], what[2], what[3], handed.value

    def alloc(self, n: int) -> List[int]:
        out = (ctypes.c_int * max(int(n), 1))()
        raise_for(self._lib.zp_alloc(self._h, int(n), out))
        return list(out[:n])

    def free(self, pages) -> None:
        pages = [int(p) for p in pages]
        arr = (ctypes.c_int * max(len(pages), 1))(*pages)
        raise_for(self._lib.zp_free(self._h, arr, len(pages)))

    def check(self) -> None:
        """Every page is either free or held, once."""
        code = self._lib.zp_check(self._h)
        assert code == 0, self._lib.zc_last_error().decode()
