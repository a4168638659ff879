"""The cache manager: which pages and which state slot each request holds.

A thin face of the native manager (csrc/host/cache_manager.cpp).  It knows nothing of tensors: groups are
(page size, number of pages, window) triples, requests are integers.  ``CachePool`` (pool.py) owns the device
memory that the page numbers index.
"""
from __future__ import annotations

import ctypes
import dataclasses
from typing import List, Optional, Sequence

import numpy as np

from ..kernels.library import load_host_library


class CacheError(RuntimeError):
    pass


class OutOfPages(CacheError):
    """A reservation that the free pages cannot cover; nothing was taken."""


@dataclasses.dataclass(frozen=True)
class GroupGeometry:
    page_size: int
    num_pages: int
    window: Optional[int] = None


_lib = None


def _host():
    global _lib
    if _lib is None:
        lib = load_host_library()
        lib.cm_create.restype = ctypes.c_void_p
        lib.cm_create.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int]
        lib.cm_destroy.argtypes = [ctypes.c_void_p]
        lib.cm_destroy.restype = None
        for name in ("cm_add_request", "cm_free", "cm_state_slot"):
            getattr(lib, name).argtypes = [ctypes.c_void_p, ctypes.c_int64]
        for name in ("cm_can_reserve", "cm_reserve", "cm_release_behind", "cm_can_admit"):
            getattr(lib, name).argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64]
        lib.cm_fits_at_all.argtypes = [ctypes.c_void_p, ctypes.c_int64]
        lib.cm_reserved_len.argtypes = [ctypes.c_void_p, ctypes.c_int64]
        lib.cm_reserved_len.restype = ctypes.c_int64
        for name in ("cm_num_free_pages", "cm_num_pages"):
            getattr(lib, name).argtypes = [ctypes.c_void_p, ctypes.c_int]
        for name in ("cm_num_groups", "cm_num_free_slots", "cm_num_requests", "cm_check"):
            getattr(lib, name).argtypes = [ctypes.c_void_p]
        lib.cm_table.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p, ctypes.c_int]
        lib.cm_fill_step.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p,
                                     ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int]
        lib.cm_reserve_all.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p,
                                       ctypes.c_void_p, ctypes.c_void_p]
        lib.cm_release_behind_all.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
        lib.cm_pack_step.argtypes = [ctypes.c_void_p, ctypes.c_int] + [ctypes.c_void_p] * 9 + [ctypes.c_int]
        _lib = lib
    return _lib


def _i32(values: Sequence[int]) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(list(values), dtype=np.int32))


class CacheManager:
    """Pages per group and state slots per request.

    * ``add(id)`` registers a request and returns its state slot;
    * ``reserve(id, length)`` makes every group cover positions [0, length), all groups or none;
    * ``release_behind(id, computed)`` gives back pages that a window has passed;
    * ``free(id)`` gives back everything (an unknown id is an error, so a double free is caught).
    """

    def __init__(self, groups: Sequence[GroupGeometry], num_state_slots: int):
        self.groups = list(groups)
        self.num_state_slots = int(num_state_slots)
        lib = _host()
        ps, npg = _i32(g.page_size for g in groups), _i32(g.num_pages for g in groups)
        win = _i32((g.window or 0) for g in groups)
        self._h = lib.cm_create(len(self.groups), ps.ctypes.data, npg.ctypes.data, win.ctypes.data,
                                self.num_state_slots)
        if not self._h:
            raise CacheError(f"invalid cache geometry: {self.groups}, {num_state_slots} state slots")
        self._lib = lib

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.cm_destroy(h)

    @property
    def handle(self):
        """The native manager, for other parts of the host library (the scheduler takes its pages from it)."""
        return self._h

    # -- requests ------------------------------------------------------------------------------------
    def add(self, request: int) -> int:
        rc = self._lib.cm_add_request(self._h, request)
        if rc == -2:
            raise CacheError(f"request {request} is already registered")
        if rc == -4:
            raise OutOfPages("no state slot is free")
        return rc

    def has(self, request: int) -> bool:
        return self._lib.cm_state_slot(self._h, request) >= 0

    def state_slot(self, request: int) -> int:
        rc = self._lib.cm_state_slot(self._h, request)
        if rc < 0:
            raise CacheError(f"request {request} is not registered")
        return rc

    def can_reserve(self, request: int, length: int) -> bool:
        return bool(self._lib.cm_can_reserve(self._h, request, length))

    def fits_at_all(self, length: int) -> bool:
        """Whether a request of ``length`` tokens could be held with every page free."""
        return bool(self._lib.cm_fits_at_all(self._h, length))

    def can_admit(self, total: int, first: int) -> bool:
        """Whether a new request of ``total`` tokens may start with a portion of ``first``: pages for the portion
        and, in groups with a window, room for the window (and one page) of the newcomer and of everyone held."""
        return bool(self._lib.cm_can_admit(self._h, total, first))

    def reserve(self, request: int, length: int) -> None:
        rc = self._lib.cm_reserve(self._h, request, length)
        if rc == -1:
            raise OutOfPages(f"request {request}: not enough free pages to reach {length} tokens")
        if rc != 0:
            raise CacheError(f"reserve({request}, {length}) failed with code {rc}")

    def reserve_all(self, ids: np.ndarray, starts: np.ndarray, counts: np.ndarray) -> None:
        """``reserve(ids[e], starts[e] + counts[e])`` for every entry of a step, in one call."""
        failed = ctypes.c_int(-1)
        rc = self._lib.cm_reserve_all(self._h, len(ids), ids.ctypes.data, starts.ctypes.data, counts.ctypes.data,
                                      ctypes.byref(failed))
        if rc == 0:
            return
        e = failed.value
        what = f"request {int(ids[e])}" if e >= 0 else "a request"
        if rc == -1:
            raise OutOfPages(f"{what}: not enough free pages to reach {int(starts[e]) + int(counts[e])} tokens")
        raise CacheError(f"reserving for {what} failed with code {rc}")

    def release_behind_all(self, ids: np.ndarray, done: np.ndarray) -> None:
        """``release_behind(ids[e], done[e])`` for every entry of a step, in one call."""
        if self._lib.cm_release_behind_all(self._h, len(ids), ids.ctypes.data, done.ctypes.data) != 0:
            raise CacheError("a request of the step is not registered")

    def reserved_len(self, request: int) -> int:
        rc = self._lib.cm_reserved_len(self._h, request)
        if rc < 0:
            raise CacheError(f"request {request} is not registered")
        return rc

    def release_behind(self, request: int, computed: int) -> int:
        rc = self._lib.cm_release_behind(self._h, request, computed)
        if rc < 0:
            raise CacheError(f"request {request} is not registered")
        return rc

    def free(self, request: int) -> None:
        if self._lib.cm_free(self._h, request) != 0:
            raise CacheError(f"request {request} is not registered (freed twice?)")

    # -- inspection ----------------------------------------------------------------------------------
    def num_free_pages(self, group: int = 0) -> int:
        return self._lib.cm_num_free_pages(self._h, group)

    def num_pages(self, group: int = 0) -> int:
        return self._lib.cm_num_pages(self._h, group)

    def num_free_slots(self) -> int:
        return self._lib.cm_num_free_slots(self._h)

    def num_requests(self) -> int:
        return self._lib.cm_num_requests(self._h)

    def table(self, request: int, group: int = 0) -> List[int]:
        n = self._lib.cm_table(self._h, request, group, None, 0)
        if n < 0:
            raise CacheError(f"request {request} is not registered")
        out = np.zeros(max(n, 1), dtype=np.int32)
        self._lib.cm_table(self._h, request, group, out.ctypes.data, n)
        return out[:n].tolist()

    def check(self) -> None:
        """Raise if a page or slot is lost, held twice or both free and held."""
        if self._lib.cm_check(self._h) != 0:
            raise CacheError("the cache manager's books are inconsistent")

    # -- step metadata -------------------------------------------------------------------------------
    def fill_step(self, group: int, ids: np.ndarray, starts: np.ndarray, counts: np.ndarray,
                  slot_mapping: np.ndarray, block_tables: np.ndarray) -> None:
        """Write the slots of every token and the padded block table of every entry (int32 arrays, in place)."""
        assert ids.dtype == np.int64 and starts.dtype == np.int32 and counts.dtype == np.int32
        assert slot_mapping.dtype == np.int32 and block_tables.dtype == np.int32 and block_tables.ndim == 2
        assert slot_mapping.flags.c_contiguous and block_tables.flags.c_contiguous
        assert block_tables.shape[0] >= len(ids) and slot_mapping.size >= int(counts.sum())
        rc = self._lib.cm_fill_step(self._h, group, len(ids), ids.ctypes.data, starts.ctypes.data, counts.ctypes.data,
                                    slot_mapping.ctypes.data, block_tables.ctypes.data, block_tables.shape[1])
        if rc == -1:
            raise CacheError("a token of the step has no page (reserve before the step; was its page released?)")
        if rc != 0:
            raise CacheError(f"fill_step failed with code {rc}")

    def pack_step(self, ids: np.ndarray, starts: np.ndarray, counts: np.ndarray, tokens: np.ndarray,
                  feeds: np.ndarray, want_counts: np.ndarray, wants: np.ndarray, buf: np.ndarray,
                  offsets: np.ndarray, max_blocks: int) -> int:
        """Write a step's metadata into the int32 staging buffer ``buf``: token ids, positions, entry per token,
        first row and length per entry, state slots, wanted rows, and per group the cache slots and block tables
        (``fill_step``); ``offsets`` (int64) says where each array starts, in the order of ``cm_pack_step``.
        Returns the number of (row, feed) pairs written."""
        assert ids.dtype == np.int64 and offsets.dtype == np.int64 and buf.dtype == np.int32
        for a in (starts, counts, tokens, feeds, want_counts, wants):
            assert a.dtype == np.int32 and a.flags.c_contiguous
        rc = self._lib.cm_pack_step(self._h, len(ids), ids.ctypes.data, starts.ctypes.data, counts.ctypes.data,
                                    tokens.ctypes.data, feeds.ctypes.data, want_counts.ctypes.data, wants.ctypes.data,
                                    buf.ctypes.data, offsets.ctypes.data, int(max_blocks))
        if rc == -1:
            raise CacheError("a token of the step has no page (reserve before the step; was its page released?)")
        if rc < 0:
            raise CacheError(f"packing the step failed with code {rc}")
        return rc
