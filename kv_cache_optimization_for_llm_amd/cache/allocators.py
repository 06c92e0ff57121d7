"""Python faces of the native allocators (``csrc/host/cache_alloc.cpp``)."""
from __future__ import annotations

import ctypes
from typing import List, Sequence, Tuple

from ..ops.library import host_lib


class CacheAccountingError(RuntimeError):
    """A page was freed twice, freed without being held, or the pool's books do not add up."""


class PagePool:
    """Fixed-size pages, LIFO free stack, per-page reference counts
    (reference: ``paged_attention/src/engine.cu:376-404``)."""

    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise ValueError(f"a page pool needs at least one page, got {num_pages}")
        self._lib = host_lib()
        self._h = self._lib.kva_pool_create(num_pages)
        if not self._h:
            raise MemoryError("page pool could not be created")
        self.num_pages = num_pages

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.kva_pool_destroy(h)

    @property
    def free_count(self) -> int:
        return self._lib.kva_pool_free_count(self._h)

    @property
    def held_count(self) -> int:
        return self.num_pages - self.free_count

    @property
    def takes(self) -> int:
        return self._lib.kva_pool_takes(self._h)

    @property
    def reuses(self) -> int:
        return self._lib.kva_pool_reuses(self._h)

    def take(self, n: int) -> List[int] | None:
        """``n`` pages, or ``None`` (and nothing taken) when fewer are free."""
        if n == 0:
            return []
        buf = (ctypes.c_int * n)()
        if self._lib.kva_pool_take(self._h, n, buf) != 0:
            return None
        return list(buf)

    def share(self, page: int) -> int:
        rc = self._lib.kva_pool_share(self._h, page)
        if rc < 0:
            raise CacheAccountingError(f"page {page} is not held and cannot be shared")
        return rc

    def drop(self, pages: Sequence[int]) -> int:
        n = len(pages)
        if n == 0:
            return 0
        buf = (ctypes.c_int * n)(*pages)
        freed = self._lib.kva_pool_drop(self._h, buf, n)
        if freed < 0:
            raise CacheAccountingError(f"page {pages[-1 - freed]} was dropped while not held "
                                       "(freed twice, or never taken)")
        return freed

    def refcount(self, page: int) -> int:
        return self._lib.kva_pool_refcount(self._h, page)

    def accounting_holds(self) -> bool:
        return bool(self._lib.kva_pool_accounting_holds(self._h))


class BuddyAllocator:
    """Binary buddy allocator over ``pool_units`` units (reference: ``base/src/engine.cu:169-254``)."""

    def __init__(self, pool_units: int):
        if pool_units <= 0:
            raise ValueError(f"a buddy pool needs at least one unit, got {pool_units}")
        self._lib = host_lib()
        self._h = self._lib.kva_buddy_create(pool_units)
        if not self._h:
            raise MemoryError("buddy allocator could not be created")
        self.pool_units = pool_units

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.kva_buddy_destroy(h)

    def round(self, units: int) -> int:
        return self._lib.kva_buddy_round(units)

    def alloc(self, units: int) -> int:
        """Start of a self-aligned run of ``round(units)`` units, or -1."""
        return self._lib.kva_buddy_alloc(self._h, units)

    def free(self, start: int, units: int) -> None:
        if self._lib.kva_buddy_free(self._h, start, units) != 0:
            raise CacheAccountingError(f"run ({start}, {units}) is not an allocated run (freed twice?)")

    @property
    def free_units(self) -> int:
        return self._lib.kva_buddy_free_units(self._h)

    @property
    def reserved_units(self) -> int:
        return self._lib.kva_buddy_reserved_units(self._h)

    @property
    def fragmentation_failures(self) -> int:
        return self._lib.kva_buddy_fragmentation_failures(self._h)

    def free_runs(self) -> List[Tuple[int, int]]:
        """Free runs as (start, size), sorted by start."""
        cap = 64
        while True:
            buf = (ctypes.c_int * (2 * cap))()
            n = self._lib.kva_buddy_free_runs(self._h, buf, cap)
            if n <= cap:
                return [(buf[2 * i], 1 << buf[2 * i + 1]) for i in range(n)]
            cap = n
