"""The cache manager: paged keys and values with a block table per request, per-request state
slots, and the contiguous (buddy) mode as a second way of handing out the same pages.

Layout.  Mixer calls with the same needs (:class:`~..parts.base.KVCacheSpec`: the arrays kept per
token - names, per-token shapes, layout inside a page - and whether all positions stay or a
window of them) form a *group*.  A group owns a pool of ``num_pages`` pages and one block table
``[seats, max_blocks]``; a page holds ``page_size`` tokens of every array of every cache slot of
the group (slot = one mixer call's arrays, each ``[pages, *page_shape]``: for attention a K array
``[pages, kv_heads, page_size, head_dim]`` and a V array ``[pages, kv_heads, head_dim,
page_size]``), so one table row serves all layers of the group.  Groups with other needs have
pools and tables of their own.  The manager allocates what the description says and hands the
arrays over by name; it never looks inside them.

Paged mode (reference: ``paged_attention/src/engine.cu:176-254, 376-454``): pages are taken one
by one as a request grows, dropped when it ends or - in a window group - once every position
on them lies behind the window, and reused at once (the free stack is LIFO).

Contiguous mode (reference: ``base/src/engine.cu:257-375``): at admission a request reserves,
per group, one buddy-allocated power-of-two run of pages that it keeps until it ends; its block
table row is simply ``start, start+1, ...``.  The kernels are the same in both modes; what
differs is how much is reserved against how much holds a token, which is what the reference's
comparison measures.

Seats.  A live request holds a seat: its row in every block table and its index into the state
arena, where each mixer call that asked for a :class:`~..parts.base.StateSpec` has a
``[seats, *shape]`` tensor.  A seat's state rows are zeroed when the seat is taken.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from ..parts.base import KVCacheSpec, StateSpec
from .allocators import BuddyAllocator, CacheAccountingError, PagePool


class CacheError(RuntimeError):
    pass


def page_bytes(group_specs, page_size: int, dtype) -> int:
    """Bytes of one page over all groups: every array of every cache slot, ``page_size`` tokens."""
    return sum(len(slots) * spec.bytes_per_token(dtype) * int(page_size) for spec, slots in group_specs)


@dataclass
class _Seat:
    request_id: object
    length: int = 0                                     # tokens whose K/V are in the cache
    next_block: List[int] = field(default_factory=list)  # per group: first logical block not mapped yet
    first_block: List[int] = field(default_factory=list)  # per group: first logical block still mapped
    run: List[Optional[Tuple[int, int]]] = field(default_factory=list)  # contiguous: (start, pages)
    mapped_tokens: int = 0                              # paged: positions below this have a page in every group


class CacheGroup:
    def __init__(self, index: int, spec: KVCacheSpec, slot_ids: Sequence[int], page_size: int,
                 num_pages: int, max_seqs: int, max_blocks: int, mode: str):
        self.index, self.spec, self.slot_ids = index, spec, list(slot_ids)
        self.page_size, self.num_pages, self.max_blocks = page_size, num_pages, max_blocks
        self.pool = PagePool(num_pages) if mode == "paged" else None
        self.buddy = BuddyAllocator(num_pages) if mode == "contiguous" else None
        self.table_host = np.full((max_seqs, max_blocks), -1, dtype=np.int32)
        self.table_dev = None
        self._table_pinned = None
        self.arrays: Dict[str, object] = {}     # name -> [slots, pages, *page_shape] on the device
        self.dirty: Dict[int, List[int]] = {}

    def free_pages(self) -> int:
        return self.pool.free_count if self.pool is not None else self.buddy.free_units

    def pages_for(self, tokens: int, portion: Optional[int] = None) -> int:
        """Most pages one request holds in this group at any time while a prompt of ``tokens``
        tokens is brought in by steps of at most ``portion`` tokens.  All keys stay: one page per
        ``page_size`` tokens.  A window group keeps only what the newest position can still see
        plus the step being written, whatever the prompt's length: ``window - 1 + portion``
        positions, which touch one page more than they fill when they straddle page edges."""
        whole = (tokens + self.page_size - 1) // self.page_size
        if self.spec.kind != "window" or self.spec.window <= 0:
            return whole
        step = min(tokens, portion) if portion else tokens
        span = self.spec.window - 1 + step
        return min(whole, (span + self.page_size - 1) // self.page_size + 1)

    def mark_dirty(self, seat: int, lo: int, hi: int) -> None:
        d = self.dirty.get(seat)
        if d is None:
            self.dirty[seat] = [lo, hi]
        else:
            d[0], d[1] = min(d[0], lo), max(d[1], hi)

    def slot_of(self, cache_slot: int) -> int:
        return self.slot_ids.index(cache_slot)


class CacheManager:
    def __init__(self, group_specs: Sequence[Tuple[KVCacheSpec, Sequence[int]]],
                 state_specs: Dict[int, StateSpec], *, page_size: int, num_pages: int,
                 max_seqs: int, max_seq_len: int, mode: str = "paged", device=None, dtype=None):
        if mode not in ("paged", "contiguous"):
            raise CacheError(f"cache mode {mode!r} is not one of 'paged', 'contiguous'")
        if page_size <= 0 or num_pages <= 0 or max_seqs <= 0 or max_seq_len <= 0:
            raise CacheError("page_size, num_pages, max_seqs and max_seq_len must be positive")
        self.mode, self.page_size, self.num_pages = mode, page_size, num_pages
        self.max_seqs, self.max_seq_len = max_seqs, max_seq_len
        self.max_blocks = (max_seq_len + page_size - 1) // page_size
        self.device, self.dtype = device, dtype
        self.groups = [CacheGroup(i, spec, slots, page_size, num_pages, max_seqs, self.max_blocks, mode)
                       for i, (spec, slots) in enumerate(group_specs)]
        self.state_specs = dict(state_specs)
        self.state: Dict[int, object] = {}
        self._seats: List[Optional[_Seat]] = [None] * max_seqs
        self._free_seats = list(range(max_seqs - 1, -1, -1))   # popped from the back: lowest first
        self.peak_held_pages = 0
        self._no_pages = [0] * len(self.groups)     # shared answer of pages_needed; never modified
        self._flush_event = None     # set while an upload of table spans may still be reading the host table
        if device is not None:
            self._allocate_device()

    # ------------------------------------------------------------------ device memory
    def _allocate_device(self) -> None:
        import torch
        for g in self.groups:
            for a in g.spec.arrays:
                g.arrays[a.name] = torch.zeros((len(g.slot_ids), g.num_pages, *a.page_shape(g.page_size)),
                                               dtype=a.dtype or self.dtype, device=self.device)
            pinned = torch.full((self.max_seqs, self.max_blocks), -1, dtype=torch.int32,
                                pin_memory=True)
            g._table_pinned = pinned
            g.table_host = pinned.numpy()
            g.table_dev = torch.full((self.max_seqs, self.max_blocks), -1, dtype=torch.int32,
                                     device=self.device)
        for slot, spec in self.state_specs.items():
            self.state[slot] = torch.zeros((self.max_seqs, *spec.shape), dtype=spec.dtype,
                                           device=self.device)

    def flush_tables(self) -> None:
        """Brings the device block tables up to date (only the spans that changed)."""
        queued = False
        for g in self.groups:
            if g.table_dev is not None:
                for seat, (lo, hi) in g.dirty.items():
                    g.table_dev[seat, lo:hi].copy_(g._table_pinned[seat, lo:hi], non_blocking=True)
                    queued = True
            g.dirty.clear()
        if queued:
            import torch
            self._flush_event = torch.cuda.Event()
            self._flush_event.record()

    def _before_table_write(self) -> None:
        """The uploads read the pinned host table when they execute, not when they are queued: a
        caller that runs ahead of the device must not change the table under them."""
        if self._flush_event is not None:
            self._flush_event.synchronize()
            self._flush_event = None

    def kv_arrays(self, cache_slot: int):
        """(group, {array name: the slot's ``[pages, *page_shape]`` tensor})."""
        for g in self.groups:
            if cache_slot in g.slot_ids:
                i = g.slot_of(cache_slot)
                return g, {name: t[i] for name, t in g.arrays.items()}
        raise CacheError(f"cache slot {cache_slot} belongs to no group")

    def page_bytes(self) -> int:
        """Bytes one page takes over all groups, slots and arrays."""
        return page_bytes(((g.spec, g.slot_ids) for g in self.groups), self.page_size, self.dtype)

    def group_of(self, cache_slot: int) -> Optional[CacheGroup]:
        for g in self.groups:
            if cache_slot in g.slot_ids:
                return g
        return None

    # ------------------------------------------------------------------ seats
    @property
    def free_seats(self) -> int:
        return len(self._free_seats)

    def live_seats(self) -> List[int]:
        return [i for i, s in enumerate(self._seats) if s is not None]

    def seat(self, seat: int) -> _Seat:
        s = self._seats[seat] if 0 <= seat < self.max_seqs else None
        if s is None:
            raise CacheError(f"seat {seat} is not taken")
        return s

    def length(self, seat: int) -> int:
        return self.seat(seat).length

    def capacity_tokens(self, seat: int) -> int:
        """Most tokens this seat may ever hold."""
        s = self.seat(seat)
        cap = min(self.max_seq_len, self.max_blocks * self.page_size)
        if self.mode == "contiguous":
            for run in s.run:
                cap = min(cap, run[1] * self.page_size)
        return cap

    def admit(self, request_id, reserve_tokens: Optional[int] = None) -> Optional[int]:
        """Takes a seat for a request; ``None`` when no seat is free or (contiguous mode) the
        reservation of ``reserve_tokens`` tokens cannot be placed."""
        if not self._free_seats:
            return None
        self._before_table_write()
        ng = len(self.groups)
        st = _Seat(request_id, 0, [0] * ng, [0] * ng, [None] * ng)
        seat = self._free_seats[-1]
        if self.mode == "contiguous":
            if reserve_tokens is None or reserve_tokens <= 0:
                raise CacheError("contiguous mode reserves at admission: reserve_tokens is needed")
            pages = (min(reserve_tokens, self.max_seq_len) + self.page_size - 1) // self.page_size
            placed = []
            for g in self.groups:
                start = g.buddy.alloc(pages)
                if start < 0:
                    for pg, (s0, n0) in placed:
                        pg.buddy.free(s0, n0)
                    return None
                size = g.buddy.round(pages)
                placed.append((g, (start, size)))
            for g, (start, size) in placed:
                st.run[g.index] = (start, size)
                n = min(size, self.max_blocks)
                g.table_host[seat, :n] = np.arange(start, start + n, dtype=np.int32)
                g.mark_dirty(seat, 0, n)
        self._free_seats.pop()
        self._seats[seat] = st
        for t in self.state.values():
            t[seat].zero_()
        self._note_peak()
        return seat

    def free(self, seat: int) -> None:
        """Gives back everything the seat holds."""
        s = self.seat(seat)
        self._before_table_write()
        for g in self.groups:
            gi = g.index
            if self.mode == "paged":
                lo, hi = s.first_block[gi], s.next_block[gi]
                pages = [int(p) for p in g.table_host[seat, lo:hi] if p >= 0]
                g.pool.drop(pages)
                if hi > 0:
                    g.table_host[seat, :hi] = -1
                    g.mark_dirty(seat, 0, hi)
            else:
                start, size = s.run[gi]
                g.buddy.free(start, size)
                n = min(size, self.max_blocks)
                g.table_host[seat, :n] = -1
                g.mark_dirty(seat, 0, n)
        self._seats[seat] = None
        self._free_seats.append(seat)
        self._free_seats.sort(reverse=True)

    # ------------------------------------------------------------------ growth
    def pages_needed(self, seat: int, new_len: int) -> List[int]:
        """Pages each group must still map so that positions ``< new_len`` have a place."""
        s = self.seat(seat)
        if self.mode == "contiguous" or new_len <= s.mapped_tokens:
            return self._no_pages
        blocks = (new_len + self.page_size - 1) // self.page_size
        return [max(0, blocks - s.next_block[g.index]) for g in self.groups]

    def pages_outstanding(self, seat: int, final_len: int, portion: Optional[int] = None) -> List[int]:
        """Pages each group may still have to find for this seat until ``final_len`` tokens are in
        the cache (a prompt is mapped portion by portion): what the group needs at most at one
        time, less what the seat holds now."""
        s = self.seat(seat)
        if self.mode == "contiguous":
            return self._no_pages
        return [max(0, g.pages_for(final_len, portion) - (s.next_block[g.index] - s.first_block[g.index]))
                for g in self.groups]

    def can_grow(self, seat: int, new_len: int) -> bool:
        if new_len > self.capacity_tokens(seat):
            return False
        if self.mode == "contiguous":
            return True
        need = self.pages_needed(seat, new_len)
        return all(n <= g.free_pages() for n, g in zip(need, self.groups))

    def grow(self, seat: int, new_len: int) -> bool:
        """Maps pages so positions ``< new_len`` can be written.  All groups or none."""
        s = self.seat(seat)
        if self.mode == "paged" and new_len <= s.mapped_tokens:
            return True         # the common decode step: the page is there already
        if new_len > self.capacity_tokens(seat):
            return False
        if self.mode == "contiguous":
            return True
        need = self.pages_needed(seat, new_len)
        if any(n > g.free_pages() for n, g in zip(need, self.groups)):
            return False
        if any(need):
            self._before_table_write()
        for n, g in zip(need, self.groups):
            if n == 0:
                continue
            pages = g.pool.take(n)
            if pages is None:   # cannot happen after the check above
                raise CacheAccountingError("page pool refused pages it reported free")
            lo = s.next_block[g.index]
            if (g.table_host[seat, lo:lo + n] != -1).any():
                raise CacheAccountingError(f"seat {seat}: a block about to be mapped is mapped already")
            g.table_host[seat, lo:lo + n] = np.asarray(pages, dtype=np.int32)
            g.mark_dirty(seat, lo, lo + n)
            s.next_block[g.index] = lo + n
        # never past the longest sequence; a model without any paged group has a place for all of them
        mapped = min(s.next_block) * self.page_size if s.next_block else new_len
        s.mapped_tokens = min(mapped, self.capacity_tokens(seat))
        self._note_peak()
        return True

    def slot_mapping(self, seat: int, start: int, count: int, group: int) -> np.ndarray:
        """Cache slots (page * page_size + row) of positions ``start .. start+count-1``."""
        g = self.groups[group]
        pos = np.arange(start, start + count, dtype=np.int64)
        pages = g.table_host[seat, pos // self.page_size].astype(np.int64)
        if (pages < 0).any():
            raise CacheError(f"seat {seat}: positions {start}..{start + count - 1} are not all mapped "
                             f"in group {group}")
        return (pages * self.page_size + pos % self.page_size).astype(np.int32)

    def slot_mapping_each(self, seats: np.ndarray, positions: np.ndarray, group: int) -> np.ndarray:
        """Cache slots of one position per seat (a decode step), in one go."""
        g = self.groups[group]
        pages = g.table_host[seats, positions // self.page_size].astype(np.int64)
        if (pages < 0).any():
            bad = int(np.nonzero(pages < 0)[0][0])
            raise CacheError(f"seat {int(seats[bad])}: position {int(positions[bad])} is not mapped in group {group}")
        return (pages * self.page_size + positions % self.page_size).astype(np.int32)

    def commit(self, seat: int, new_len: int) -> None:
        """The step wrote positions up to ``new_len``; window groups give back what lies behind."""
        s = self.seat(seat)
        if new_len < s.length:
            raise CacheError(f"seat {seat}: length cannot shrink ({s.length} -> {new_len})")
        s.length = new_len
        if self.mode != "paged":
            return
        for g in self.groups:
            if g.spec.kind != "window" or g.spec.window <= 0:
                continue
            # the next query sits at position >= new_len and reads keys >= new_len - window + 1
            keep_from = max(0, new_len - g.spec.window + 1) // self.page_size
            lo = s.first_block[g.index]
            hi = min(keep_from, s.next_block[g.index])
            if hi > lo:
                self._before_table_write()
                pages = [int(p) for p in g.table_host[seat, lo:hi] if p >= 0]
                g.pool.drop(pages)
                g.table_host[seat, lo:hi] = -1
                g.mark_dirty(seat, lo, hi)
                s.first_block[g.index] = hi

    # ------------------------------------------------------------------ books
    def _note_peak(self) -> None:
        held = sum(g.num_pages - g.free_pages() for g in self.groups)
        self.peak_held_pages = max(self.peak_held_pages, held)

    def stats(self) -> dict:
        """Occupancy in tokens, as the reference's step telemetry reports it
        (``paged_attention/src/engine.cu:755-768``, ``base/src/engine.cu:513-525``)."""
        g0 = self.groups[0] if self.groups else None
        live = sum(s.length for s in self._seats if s is not None)
        out = {
            "running": self.max_seqs - len(self._free_seats),
            "kv_tokens_live": live,
            "kv_tokens_total": self.num_pages * self.page_size,
            "kv_tokens_reserved": 0 if g0 is None else (g0.num_pages - g0.free_pages()) * self.page_size,
            "fragmentation_failures": 0,
            "pages_reused": 0,
        }
        if g0 is not None and g0.buddy is not None:
            out["fragmentation_failures"] = sum(g.buddy.fragmentation_failures for g in self.groups)
        if g0 is not None and g0.pool is not None:
            out["pages_reused"] = sum(g.pool.reuses for g in self.groups)
        return out

    def check(self) -> None:
        """Raises unless no page is lost, held twice or mapped while free."""
        for g in self.groups:
            mapped: Dict[int, int] = {}
            for seat, s in enumerate(self._seats):
                row = g.table_host[seat]
                if s is None:
                    if (row != -1).any():
                        raise CacheAccountingError(f"group {g.index}: free seat {seat} still maps pages")
                    continue
                if self.mode == "paged":
                    lo, hi = s.first_block[g.index], s.next_block[g.index]
                    if (row[:lo] != -1).any() or (row[hi:] != -1).any() or (row[lo:hi] < 0).any():
                        raise CacheAccountingError(
                            f"group {g.index}: seat {seat} maps blocks outside [{lo}, {hi})")
                for p in row[row >= 0]:
                    mapped[int(p)] = mapped.get(int(p), 0) + 1
            if self.mode == "paged":
                if not g.pool.accounting_holds():
                    raise CacheAccountingError(f"group {g.index}: free stack and reference counts disagree")
                for p, n in mapped.items():
                    if g.pool.refcount(p) != n:
                        raise CacheAccountingError(
                            f"group {g.index}: page {p} is mapped {n} times but held "
                            f"{g.pool.refcount(p)} times")
                if len(mapped) != g.pool.held_count:
                    raise CacheAccountingError(
                        f"group {g.index}: {g.pool.held_count} pages are held but {len(mapped)} are mapped")
            else:
                if any(n != 1 for n in mapped.values()):
                    raise CacheAccountingError(f"group {g.index}: two seats share a page of their runs")
                reserved = sum(s.run[g.index][1] for s in self._seats if s is not None)
                if reserved != g.buddy.reserved_units or reserved + g.buddy.free_units != g.num_pages:
                    raise CacheAccountingError(
                        f"group {g.index}: reserved {reserved} + free {g.buddy.free_units} pages "
                        f"do not add up to {g.num_pages}")
