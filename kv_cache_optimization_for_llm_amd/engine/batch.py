"""One step's batch: a flat run of tokens from several requests, with the index arrays the
kernels need.

An entry is (request, its next tokens, the places among them whose logits are wanted).  Entries
may be portions of prompts of any length beside single decoded tokens.  The reference builds
comparable arrays for its prefill pass (``base/src/engine.cu:574-633``: token_positions,
token_slot_ids, last_token_rows) and its decode pass (``:1013-1029``); here one layout serves
both.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Sequence

import numpy as np
import torch


@dataclass
class StepEntry:
    request_id: object
    tokens: Sequence[int]           # a single token may be ``feedback_token(r)``: row r of the
                                    # engine's feedback buffer, a token still on the device
    want: Sequence[int] = ()        # indices into ``tokens`` whose logits are returned


def feedback_token(row: int) -> int:
    """The id that stands for 'the token in row ``row`` of the engine's feedback buffer'."""
    return -1 - int(row)


@dataclass
class StepBatch:
    num_tokens: int
    num_entries: int
    num_logit_rows: int
    # device int32 arrays
    token_ids: torch.Tensor          # [T]
    positions: torch.Tensor          # [T] absolute position inside the own request
    tok_seat: torch.Tensor           # [T] seat (block-table row, state row) of the token's request
    logit_rows: torch.Tensor         # [R] rows whose logits are wanted, in entry order
    slot_mapping: List[torch.Tensor]  # per cache group: [T] cache slot to write
    entry_seat: torch.Tensor         # [E]
    entry_q_start: torch.Tensor      # [E + 1] first row of each entry (last = T)
    entry_start_pos: torch.Tensor    # [E] position of the entry's first token
    # host copies of the same
    h_positions: np.ndarray = field(repr=False, default=None)
    h_tok_seat: np.ndarray = field(repr=False, default=None)
    h_entry_seat: np.ndarray = field(repr=False, default=None)
    h_entry_q_start: np.ndarray = field(repr=False, default=None)
    h_entry_start_pos: np.ndarray = field(repr=False, default=None)
    max_q_len: int = 0
    min_q_len: int = 0
    max_context: int = 0
    logits_for_all_rows: bool = False    # logit_rows is exactly 0, 1, ..., T-1
    feedback: torch.Tensor = None        # device int32: tokens that negative token_ids stand for
    meta_provider: object = None         # callable(group, row_tiles) -> attention items, or None
    static_items: bool = False           # a captured step: every set of attention items is prepared ahead
    _items: Dict[tuple, tuple] = field(default_factory=dict, repr=False)
    # the attention launches decided for this step, per geometry (ops.attention.paged_attention)
    attention_plans: Dict[tuple, list] = field(default_factory=dict, repr=False)

    def attention_items(self, group: int, row_tiles: int = 1, which: str = "all"):
        """Work items of the matrix-core attention kernels for a query-head group size: (entry,
        first row) of every ``16 * row_tiles`` query rows, row = token_in_step * group +
        head_in_group; ordered by the number of keys an item visits, most first (when the
        entries' start positions are known on the host).  ``which`` takes all entries, only the
        ``"long"`` ones (more than 16 query rows: prompt portions) or only the ``"short"`` ones
        (decoded tokens).  Returns ``(entry, row0, meta)``; ``meta`` ``[items, 8]`` repeats per
        item what the kernel would otherwise look up through the entry (q_start, q_len,
        start_pos, seat, row0), or is ``None`` when the host does not know it."""
        key = (group, row_tiles, which)
        if key not in self._items:
            if self.meta_provider is not None and which == "all":
                made = self.meta_provider(group, row_tiles)
                if made is not None:
                    self._items[key] = made
                    return made
            if self.static_items:
                raise RuntimeError(f"attention items {key} were not prepared for this captured step")
            ent, row0, meta = attention_work_items(self.h_entry_q_start, self.h_entry_start_pos,
                                                   self.h_entry_seat, group, row_tiles, which)
            n = ent.shape[0]
            parts = [ent, row0] + ([meta.reshape(-1)] if meta is not None else [])
            flat = np.concatenate(parts)
            staging = torch.empty(flat.shape[0], dtype=torch.int32, pin_memory=True)      # (a pageable source makes the copy wait)
            staging.numpy()[:] = flat
            dev = staging.to(self.token_ids.device, non_blocking=True)
            self._items[key] = (dev[:n], dev[n:2 * n], dev[2 * n:].view(n, 8) if meta is not None else None)
        return self._items[key]

    def mean_keys_of_long_entries(self) -> float:
        """Average number of keys a query token of the prompt portions visits (host estimate)."""
        lens = np.diff(self.h_entry_q_start).astype(np.float64)
        if self.h_entry_start_pos is None:
            return float(self.max_context)
        long = lens > 1
        if not long.any():
            return 0.0
        return float(((self.h_entry_start_pos[long] + (lens[long] + 1) / 2) * lens[long]).sum() / lens[long].sum())


def attention_work_items(entry_q_start: np.ndarray, entry_start_pos, entry_seat, group: int,
                         row_tiles: int, which: str):
    """Host arrays ``(entry, row0, meta)`` of :meth:`StepBatch.attention_items`; ``meta`` is
    ``None`` when start positions or seats are not known on the host.  The number of items depends
    on the entries' lengths, ``group``, ``row_tiles`` and ``which`` alone."""
    lens = np.diff(entry_q_start)
    ent, row0 = [np.zeros(0, np.int32)], [np.zeros(0, np.int32)]
    for e, n in enumerate(lens):
        if which != "all" and (int(n) * group > 16) != (which == "long"):
            continue
        starts = np.arange(0, int(n) * group, 16 * row_tiles, dtype=np.int32)
        ent.append(np.full(starts.shape[0], e, dtype=np.int32))
        row0.append(starts)
    ent, row0 = np.concatenate(ent), np.concatenate(row0)
    n = ent.shape[0]
    if entry_start_pos is None or entry_seat is None:
        return ent, row0, None
    if n > 1:
        # most keys first: the kernel hands out items in list order (and may give a
        # wavefront the i-th and the i-th last), so the long ones should start early
        last_row = np.minimum(row0 + 16 * row_tiles, lens[ent] * group) - 1
        keys = entry_start_pos[ent] + last_row // group + 1
        order = np.argsort(-keys, kind="stable")
        ent, row0 = ent[order], row0[order]
    meta = np.zeros((n, 8), dtype=np.int32)
    meta[:, 0] = entry_q_start[:-1][ent]
    meta[:, 1] = lens[ent]
    meta[:, 2] = entry_start_pos[ent]
    meta[:, 3] = entry_seat[ent]
    meta[:, 4] = row0
    return ent, row0, meta


def _align(n: int, a: int = 4) -> int:
    return (n + a - 1) // a * a


def build_batch(seats: Sequence[int], starts: Sequence[int], token_lists: Sequence[Sequence[int]],
                wants: Sequence[Sequence[int]], slot_maps: Sequence[Sequence[np.ndarray]],
                device) -> StepBatch:
    """Packs the index arrays into one pinned staging buffer and uploads it with one copy.

    ``slot_maps[g][e]`` is the slot array of entry ``e`` in cache group ``g``."""
    E = len(seats)
    lens = [len(t) for t in token_lists]
    T = int(sum(lens))
    q_start = np.zeros(E + 1, dtype=np.int32)
    np.cumsum(lens, out=q_start[1:])
    token_ids = np.concatenate([np.asarray(t, dtype=np.int32) for t in token_lists]) if T else np.zeros(0, np.int32)
    positions = np.concatenate([np.arange(s, s + n, dtype=np.int32) for s, n in zip(starts, lens)]) \
        if T else np.zeros(0, np.int32)
    tok_seat = np.repeat(np.asarray(seats, dtype=np.int32), lens)
    rows: List[int] = []
    for e, w in enumerate(wants):
        for i in w:
            if not 0 <= i < lens[e]:
                raise ValueError(f"entry {e}: wanted place {i} is outside its {lens[e]} tokens")
            rows.append(int(q_start[e]) + int(i))
    logit_rows = np.asarray(rows, dtype=np.int32)
    G = len(slot_maps)
    segs: Dict[str, np.ndarray] = {
        "token_ids": token_ids, "positions": positions, "tok_seat": tok_seat,
        "logit_rows": logit_rows, "entry_seat": np.asarray(seats, dtype=np.int32),
        "entry_q_start": q_start, "entry_start_pos": np.asarray(starts, dtype=np.int32),
    }
    for g in range(G):
        segs[f"slots{g}"] = np.concatenate(slot_maps[g]).astype(np.int32) if T else np.zeros(0, np.int32)
    offsets, total = {}, 0
    for name, arr in segs.items():
        offsets[name] = total
        total += _align(max(1, arr.shape[0]))
    staging = torch.empty(total, dtype=torch.int32, pin_memory=True)
    st_np = staging.numpy()
    for name, arr in segs.items():
        st_np[offsets[name]:offsets[name] + arr.shape[0]] = arr
    dev = staging.to(device, non_blocking=True)

    def view(name):
        return dev[offsets[name]:offsets[name] + segs[name].shape[0]]

    return StepBatch(
        num_tokens=T, num_entries=E, num_logit_rows=len(rows),
        token_ids=view("token_ids"), positions=view("positions"), tok_seat=view("tok_seat"),
        logit_rows=view("logit_rows"), slot_mapping=[view(f"slots{g}") for g in range(G)],
        entry_seat=view("entry_seat"), entry_q_start=view("entry_q_start"),
        entry_start_pos=view("entry_start_pos"),
        h_positions=positions, h_tok_seat=tok_seat, h_entry_seat=segs["entry_seat"],
        h_entry_q_start=q_start, h_entry_start_pos=segs["entry_start_pos"],
        logits_for_all_rows=rows == list(range(T)),
        max_q_len=max(lens) if lens else 0, min_q_len=min(lens) if lens else 0,
        max_context=max((s + n for s, n in zip(starts, lens)), default=0),
    )
