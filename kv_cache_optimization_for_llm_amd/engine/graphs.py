"""HIP graphs for decode steps and for steps with prompt portions whose shape comes back.

A decode step of a small model is a few hundred short kernels; launched one by one the host
cannot keep the GPU busy.  For batches in which every entry brings exactly one token, the whole
forward pass is captured once per (number of entries, context bucket) into a HIP graph over
static index buffers; later steps of that shape copy their indices into the buffers (one small
host-to-device copy) and replay the graph.

Steps that hold prompt portions are eager the first time their shape (the entries' lengths, the
wanted places, the context bucket) is seen; from the second time on the shape has a graph of its
own (:class:`PortionGraphs`): launching the ~150 kernels of such a step one by one costs the host
more time than a portion of a few hundred tokens costs a small model on the device.

What is inside a graph: the model's kernels and the vendor GEMM calls.  What stays outside: the
upload of indices and block-table spans, sampling, and every allocation.  Nothing inside clears
memory with a memset node.
"""
from __future__ import annotations

import gc

from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from collections import OrderedDict

from .batch import StepBatch, attention_work_items


def context_bucket(max_context: int) -> int:
    """Contexts are bucketed to powers of two (at least 256) so that the number of key splits of
    the attention kernel - a launch parameter frozen into the graph - fits every step that
    replays it."""
    b = 256
    while b < max_context:
        b *= 2
    return b


class _DecodeSlot:
    """Static buffers, batch view and (once captured) the graph for one (entries, bucket) shape."""

    def __init__(self, n: int, bucket: int, num_groups: int, device, feedback=None):
        self.n, self.bucket = n, bucket
        # layout of the int32 staging buffer: token_ids, positions, tok_seat, entry_start_pos,
        # then one slot mapping per cache group; each n long
        # ... and, last, one record of 8 per entry for the attention kernel (q_start, q_len,
        # start_pos, seat, row0, 0, 0, 0): with at most 16 query heads per kv head a decoded
        # token is one work item, so the records can be written here every step
        self.fields = 4 + num_groups + 8
        self.staging = torch.zeros(self.fields * n, dtype=torch.int32, pin_memory=True)
        self.dev = torch.zeros(self.fields * n, dtype=torch.int32, device=device)
        self.meta_at = (4 + num_groups) * n
        self.const = torch.cat([torch.arange(n + 1, dtype=torch.int32),          # entry_q_start
                                torch.arange(n, dtype=torch.int32)]).to(device)   # logit rows
        v = lambda i: self.dev[i * n:(i + 1) * n]
        self.batch = StepBatch(
            num_tokens=n, num_entries=n, num_logit_rows=n,
            token_ids=v(0), positions=v(1), tok_seat=v(2), logit_rows=self.const[n + 1:],
            slot_mapping=[v(4 + g) for g in range(num_groups)],
            entry_seat=v(2), entry_q_start=self.const[:n + 1], entry_start_pos=v(3),
            max_q_len=1, min_q_len=1, max_context=bucket, logits_for_all_rows=True, feedback=feedback)
        # attention work items depend on this array only, so they are the same every step; the
        # eager warm-up run uploads them, the captured run finds them cached
        self.batch.h_entry_q_start = np.arange(n + 1, dtype=np.int32)
        items = torch.arange(n, dtype=torch.int32).to(device)
        zeros = torch.zeros(n, dtype=torch.int32, device=device)
        meta = self.dev[self.meta_at:self.meta_at + 8 * n].view(n, 8)
        self.batch.meta_provider = lambda group, row_tiles: \
            (items, zeros, meta) if group <= 16 and row_tiles == 1 else None
        m = self.staging.numpy()[self.meta_at:self.meta_at + 8 * n].reshape(n, 8)
        m[:, 0], m[:, 1] = np.arange(n), 1
        self.copied = torch.cuda.Event()
        self.graph: Optional[torch.cuda.CUDAGraph] = None
        self.logits: Optional[torch.Tensor] = None
        self.warm = False

    def fill(self, tokens: np.ndarray, positions: np.ndarray, seats: np.ndarray,
             slot_maps: Sequence[np.ndarray]) -> None:
        n = self.n
        self.copied.synchronize()        # the previous upload has left the staging buffer
        st = self.staging.numpy()
        st[0:n], st[n:2 * n], st[2 * n:3 * n], st[3 * n:4 * n] = tokens, positions, seats, positions
        for g, sm in enumerate(slot_maps):
            st[(4 + g) * n:(5 + g) * n] = sm
        m = st[self.meta_at:self.meta_at + 8 * n].reshape(n, 8)
        m[:, 2], m[:, 3] = positions, seats
        self.dev.copy_(self.staging, non_blocking=True)
        self.copied.record()


class DecodeGraphs:
    MAX_SHAPES = 256           # captured (entries, context bucket) shapes kept (least recently used goes first) ...
    MAX_KEPT_ROWS = 8192       # ... and the rows of all of them: a graph keeps its logits [entries, vocabulary]

    def __init__(self, model, cache, device, feedback=None):
        self.model, self.cache, self.device, self.feedback = model, cache, device, feedback
        self.slots: "OrderedDict[Tuple[int, int], _DecodeSlot]" = OrderedDict()
        self.replays = 0
        self.captures = 0

    def run(self, tokens: np.ndarray, positions: np.ndarray, seats: np.ndarray,
            slot_maps: Sequence[np.ndarray]) -> torch.Tensor:
        """Logits [n, vocab] of a pure decode step (one token per entry)."""
        n = int(tokens.shape[0])
        bucket = context_bucket(int(positions.max()) + 1)
        key = (n, bucket)
        slot = self.slots.get(key)
        if slot is None:
            while self.slots and (len(self.slots) >= self.MAX_SHAPES or
                                  sum(s.n for s in self.slots.values()) + n > self.MAX_KEPT_ROWS):
                self.slots.popitem(last=False)
            slot = self.slots[key] = _DecodeSlot(n, bucket, len(self.cache.groups), self.device, self.feedback)
        else:
            self.slots.move_to_end(key)
        slot.fill(tokens, positions, seats, slot_maps)
        if not slot.warm:
            # first step of this shape runs eagerly: it warms up lazy initialisation (GEMM
            # workspaces, kernel loading) that must not happen during capture
            slot.warm = True
            return self.model.forward(slot.batch, self.cache)
        if slot.graph is None:
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            # No garbage collection while the stream captures: an unreachable engine of earlier
            # (its pinned tables, events, graphs) freed in the middle of a capture makes calls that
            # a capturing stream forbids, and the failure is raised inside a destructor, where it
            # ends the process.  The collector stays off until the capture ends; what is garbage
            # now is collected at some later allocation, outside a capture.  (A full collection
            # here, before every capture, was 28 ms each: a third of a serving loop's host time
            # while new step shapes kept coming.)
            gc_was_on = gc.isenabled()
            gc.disable()
            try:
                with torch.cuda.graph(g):
                    slot.logits = self.model.forward(slot.batch, self.cache)
            finally:
                if gc_was_on:
                    gc.enable()
            slot.graph = g
            self.captures += 1
        slot.graph.replay()
        self.replays += 1
        return slot.logits


class _PortionSlot:
    """Static buffers, batch view and (once captured) the graph of one step shape that holds
    prompt portions: ``lens`` tokens per entry, logits wanted at ``rows``."""

    def __init__(self, lens: Tuple[int, ...], rows: Tuple[int, ...], bucket: int, variants: Sequence[tuple],
                 num_groups: int, device, feedback=None):
        self.lens = np.asarray(lens, dtype=np.int64)
        E, T, R = len(lens), int(sum(lens)), len(rows)
        self.T, self.E = T, E
        self.q_start = np.zeros(E + 1, dtype=np.int32)
        np.cumsum(lens, out=self.q_start[1:])
        # the int32 staging buffer: token_ids, positions, tok_seat [T each], entry_seat,
        # entry_start_pos [E each], one slot mapping [T] per cache group, then for every set of
        # attention items the forward pass asks for: entry [n], row0 [n], meta [n, 8]
        self.at: Dict[str, Tuple[int, int]] = {}
        total = 0
        for name, n in [("token_ids", T), ("positions", T), ("tok_seat", T), ("entry_seat", E),
                        ("entry_start_pos", E)] + [(f"slots{g}", T) for g in range(num_groups)]:
            self.at[name] = (total, n)
            total += (n + 3) // 4 * 4
        self.variants = list(variants)
        zeros = np.zeros(E, dtype=np.int32)
        self.items_at = []
        for group, tiles, which in self.variants:
            n = attention_work_items(self.q_start, zeros, zeros, group, tiles, which)[0].shape[0]
            self.items_at.append((total, n))
            total += (10 * n + 3) // 4 * 4
        self.staging = torch.zeros(max(1, total), dtype=torch.int32, pin_memory=True)
        self.dev = torch.zeros(max(1, total), dtype=torch.int32, device=device)
        self.const = torch.cat([torch.from_numpy(self.q_start),
                                torch.tensor(rows, dtype=torch.int32)]).to(device)
        v = lambda name: self.dev[self.at[name][0]:self.at[name][0] + self.at[name][1]]
        self.batch = StepBatch(
            num_tokens=T, num_entries=E, num_logit_rows=R,
            token_ids=v("token_ids"), positions=v("positions"), tok_seat=v("tok_seat"),
            logit_rows=self.const[E + 1:], slot_mapping=[v(f"slots{g}") for g in range(num_groups)],
            entry_seat=v("entry_seat"), entry_q_start=self.const[:E + 1], entry_start_pos=v("entry_start_pos"),
            max_q_len=int(max(lens)), min_q_len=int(min(lens)), max_context=bucket,
            logits_for_all_rows=tuple(rows) == tuple(range(T)), feedback=feedback, static_items=True)
        self.batch.h_entry_q_start = self.q_start
        for (group, tiles, which), (o, n) in zip(self.variants, self.items_at):
            self.batch._items[(group, tiles, which)] = (self.dev[o:o + n], self.dev[o + n:o + 2 * n],
                                                        self.dev[o + 2 * n:o + 10 * n].view(n, 8))
        self.copied = torch.cuda.Event()
        self.graph: Optional[torch.cuda.CUDAGraph] = None
        self.logits: Optional[torch.Tensor] = None

    def fill(self, tokens: np.ndarray, seats: np.ndarray, starts: np.ndarray,
             slot_maps: Sequence[np.ndarray]) -> None:
        self.copied.synchronize()        # the previous upload has left the staging buffer
        st = self.staging.numpy()

        def put(name, arr):
            o, n = self.at[name]
            st[o:o + n] = arr
        put("token_ids", tokens)
        put("positions", np.repeat(starts - self.q_start[:-1], self.lens) + np.arange(self.T, dtype=np.int32))
        put("tok_seat", np.repeat(seats, self.lens))
        put("entry_seat", seats)
        put("entry_start_pos", starts)
        for g, sm in enumerate(slot_maps):
            put(f"slots{g}", sm)
        for (group, tiles, which), (o, n) in zip(self.variants, self.items_at):
            ent, row0, meta = attention_work_items(self.q_start, starts, seats, group, tiles, which)
            st[o:o + n], st[o + n:o + 2 * n] = ent, row0
            st[o + 2 * n:o + 10 * n] = meta.reshape(-1)
        self.batch.h_entry_start_pos, self.batch.h_entry_seat = starts, seats
        self.dev.copy_(self.staging, non_blocking=True)
        self.copied.record()


class PortionGraphs:
    """Graphs for steps that hold prompt portions (alone or beside decoded tokens).

    A shape is (tokens per entry, wanted places, context bucket, whether the portions' rows visit
    enough keys for the workgroup attention kernel): everything the forward pass decides on the
    host.  Its first step runs eagerly and tells which sets of attention work items the pass asks
    for; the step at which it has come ``CAPTURE_AT`` times is captured over static buffers; later
    ones upload their indices and replay.  Logits come back in the shape's static buffer: they hold
    until its next step."""

    MAX_TOKENS = 4096          # tokens of one captured step
    MAX_LOGIT_ROWS = 64        # a graph keeps its logits: [rows, vocabulary] fp32
    MAX_SHAPES = 32            # captured shapes kept (least recently used goes first) ...
    MAX_KEPT_TOKENS = 16384    # ... and the tokens of all of them: a graph keeps its step's activations
    MAX_SEEN = 4096
    # A capture costs some 6 ms of host time and a place among the shapes kept.  Under a load of random
    # prompt lengths most shapes come twice at most: captured at their second step, 500 captures in
    # 17 s pushed each other out of the 32 places before any was replayed much.  The shapes that
    # carry such a load (so many decoded tokens beside a full portion) come again and again.
    CAPTURE_AT = 3

    def __init__(self, model, cache, device, feedback=None):
        self.model, self.cache, self.device, self.feedback = model, cache, device, feedback
        self.seen: Dict[tuple, tuple] = {}
        self.times: Dict[tuple, int] = {}            # steps a seen shape has come (while it has no graph)
        self.slots: "OrderedDict[tuple, _PortionSlot]" = OrderedDict()
        self.replays = 0
        self.captures = 0

    @staticmethod
    def shape_key(lens: Sequence[int], starts: Sequence[int], rows: Sequence[int]) -> Optional[tuple]:
        from ..ops.attention import LDS_MEAN_KEYS_STEPS
        T = int(sum(lens))
        if T > PortionGraphs.MAX_TOKENS or len(rows) > PortionGraphs.MAX_LOGIT_ROWS:
            return None
        ln, st = np.asarray(lens, dtype=np.float64), np.asarray(starts, dtype=np.float64)
        long = ln > 1
        mean_keys = float(((st[long] + (ln[long] + 1) / 2) * ln[long]).sum() / ln[long].sum())
        bucket = context_bucket(int(max(s + n for s, n in zip(starts, lens))))
        return (tuple(int(n) for n in lens), tuple(int(r) for r in rows), bucket,
                tuple(mean_keys >= t for t in LDS_MEAN_KEYS_STEPS))

    def note(self, key: tuple, batch: StepBatch) -> None:
        """After the eager run of a shape: the sets of attention items its forward pass used."""
        if key not in self.seen:
            if len(self.seen) >= self.MAX_SEEN:
                self.seen.clear()
                self.times.clear()
            self.seen[key] = tuple(batch._items.keys())
            self.times[key] = 1

    def run(self, key: tuple, tokens: np.ndarray, seats: np.ndarray, starts: np.ndarray,
            slot_maps: Sequence[np.ndarray]) -> Optional[torch.Tensor]:
        """Logits ``[wanted places, vocab]`` of the step, or ``None`` when the shape is new (the
        caller runs it eagerly and calls :meth:`note`)."""
        variants = self.seen.get(key)
        if variants is None:
            return None
        slot = self.slots.get(key)
        if slot is None:
            self.times[key] = self.times.get(key, 1) + 1
            if self.times[key] < self.CAPTURE_AT:
                return None
            lens, rows, bucket, _ = key
            while self.slots and (len(self.slots) >= self.MAX_SHAPES or
                                  sum(s.T for s in self.slots.values()) + sum(lens) > self.MAX_KEPT_TOKENS):
                self.slots.popitem(last=False)
            slot = self.slots[key] = _PortionSlot(lens, rows, bucket, variants, len(self.cache.groups),
                                                  self.device, self.feedback)
        else:
            self.slots.move_to_end(key)
        slot.fill(tokens, seats, starts, slot_maps)
        if slot.graph is None:
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            gc_was_on = gc.isenabled()        # as for decode graphs: nothing is collected while the stream captures
            gc.disable()
            try:
                with torch.cuda.graph(g):
                    slot.logits = self.model.forward(slot.batch, self.cache)
            finally:
                if gc_was_on:
                    gc.enable()
            slot.graph = g
            self.captures += 1
        slot.graph.replay()
        self.replays += 1
        return slot.logits
