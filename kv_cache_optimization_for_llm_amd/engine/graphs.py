"""HIP graphs for decode steps.

A decode step of a small model is a few hundred short kernels; launched one by one the host
cannot keep the GPU busy.  For batches in which every entry brings exactly one token, the whole
forward pass is captured once per (number of entries, context bucket) into a HIP graph over
static index buffers; later steps of that shape copy their indices into the buffers (one small
host-to-device copy) and replay the graph.

What is inside a graph: the model's kernels and the vendor GEMM calls.  What stays outside: the
upload of indices and block-table spans, sampling, and every allocation.  Nothing inside clears
memory with a memset node.
"""
from __future__ import annotations

import gc

from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from .batch import StepBatch


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
    def __init__(self, model, cache, device, feedback=None):
        self.model, self.cache, self.device, self.feedback = model, cache, device, feedback
        self.slots: Dict[Tuple[int, int], _DecodeSlot] = {}
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
            slot = self.slots[key] = _DecodeSlot(n, bucket, len(self.cache.groups), self.device, self.feedback)
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
            # ends the process.  Collect first, then keep the collector off until the capture ends.
            gc.collect()
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
