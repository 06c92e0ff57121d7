"""The engine: a model folder, a cache and ONE step function.

``Engine.step(entries)`` takes a batch of (request, its next tokens, wanted places) - portions
of prompts of any length beside single decoded tokens - runs exactly those tokens through the
model against the cache that earlier steps left, and returns the logits at the wanted places.
The reference has two separate passes for this (``prefillBatch`` ``base/src/engine.cu:550-979``,
which cannot continue a partly cached prompt, and ``decodeStep`` ``:982-1311``).
"""
from __future__ import annotations

import os
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import CacheManager
from ..cache.manager import page_bytes as cache_page_bytes
from ..config.model_config import read_config_json
from ..models.builder import Model, spec_for_config
from ..ops.library import KernelLibraryError, hip_lib
from ..weights.loader import load_tensors
from ..weights.random_init import random_tensors_on_device
from .batch import StepBatch, StepEntry, build_batch

_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32,
           "bf16": torch.bfloat16, "fp32": torch.float32}


class CacheExhausted(RuntimeError):
    """A step needs more pages (or a longer reservation) than the cache can give."""


class EngineError(RuntimeError):
    pass


@dataclass
class EngineOptions:
    dtype: str = "bfloat16"             # "bfloat16": serving kernels; "float32": true 32-bit everywhere
    cache_mode: str = "paged"           # "paged" | "contiguous"
    page_size: int = 16                 # tokens per page (reference: BLOCK_SIZE, paged config.h:181)
    # Pool size in tokens.  None: what is free on the device after weights, tables and the GEMM
    # workspace, less ``memory_margin_bytes`` and a step's activations, but never more than every
    # seat at its longest (reference: the pool is sized last, from leftover memory,
    # base/src/engine.cu:257-299, paged_attention/src/engine.cu:186-215).
    cache_tokens: Optional[int] = None
    memory_margin_bytes: int = 2 << 30  # left free when the pool is sized from leftover memory
    max_seqs: int = 8                   # seats (reference: MAX_SEQUENCES)
    max_seq_len: Optional[int] = None   # longest request (default: max_position_embeddings)
    max_batch_tokens: int = 8192        # most tokens one step may bring (reference: MAX_BATCH_TOKENS)
    max_logit_rows: Optional[int] = None  # most places a step may want logits at (default: max_batch_tokens;
                                          # a server that samples one token per request needs max_seqs)
    use_graphs: bool = True             # replay decode-only steps, and steps with prompt portions whose
                                        # shape comes back, as HIP graphs (bfloat16 engine)
    # Row counts (tokens per step) for which the vendor GEMM library's algorithms are timed at
    # start-up and the fastest kept, e.g. the prompt portion size and large decode batches
    # (bfloat16 engine; a few seconds per row count and matrix shape; row counts down to half of a
    # timed one share what was found for it).  Empty: the library's own choice.
    gemm_tune_rows: Sequence[int] = ()
    device: str = "cuda:0"


def pool_pages_from_memory(free_bytes: int, page_bytes: int, *, page_size: int, max_seqs: int,
                           max_seq_len: int, margin_bytes: int, step_bytes: int = 0) -> int:
    """Pages of a cache pool that is sized from leftover device memory: ``free_bytes`` less a
    margin and a step's activations, in whole pages of ``page_bytes`` (all cache slots of all
    groups together), but no more than every seat needs at its longest.  The reference sizes
    its pool this way after everything else is allocated
    (``paged_attention/src/engine.cu:186-215``: free memory - 128 MiB, in pages)."""
    if page_bytes <= 0 or page_size <= 0:
        raise EngineError("page_bytes and page_size must be positive")
    most = max_seqs * ((max_seq_len + page_size - 1) // page_size)
    room = (int(free_bytes) - int(margin_bytes) - int(step_bytes)) // page_bytes
    if room < 1:
        raise EngineError(
            f"no room for a cache pool: {free_bytes / 2**30:.2f} GiB free, {margin_bytes / 2**30:.2f} GiB "
            f"margin, {step_bytes / 2**30:.2f} GiB for a step's activations, {page_bytes} bytes a page")
    return int(min(most, room))


def require_gpu(device: str = "cuda:0") -> torch.device:
    if not torch.cuda.is_available():
        raise KernelLibraryError(
            "no GPU is visible to torch; this engine runs on the GPU only (hand-written HIP "
            "kernels for gfx950) and has no CPU path")
    hip_lib()
    return torch.device(device)


class Engine:
    """``Engine(model_dir)`` loads a model folder.  ``Engine(None, config_dict=..., random_seed=...)``
    builds the same model with random weights made on the device (for measurements; the values
    differ from the folder the random-weights mode writes for the same seed)."""

    def __init__(self, model_dir: Optional[str], options: Optional[EngineOptions] = None, *,
                 config_dict: Optional[dict] = None, random_seed: Optional[int] = None):
        self.options = options = options or EngineOptions()
        if options.dtype not in _DTYPES:
            raise EngineError(f"dtype {options.dtype!r} is not one of bfloat16, float32")
        self.dtype = _DTYPES[options.dtype]
        self.device = require_gpu(options.device)
        if self.dtype == torch.float32:
            # the 32-bit path never uses a reduced-precision matrix mode
            torch.backends.cuda.matmul.allow_tf32 = False
            torch.backends.cudnn.allow_tf32 = False
        self.model_dir = model_dir
        if model_dir is None and (config_dict is None or random_seed is None):
            raise EngineError("without a model folder, config_dict and random_seed are needed")
        self.config_dict = read_config_json(model_dir) if model_dir is not None else dict(config_dict)
        self.config, self.spec = spec_for_config(self.config_dict)
        self.model = Model(self.spec, self.dtype, self.device)
        if model_dir is not None:
            tensors = load_tensors(model_dir, self.model.tensor_specs(), self.dtype, self.device,
                                   self.spec.ignorable_tensors)
        else:
            tensors = random_tensors_on_device(self.model.tensor_specs(), random_seed, self.dtype,
                                               self.device)
        self.model.load(tensors)
        del tensors
        self.gemm_tuning: List[dict] = []
        if options.gemm_tune_rows and self.dtype == torch.bfloat16:
            import sys
            self.gemm_tuning = self.model.tune_products(
                options.gemm_tune_rows, say=lambda line: print(f"[kva tune] {line}", file=sys.stderr, flush=True))
        self.vocab_size = self.spec.vocab_size
        max_seq_len = options.max_seq_len or self.spec.max_positions
        max_seq_len = min(max_seq_len, self.spec.max_positions)
        self.model.limit_positions(max_seq_len)     # per-position tables no longer than the longest request
        if options.max_batch_tokens < 1:
            raise EngineError("max_batch_tokens must be at least 1")
        self.max_batch_tokens = int(options.max_batch_tokens)
        self.max_logit_rows = int(options.max_logit_rows or options.max_batch_tokens)
        if self.max_logit_rows < 1:
            raise EngineError("max_logit_rows must be at least 1")
        groups, states = self.model.cache_requirements()
        if options.cache_tokens:
            num_pages = (options.cache_tokens + options.page_size - 1) // options.page_size
        else:
            page_bytes = cache_page_bytes(groups, options.page_size, self.dtype)    # as the mixers' specs say
            if page_bytes == 0:
                num_pages = 1           # no mixer keeps keys and values
            else:
                torch.cuda.empty_cache()        # what loading left cached is free for the pool as well
                free_bytes, _ = torch.cuda.mem_get_info(self.device)
                tables = sum(4 * options.max_seqs * ((max_seq_len + options.page_size - 1) // options.page_size)
                             for _ in groups)
                num_pages = pool_pages_from_memory(
                    free_bytes - tables, page_bytes, page_size=options.page_size, max_seqs=options.max_seqs,
                    max_seq_len=max_seq_len, margin_bytes=options.memory_margin_bytes,
                    step_bytes=self.model.step_activation_bytes(self.max_batch_tokens, self.max_logit_rows))
        self.cache = CacheManager(groups, states, page_size=options.page_size, num_pages=num_pages,
                                  max_seqs=options.max_seqs, max_seq_len=max_seq_len,
                                  mode=options.cache_mode, device=self.device, dtype=self.dtype)
        self.max_seq_len = max_seq_len
        # The step's arena (reference: one block of scratch for MAX_BATCH_TOKENS rows,
        # base/src/engine.cu:62-122): what the largest step needs for its intermediate results is
        # taken from the device once, here, and handed to torch's caching allocator, which cuts
        # every later step's tensors out of this block instead of asking the device again.
        self.step_arena_bytes = self.model.step_activation_bytes(self.max_batch_tokens, self.max_logit_rows)
        arena = torch.empty(self.step_arena_bytes, dtype=torch.uint8, device=self.device)
        del arena
        self._seat_of: Dict[object, int] = {}
        self.steps_run = 0
        # tokens that stay on the device between steps: a sampler leaves its output here and the
        # next step's single-token entries may name a row of it instead of a token id
        self.feedback = torch.zeros(max(1, options.max_seqs), dtype=torch.int32, device=self.device)
        self.graphs = None
        self.portion_graphs = None
        if options.use_graphs and self.dtype == torch.bfloat16 and self.model.graph_safe():
            from .graphs import DecodeGraphs, PortionGraphs
            self.graphs = DecodeGraphs(self.model, self.cache, self.device, self.feedback)
            self.portion_graphs = PortionGraphs(self.model, self.cache, self.device, self.feedback)

    # ------------------------------------------------------------------ requests
    def has_request(self, request_id) -> bool:
        return request_id in self._seat_of

    def seat_of(self, request_id) -> int:
        return self._seat_of[request_id]

    def add_request(self, request_id, reserve_tokens: Optional[int] = None) -> Optional[int]:
        """Gives the request a seat (and, in contiguous mode, its reservation).  ``None`` when
        there is no seat or no room for the reservation."""
        if request_id in self._seat_of:
            raise EngineError(f"request {request_id!r} is live already")
        if self.cache.mode == "contiguous" and reserve_tokens is None:
            reserve_tokens = self.max_seq_len       # the reference's 'max' policy
        seat = self.cache.admit(request_id, reserve_tokens)
        if seat is not None:
            self._seat_of[request_id] = seat
        return seat

    def bind_request(self, request_id, seat: int) -> None:
        """For a scheduler that takes seats from the cache manager itself: names the request that
        sits in ``seat``, so that its entries are recognised by :meth:`step_planned`."""
        if request_id in self._seat_of:
            raise EngineError(f"request {request_id!r} is live already")
        self.cache.seat(seat)               # raises unless the seat is taken
        self._seat_of[request_id] = seat

    def unbind_request(self, request_id) -> None:
        """The scheduler has given the request's seat back itself."""
        self._seat_of.pop(request_id, None)

    def release(self, request_id) -> None:
        """The request is finished: its pages, reservation and seat are given back."""
        seat = self._seat_of.pop(request_id)
        self.cache.free(seat)

    def length(self, request_id) -> int:
        return self.cache.length(self._seat_of[request_id])

    # ------------------------------------------------------------------ the step
    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """Runs one batch; returns fp32 logits ``[wanted places, vocab]`` on the device, in the
        order of the entries and of each entry's ``want``.  A step replayed from a graph returns
        the graph's own buffer: it holds until the next step of the same shape, so copy what has
        to outlive that."""
        logits = self._run(entries)
        self.finish(entries)
        return logits

    def step_planned(self, entries: Sequence[StepEntry], seats: Sequence[int],
                     starts: Sequence[int]) -> torch.Tensor:
        """The step for a scheduler that owns the seats itself: entry ``i`` belongs to
        ``seats[i]`` and starts at position ``starts[i]``; lengths are committed by the caller."""
        for e, seat, start in zip(entries, seats, starts):
            if self._seat_of.get(e.request_id) != seat or self.cache.length(seat) != start:
                raise EngineError(f"plan does not fit the cache: request {e.request_id!r}")
        logits = self._run(entries)
        self.steps_run += 1
        return logits

    def _run(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        seats, starts, toks, wants = self._place(entries)
        groups = self.cache.groups
        if all(len(t) == 1 for t in toks):
            # a decode step: one position per entry, everything in whole arrays
            seats_a, starts_a = np.asarray(seats, dtype=np.int32), np.asarray(starts, dtype=np.int32)
            slots = [self.cache.slot_mapping_each(seats_a, starts_a, g.index) for g in groups]
            self.cache.flush_tables()
            if self.graphs is not None:
                logits = self.graphs.run(np.asarray([t[0] for t in toks], dtype=np.int32), starts_a, seats_a, slots)
                rows = [e for e, w in enumerate(wants) for _ in w]
                if rows != list(range(len(entries))):
                    logits = logits[torch.tensor(rows, dtype=torch.long, device=self.device)] if rows \
                        else logits[:0]
                return logits
            slot_maps = [[m[i:i + 1] for i in range(len(seats))] for m in slots]
        else:
            slot_maps = [[self.cache.slot_mapping(seat, start, len(arr), g.index)
                          for seat, start, arr in zip(seats, starts, toks)] for g in groups]
            self.cache.flush_tables()
            if self.portion_graphs is not None:
                # a step shape that has been seen before runs from its graph
                lens = [len(t) for t in toks]
                first = np.cumsum([0] + lens[:-1])
                key = self.portion_graphs.shape_key(lens, starts, [int(f) + int(i) for f, w in zip(first, wants) for i in w])
                if key is not None:
                    logits = self.portion_graphs.run(
                        key, np.concatenate([np.asarray(t, dtype=np.int32) for t in toks]),
                        np.asarray(seats, dtype=np.int32), np.asarray(starts, dtype=np.int32),
                        [np.concatenate(m).astype(np.int32) for m in slot_maps])
                    if logits is not None:
                        return logits
                    batch = build_batch(seats, starts, toks, wants, slot_maps, self.device)
                    batch.feedback = self.feedback
                    logits = self.model.forward(batch, self.cache)
                    self.portion_graphs.note(key, batch)
                    return logits
        batch = build_batch(seats, starts, toks, wants, slot_maps, self.device)
        batch.feedback = self.feedback
        return self.model.forward(batch, self.cache)

    def _place(self, entries: Sequence[StepEntry]):
        """Seats, start positions and pages for every entry of the step."""
        if not entries:
            raise EngineError("a step needs at least one entry")
        seen = set()
        seats, starts, toks, wants = [], [], [], []
        vocab, lowest_single = self.vocab_size, -self.feedback.shape[0]
        for e in entries:       # refuse a bad step before anything is admitted or mapped
            if e.request_id in seen:
                raise EngineError(f"request {e.request_id!r} appears twice in one step")
            seen.add(e.request_id)
            n = len(e.tokens)
            if n == 0:
                raise EngineError(f"request {e.request_id!r}: an entry needs at least one token")
            if n == 1:
                arr = e.tokens if isinstance(e.tokens, list) else list(e.tokens)
                lo = hi = int(arr[0])
                lowest = lowest_single           # a lone token may be a feedback row
            else:
                arr = np.asarray(e.tokens, dtype=np.int64)
                lo, hi, lowest = int(arr.min()), int(arr.max()), 0
            if lo < lowest or hi >= vocab:
                raise EngineError(f"request {e.request_id!r}: token id outside [0, {vocab})")
            for i in e.want:
                if not 0 <= i < n:
                    raise EngineError(f"request {e.request_id!r}: wanted place {i} is outside its "
                                      f"{n} tokens")
            toks.append(arr)
            wants.append(e.want if isinstance(e.want, list) else list(e.want))
        total = sum(len(t) for t in toks)
        if total > self.max_batch_tokens:
            raise EngineError(f"a step of {total} tokens is larger than max_batch_tokens "
                              f"({self.max_batch_tokens}); cut the prompts into smaller portions")
        wanted = sum(len(w) for w in wants)
        if wanted > self.max_logit_rows:
            raise EngineError(f"a step that wants logits at {wanted} places is larger than max_logit_rows "
                              f"({self.max_logit_rows})")
        seat_of, cache = self._seat_of, self.cache
        for e in entries:
            seat = seat_of.get(e.request_id)
            if seat is None:
                if self.add_request(e.request_id) is None:
                    raise CacheExhausted(f"no seat (or reservation) for request {e.request_id!r}")
                seat = seat_of[e.request_id]
            seats.append(seat)
            starts.append(cache.length(seat))
        # map the pages the step writes to
        for e, seat, start, arr in zip(entries, seats, starts, toks):
            if not cache.grow(seat, start + len(arr)):
                need = cache.pages_needed(seat, start + len(arr))
                raise CacheExhausted(
                    f"request {e.request_id!r} needs {need} more pages for positions "
                    f"{start}..{start + len(arr) - 1} (capacity {cache.capacity_tokens(seat)} "
                    f"tokens, free pages {[g.free_pages() for g in cache.groups]})")
        return seats, starts, toks, wants

    def finish(self, entries: Sequence[StepEntry]) -> None:
        for e in entries:
            seat = self._seat_of[e.request_id]
            self.cache.commit(seat, self.cache.length(seat) + len(e.tokens))
        self.steps_run += 1
