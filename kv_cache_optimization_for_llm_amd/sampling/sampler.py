"""Greedy and temperature sampling over a step's logits, on the device.

Options and their meaning follow the reference (``base/src/main.cu:57-84``,
``base/src/kernels.cu:489-835``, ``python/sampling_reference.py``):

* ``temperature`` <= 0: greedy, the maximum logit, ties to the lowest token id;
* ``temperature`` > 0: inverse-CDF sampling of ``softmax(logits / temperature)`` with the
  counter-based uniform ``counter_uniform(seed, key, step)``; ``key = request_id * 8 +
  seq_index`` as in the reference, ``step`` = the absolute position the sampled token will take,
  so a draw is a pure function of (seed, request, position) - the intent the reference states at
  ``base/src/kernels.cuh:158-160`` - and a recomputed request draws the same tokens again;
* ``repetition_penalty`` (reference: fixed 1.15, ``base/src/config.h:83``): logits of tokens the
  request has already emitted are divided (if positive) or multiplied (if negative) by it, from
  the second generated token on.  The emitted-token mask lives in the request's seat, one byte
  per vocabulary entry.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Sequence

import numpy as np
import torch

from ..ops import kernels as K


def counter_uniform(seed: int, key: int, step: int) -> float:
    """Host mirror of the device function (splitmix64 finaliser, top 24 bits)."""
    M = (1 << 64) - 1
    z = (((key & 0xFFFFFFFF) << 32) ^ (step & 0xFFFFFFFF)) & M
    z ^= ((seed & 0xFFFFFFFF) * 0x9E3779B97F4A7C15) & M
    z = (z + 0x9E3779B97F4A7C15) & M
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M
    z ^= z >> 31
    return (z >> 40) * (1.0 / 16777216.0)


@dataclass
class SampleRow:
    seat: int
    temperature: float = 0.0
    rng_key: int = 0
    rng_step: int = 0
    apply_penalty: bool = False


def _as_i32(values: Sequence[int]) -> np.ndarray:
    return (np.asarray(values, dtype=np.int64) & 0xFFFFFFFF).astype(np.uint32).view(np.int32)


class PendingTokens:
    """Sampled tokens on their way to the host: the kernel that chooses them writes them into
    pinned memory as well, and :meth:`wait` blocks until the stream has passed it."""

    def __init__(self, host: torch.Tensor, event: "torch.cuda.Event", n: int):
        self._host, self._event, self._n = host, event, n
        self._value: Optional[np.ndarray] = None

    def wait(self) -> np.ndarray:
        if self._value is None:
            self._event.synchronize()
            self._value = self._host.numpy()[:self._n].copy()
        return self._value


class Sampler:
    # the kernel that chooses the tokens writes them to the pinned host buffer itself (no copy
    # kernel behind it on the stream)
    KERNEL_WRITES_HOST = True

    def __init__(self, vocab_size: int, max_seqs: int, device, *, seed: int = 0,
                 repetition_penalty: float = 1.0, chunks: int = 128):
        if repetition_penalty <= 0:
            raise ValueError("repetition_penalty must be positive")
        self.vocab_size, self.device, self.seed = vocab_size, device, int(seed)
        self.penalty = float(repetition_penalty)
        self.chunks = max(1, min(chunks, (vocab_size + 255) // 256))
        self.mask: Optional[torch.Tensor] = None
        if self.penalty != 1.0:
            self.mask = torch.zeros((max_seqs, vocab_size), dtype=torch.uint8, device=device)
        # pinned landing buffers for sample_async, used in turn (two samplings may be in flight)
        self._landing: List[torch.Tensor] = []
        self._kernel_writes_host = False
        self._landing_next = 0
        # per-row arguments of a sampling (temperatures, random-stream keys and steps, seats)
        self._args_dev: Optional[torch.Tensor] = None
        self._args_host: List[tuple] = []
        self._args_next = 0

    def _row_arguments(self, n: int):
        """A pinned staging array [5, capacity] int32 to fill (float rows as their bits) and the
        device array it is copied to by :meth:`_send_row_arguments`."""
        if self._args_dev is None or self._args_dev.shape[1] < n:
            cap = max(64, n)
            self._args_dev = torch.zeros((5, cap), dtype=torch.int32, device=self.device)
            self._args_host = [(torch.zeros((5, cap), dtype=torch.int32, pin_memory=True), torch.cuda.Event())
                               for _ in range(3)]
        self._args_next = (self._args_next + 1) % len(self._args_host)
        staging, copied = self._args_host[self._args_next]
        copied.synchronize()             # its last copy has left it (three steps ago)
        return staging.numpy(), self._args_dev

    def _send_row_arguments(self) -> None:
        staging, copied = self._args_host[self._args_next]
        self._args_dev.copy_(staging, non_blocking=True)
        copied.record()

    def reset_seat(self, seat: int, emitted: Sequence[int] = ()) -> None:
        """A request takes the seat: clear its mask and mark what it has emitted before (a
        recomputed request arrives with its earlier output)."""
        if self.mask is None:
            return
        self.mask[seat].zero_()
        if len(emitted):
            self.mark([seat] * len(emitted), emitted)

    def mark(self, seats: Sequence[int], tokens: Sequence[int]) -> None:
        if self.mask is None or not len(seats):
            return
        s = torch.from_numpy(np.asarray(seats, dtype=np.int32)).to(self.device)
        t = torch.from_numpy(np.asarray(tokens, dtype=np.int32)).to(self.device)
        K.mark_tokens(self.mask, s, t)

    def sample(self, logits: torch.Tensor, rows: Sequence[SampleRow]) -> np.ndarray:
        """One token per logits row; returns host int32."""
        return self.sample_async(logits, rows).wait()

    def sample_async(self, logits: torch.Tensor, rows: Sequence[SampleRow],
                     out: Optional[torch.Tensor] = None) -> PendingTokens:
        """Queues the sampling of one token per logits row (the tokens land in pinned host memory
        too), without waiting for it.  ``out`` (device int32, at least ``len(rows)`` long) takes the tokens,
        row by row, and may be read by later work on the same stream."""
        n = len(rows)
        if logits.shape != (n, self.vocab_size):
            raise ValueError(f"logits {tuple(logits.shape)} do not fit {n} rows of {self.vocab_size}")
        if out is None:
            out = torch.empty(max(n, 1), dtype=torch.int32, device=self.device)
        if out.dtype != torch.int32 or out.dim() != 1 or out.shape[0] < n:
            raise ValueError("sample: out must be a device int32 vector with a place per row")
        out = out[:n]
        if len(self._landing) < 3 or self._landing[0].shape[0] < n:
            size = max(64, n)
            self._landing = [torch.zeros(size, dtype=torch.int32, pin_memory=True) for _ in range(3)]
            # where the runtime does not map pinned memory for the device, a copy follows the kernels instead
            self._kernel_writes_host = self.KERNEL_WRITES_HOST and all(K.host_memory_is_mapped(t) for t in self._landing)
        host = self._landing[self._landing_next]
        self._landing_next = (self._landing_next + 1) % len(self._landing)
        event = torch.cuda.Event()
        if n == 0:
            event.record()
            return PendingTokens(host, event, 0)
        any_sampled = any(r.temperature > 0 for r in rows)
        use_mask = self.mask is not None and any(r.apply_penalty for r in rows)
        inv_t = key = step = seat_t = mark_seat = None
        if any_sampled or self.mask is not None:
            # the per-row arguments go up in one copy from pinned memory (five small pageable
            # tensors, each copied by itself, were 0.4 ms of host time apiece in a serving loop)
            host_args, dev_args = self._row_arguments(n)
            if any_sampled:
                host_args[0, :n] = np.asarray([1.0 / r.temperature if r.temperature > 0 else 0.0 for r in rows],
                                              dtype=np.float32).view(np.int32)
                host_args[1, :n] = _as_i32([r.rng_key for r in rows])
                host_args[2, :n] = _as_i32([r.rng_step for r in rows])
                inv_t, key, step = dev_args[0, :n].view(torch.float32), dev_args[1, :n], dev_args[2, :n]
            if use_mask:
                host_args[3, :n] = [r.seat if r.apply_penalty else -1 for r in rows]
                seat_t = dev_args[3, :n]
            if self.mask is not None:
                # every token a request emits is marked in its mask row, by the launch that chooses it
                host_args[4, :n] = [r.seat for r in rows]
                mark_seat = dev_args[4, :n]
            self._send_row_arguments()
        K.sample(logits, out, chunks=self.chunks, inv_temperature=inv_t, seed=self.seed, rng_key=key,
                 rng_step=step, penalty_mask=self.mask if use_mask else None, row_seat=seat_t,
                 penalty=self.penalty, mark_mask=self.mask if mark_seat is not None else None,
                 mark_seat=mark_seat, host_tokens=host if self._kernel_writes_host else None)
        if not self._kernel_writes_host:
            host[:n].copy_(out, non_blocking=True)
        event.record()
        return PendingTokens(host, event, n)
