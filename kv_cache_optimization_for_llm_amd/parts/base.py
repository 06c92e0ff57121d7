"""Interfaces of the parts a layer is put together from.

A part knows its own sizes and constants (given at construction), the tensors it reads from a
checkpoint and how to run on a batch.  It never knows which model it is in.

* :class:`Norm`             ``forward(x, out=None, delta=None, row_idx=None)``
* :class:`PositionEncoding` ``apply_and_cache(qkv, positions, geometry, kv)``
* :class:`Mixer`            ``forward(x, ctx)`` with a :class:`MixerContext`; declares the cache it
  needs (:class:`KVCacheSpec`: all keys or a window of them) and/or a fixed-size per-request
  state (:class:`StateSpec`)
* :class:`FeedForward`      ``forward(x, ctx)``
* :class:`Block`            ``forward(hidden, delta, ctx)`` -> ``(hidden, delta)``: the arrangement
  of norms, mixer, feed-forward and residual sums; ``delta`` is a branch output that has not
  been added to the residual stream yet, so the next norm can fuse the add
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional, Tuple

import torch

from ..models.spec import TensorSpec


@dataclass(frozen=True)
class KVCacheSpec:
    """Paged key/value storage one mixer call needs, per token: ``num_kv_heads * head_dim`` keys
    and as many values.  ``kind`` is ``"full"`` (every position stays) or ``"window"`` (only the
    last ``window`` positions are ever read, pages behind them are given back)."""

    num_kv_heads: int
    head_dim: int
    kind: str = "full"
    window: int = 0


@dataclass(frozen=True)
class StateSpec:
    """Fixed-size state one mixer call keeps per request (zeroed when a request takes a seat)."""

    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class KVView:
    """What a mixer call sees of the paged cache: its own K array
    ``[pages, kv_heads, page_size, head_dim]`` and V array (transposed inside a page)
    ``[pages, kv_heads, head_dim, page_size]``, the block table ``[seats, max_blocks]`` of its
    group, and for each token of the step the slot (page * page_size + row) to write to."""

    k_cache: torch.Tensor
    v_cache: torch.Tensor
    block_table: torch.Tensor
    slot_mapping: torch.Tensor
    page_size: int
    writes: bool = True


@dataclass
class MixerContext:
    batch: "object"                       # engine.batch.StepBatch
    kv: Optional[KVView] = None
    state: Optional[torch.Tensor] = None  # [seats, *StateSpec.shape] of this mixer call


class Part:
    """Common behaviour: named tensors relative to a prefix."""

    # True when forward() only launches kernels on the current stream over device tensors it is
    # given or allocates with torch (no host copies, no synchronisation, no data-dependent
    # shapes): such a part may be captured into a HIP graph.
    graph_safe = False

    def __init__(self, prefix: str = ""):
        self.prefix = prefix

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        """Full tensor name -> spec of every tensor this part reads."""
        return {}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        """Takes the tensors named by ``tensor_specs`` (already on the device)."""


class Norm(Part):
    def forward(self, x: torch.Tensor, out: Optional[torch.Tensor] = None,
                delta: Optional[torch.Tensor] = None,
                row_idx: Optional[torch.Tensor] = None) -> torch.Tensor:
        raise NotImplementedError


class PositionEncoding(Part):
    def apply_and_cache(self, qkv: torch.Tensor, positions: torch.Tensor, num_q_heads: int,
                        num_kv_heads: int, head_dim: int, kv: Optional[KVView]) -> None:
        """Encodes positions into the Q and K heads of ``qkv`` in place and, when ``kv`` allows
        writing, stores the encoded K and the plain V at the tokens' cache slots."""
        raise NotImplementedError


class Mixer(Part):
    def kv_cache_spec(self) -> Optional[KVCacheSpec]:
        return None

    def state_spec(self) -> Optional[StateSpec]:
        return None

    def forward(self, x: torch.Tensor, ctx: MixerContext) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, x: torch.Tensor, ctx: MixerContext) -> torch.Tensor:
        raise NotImplementedError


class Block(Part):
    def __init__(self, mixer: Mixer, feed_forward: FeedForward, mixer_norm: Norm, ffn_norm: Norm):
        super().__init__("")
        self.mixer, self.feed_forward = mixer, feed_forward
        self.mixer_norm, self.ffn_norm = mixer_norm, ffn_norm

    def parts(self):
        return (self.mixer_norm, self.mixer, self.ffn_norm, self.feed_forward)

    def forward(self, hidden: torch.Tensor, delta: Optional[torch.Tensor], ctx: MixerContext):
        raise NotImplementedError
