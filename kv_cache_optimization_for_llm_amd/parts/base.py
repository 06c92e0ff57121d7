"""Interfaces of the parts a layer is put together from.

A part knows its own sizes and constants (given at construction), the tensors it reads from a
checkpoint and how to run on a batch.  It never knows which model it is in.

* :class:`Norm`             ``forward(x, out=None, delta=None, row_idx=None)``
* :class:`PositionEncoding` ``apply_and_cache(qkv, positions, geometry, kv)``
* :class:`Mixer`            ``forward(x, ctx)`` with a :class:`MixerContext`; declares the cache it
  needs (:class:`KVCacheSpec`: named arrays per token, all positions or a window of them) and/or a fixed-size per-request
  state (:class:`StateSpec`)
* :class:`FeedForward`      ``forward(x, ctx)``
* :class:`Block`            ``forward(hidden, delta, ctx, next_norm=None)`` -> ``(hidden, delta)``:
  the arrangement of norms, mixer, feed-forward and residual sums; ``delta`` is a branch output
  that has not been added to the residual stream yet (the next norm fuses the add), or
  :class:`NormedRows` when the add is done and the next norm is already prepared

Fusing across parts.  A part that sets ``fuses_tail = True`` takes two optional extras in
``forward``: its input may be :class:`NormedRows` (an unfinished norm) and ``tail``
(:class:`BranchTail`) asks it to add its output to the residual stream and prepare the next
norm inside its last product.  Parts without the flag get plain tensors and return plain tensors;
the block does the rest with separate kernels.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional, Tuple

import torch

from ..models.spec import TensorSpec


@dataclass(frozen=True)
class CacheArray:
    """One array of a paged cache entry: what a mixer call keeps per token under ``name``.

    ``token_shape`` is the shape of one token's entry; ``token_axis`` says where the page's token
    axis lies inside a page: a page of the array has ``token_shape`` with ``page_size`` inserted at
    that index, and the whole array is ``[pages, *page_shape]``.  Keys of attention heads
    ``(kv_heads, head_dim)`` with ``token_axis=1`` give pages ``[kv_heads, page_size, head_dim]``;
    values with ``token_axis=2`` give the transposed ``[kv_heads, head_dim, page_size]``; one
    latent vector ``(width,)`` with ``token_axis=0`` gives ``[page_size, width]``.  ``dtype``
    ``None`` is the engine's storage type."""

    name: str
    token_shape: Tuple[int, ...]
    token_axis: int = 0
    dtype: Optional[torch.dtype] = None

    def __post_init__(self):
        if not self.token_shape or any(int(n) <= 0 for n in self.token_shape):
            raise ValueError(f"cache array {self.name!r}: token shape {self.token_shape} must be positive")
        if not 0 <= self.token_axis <= len(self.token_shape):
            raise ValueError(f"cache array {self.name!r}: token axis {self.token_axis} lies outside its page")

    def page_shape(self, page_size: int) -> Tuple[int, ...]:
        shape = list(self.token_shape)
        shape.insert(self.token_axis, int(page_size))
        return tuple(shape)

    def elements_per_token(self) -> int:
        n = 1
        for d in self.token_shape:
            n *= int(d)
        return n


@dataclass(frozen=True)
class KVCacheSpec:
    """Paged storage one mixer call needs: the arrays it keeps per token (names, per-token
    shapes, layout inside a page) and which positions stay.  ``kind`` is ``"full"`` (every
    position stays) or ``"window"`` (only the last ``window`` positions are ever read, pages
    behind them are given back).  The cache manager allocates from this description and the
    engine sizes the pool from it; neither knows what the arrays mean."""

    arrays: Tuple[CacheArray, ...]
    kind: str = "full"
    window: int = 0

    def __post_init__(self):
        names = [a.name for a in self.arrays]
        if not names or len(set(names)) != len(names):
            raise ValueError(f"a cache entry needs arrays with distinct names, got {names}")
        if self.kind not in ("full", "window"):
            raise ValueError(f"cache kind {self.kind!r} is not one of 'full', 'window'")

    def bytes_per_token(self, default_dtype: torch.dtype) -> int:
        return sum(a.elements_per_token() * torch.empty((), dtype=a.dtype or default_dtype).element_size()
                   for a in self.arrays)


def attention_cache_spec(num_kv_heads: int, head_dim: int, kind: str = "full", window: int = 0) -> KVCacheSpec:
    """Keys and values of ``num_kv_heads`` heads of ``head_dim``, as the attention kernels here
    read them: K pages ``[kv_heads, head_dim / C, page_size, C]`` (a key in chunks of C = 8
    elements, 4 where the head size is no multiple of 8; the chunks of a page's keys next to each
    other, so that a wavefront's matrix-core operand is one run of bytes), V pages transposed
    ``[kv_heads, head_dim, page_size]``."""
    chunk = 4 if head_dim % 8 else 8
    return KVCacheSpec((CacheArray("k", (int(num_kv_heads), int(head_dim) // chunk, chunk), token_axis=2),
                        CacheArray("v", (int(num_kv_heads), int(head_dim)), token_axis=2)), kind, window)


@dataclass(frozen=True)
class StateSpec:
    """Fixed-size state one mixer call keeps per request (zeroed when a request takes a seat)."""

    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class KVView:
    """What a mixer call sees of the paged cache: its own arrays by name (each
    ``[pages, *page_shape]`` as its :class:`CacheArray` says), the block table
    ``[seats, max_blocks]`` of its group, and for each token of the step the slot
    (page * page_size + row) to write to."""

    arrays: Dict[str, torch.Tensor]
    block_table: torch.Tensor
    slot_mapping: torch.Tensor
    page_size: int
    writes: bool = True

    @property
    def k_cache(self) -> torch.Tensor:      # the two arrays of attention_cache_spec
        return self.arrays["k"]

    @property
    def v_cache(self) -> torch.Tensor:
        return self.arrays["v"]


@dataclass
class MixerContext:
    batch: "object"                       # engine.batch.StepBatch
    kv: Optional[KVView] = None
    state: Optional[torch.Tensor] = None  # [seats, *StateSpec.shape] of this mixer call


@dataclass
class NormedRows:
    """Rows of the residual stream handed to a norm that has not been finished yet.

    A matrix product whose output goes into the residual stream can prepare the next norm in its
    epilogue: ``scaled = round(hidden * norm_weight)`` and, per row, partial sums of
    ``hidden^2`` (``sumsq [T, parts]``).  The normalised rows are
    ``scaled * rsqrt(sum(sumsq) / width + eps)``; a product that takes them as input applies the
    per-row factor to its result instead, so the norm costs no pass over memory.  ``norm`` is
    the norm object these rows were prepared for."""

    scaled: torch.Tensor
    sumsq: torch.Tensor
    width: int
    eps: float
    norm: object = None

    @property
    def shape(self):
        return self.scaled.shape

    @property
    def dtype(self):
        return self.scaled.dtype

    @property
    def device(self):
        return self.scaled.device

    def materialize(self, row_idx: Optional[torch.Tensor] = None) -> torch.Tensor:
        """The normalised rows as a plain tensor (all rows, or those named by ``row_idx``)."""
        from ..ops import kernels as K
        rows = self.scaled.shape[0] if row_idx is None else row_idx.shape[0]
        out = torch.empty((rows, self.scaled.shape[1]), dtype=self.scaled.dtype, device=self.scaled.device)
        return K.normed_rows_finish(self.scaled, self.sumsq, self.width, self.eps, out, row_idx)


@dataclass
class BranchTail:
    """What is to happen to a branch's output: it is added to ``hidden`` (the residual stream, in
    place) and the sum is handed to ``norm``, the norm that reads the stream next.  A mixer or
    feed-forward that is given a tail MAY do both inside its last product and return the
    :class:`NormedRows` prepared for ``norm``; returning its plain output instead is always
    allowed (the block then adds and normalises itself).  For a ``norm`` with
    ``takes_partial_sums`` the output may also come back as ``ops.kernels.PartialSums`` (fp32
    products over ranges of K, not yet added up): the block hands it to that norm as ``delta``
    like a plain output."""

    hidden: torch.Tensor
    norm: object


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

    def activation_elements(self) -> int:
        """Elements of intermediate results this part makes per token of a step (an estimate for
        sizing memory; 0 when negligible)."""
        return 0


class Norm(Part):
    def forward(self, x: torch.Tensor, out: Optional[torch.Tensor] = None,
                delta: Optional[torch.Tensor] = None,
                row_idx: Optional[torch.Tensor] = None) -> torch.Tensor:
        raise NotImplementedError

    def prepared_by_product(self):
        """``(weight, width, eps)`` if a product's epilogue may prepare this norm as
        :class:`NormedRows` (it must be ``x * rsqrt(mean(x^2) + eps) * weight``), else ``None``."""
        return None


class PositionEncoding(Part):
    def apply_and_cache(self, qkv: torch.Tensor, positions: torch.Tensor, num_q_heads: int,
                        num_kv_heads: int, head_dim: int, kv: Optional[KVView]) -> None:
        """Encodes positions into the Q and K heads of ``qkv`` in place and, when ``kv`` allows
        writing, stores the encoded K and the plain V at the tokens' cache slots."""
        raise NotImplementedError

    def rotate_half_tables(self, device, head_dim: int):
        """For encodings that a projection's epilogue can apply: ``(cos, sin)`` fp32 tables
        ``[positions, head_dim / 2]`` of a rotate-half rotation over the whole head
        (``out[j] = x[j] cos - x[j + d/2] sin``, ``out[j + d/2] = x[j] sin + x[j + d/2] cos``), or
        ``(None, None)`` if Q and K pass unchanged.  ``None`` (the default): the encoding is
        something else and only ``apply_and_cache`` applies it."""
        return None


class Mixer(Part):
    fuses_tail = False      # True: forward(x, ctx, tail=None) accepts NormedRows and a BranchTail
    # A mixer that can only take a prompt in portions that end on multiples of so many positions
    # (a state it carries is updated in blocks, say) says so here; the scheduler then cuts every
    # portion but a prompt's last at such a position.  Attention takes any cut: 1.
    portion_multiple = 1

    def kv_cache_spec(self) -> Optional[KVCacheSpec]:
        return None

    def state_spec(self) -> Optional[StateSpec]:
        return None

    def forward(self, x: torch.Tensor, ctx: MixerContext) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    fuses_tail = False

    def forward(self, x: torch.Tensor, ctx: MixerContext) -> torch.Tensor:
        raise NotImplementedError


class Block(Part):
    """The arrangement of a layer's parts.  ``norms`` holds the layer's norms by the names the
    arrangement knows; ``NORM_NAMES`` lists the names a subclass needs (checked here)."""

    NORM_NAMES: Tuple[str, ...] = ()

    def __init__(self, mixer: Mixer, feed_forward: FeedForward, norms: Dict[str, Norm]):
        super().__init__("")
        self.mixer, self.feed_forward = mixer, feed_forward
        self.norms = dict(norms)
        if set(self.norms) != set(self.NORM_NAMES):
            raise ValueError(f"{type(self).__name__} arranges norms named {sorted(self.NORM_NAMES)}, "
                             f"the layer gives {sorted(self.norms)}")

    def parts(self):
        return (*self.norms.values(), self.mixer, self.feed_forward)

    def forward(self, hidden: torch.Tensor, delta, ctx: MixerContext, next_norm: Optional[Norm] = None):
        """``delta`` is None, a plain branch output still to be added, or NormedRows prepared for
        this block's first norm.  ``next_norm`` is the norm that will read the stream after this
        block (the next block's first norm or the final norm)."""
        raise NotImplementedError

    def first_norm(self) -> Optional[Norm]:
        """The norm that reads the residual stream first in this block, if the block starts with
        one: the block before may then prepare it in its last product.  ``None``: the stream is
        handed over as it is."""
        return None
