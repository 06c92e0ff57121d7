"""A model as data: which parts each layer is made of, and in which order layers run."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple


@dataclass(frozen=True)
class PartSpec:
    """Kind of a part (a registry key) and the constants it is built with."""

    kind: str
    params: Dict[str, Any] = field(default_factory=dict)


@dataclass(frozen=True)
class TensorSpec:
    """One tensor a part reads from the checkpoint.

    ``init`` names the random-weights rule: ``"normal"`` (N(0, 0.02)), ``"norm"``
    (1 + U(-0.1, 0.1)) or ``"zeros"``.  ``role`` is ``"matrix"`` (takes the engine's compute
    dtype unless stored in 32-bit), ``"vector"`` (same rule) or ``"table"`` (integers, int32).
    """

    shape: Tuple[int, ...]
    init: str = "normal"
    role: str = "matrix"


@dataclass(frozen=True)
class LayerSpec:
    """One layer: a block arrangement around a mixer and a feed-forward."""

    block: PartSpec                      # e.g. PartSpec("pre_norm")
    mixer: PartSpec
    feed_forward: PartSpec
    mixer_norm: PartSpec
    ffn_norm: PartSpec
    prefix: str                          # tensor-name prefix, e.g. "model.layers.3."


@dataclass(frozen=True)
class LayerCall:
    """One entry of the run order.

    ``layer`` indexes ``ModelSpec.layers`` (the weights).  ``cache`` names the cache slot the
    mixer uses; two calls with the same ``cache`` share keys and values.  A call with
    ``writes_cache=False`` only reads that slot (it attends to what another call wrote this
    step and before).  ``cache=None`` means one private slot per call.
    """

    layer: int
    cache: Optional[int] = None
    writes_cache: bool = True


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    hidden_size: int
    vocab_size: int
    embedding_name: str                  # tensor name of the token table [vocab, hidden]
    layers: Tuple[LayerSpec, ...]
    order: Tuple[LayerCall, ...]
    final_norm: PartSpec
    final_norm_prefix: str
    head_name: Optional[str]             # tensor name of the output matrix; None = tied to the table
    max_positions: int
    eos_token_ids: Tuple[int, ...] = ()
    ignorable_tensors: Tuple[str, ...] = ()   # fnmatch patterns of tensors that may be present unused


def default_order(num_layers: int) -> Tuple[LayerCall, ...]:
    return tuple(LayerCall(layer=i, cache=i) for i in range(num_layers))
