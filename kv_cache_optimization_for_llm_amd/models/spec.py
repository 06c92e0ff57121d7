"""A model as data: which parts each layer is made of, and in which order layers run."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Mapping, Optional, Tuple


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
    """One layer: a block arrangement around a mixer and a feed-forward, with its norms by name.

    ``norms`` maps the names the block arrangement knows (the pre-norm block: ``"mixer"`` and
    ``"feed_forward"``, the norms in front of the two branches; an arrangement with norms after
    its branches too, or with a single one, names its own) to their specs.  The order of the
    mapping is the order in which the block's parts are listed."""

    block: PartSpec                      # e.g. PartSpec("pre_norm")
    mixer: PartSpec
    feed_forward: PartSpec
    norms: Mapping[str, PartSpec]
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
    # Constants around the layers (1 and 0 leave a value as it is): the rows taken from the token
    # table are multiplied by ``embedding_scale``; logits are multiplied by ``logit_scale`` and
    # then, with a positive ``logit_softcap`` c, replaced by c * tanh(logit / c).
    embedding_scale: float = 1.0
    logit_scale: float = 1.0
    logit_softcap: float = 0.0
    eos_token_ids: Tuple[int, ...] = ()
    ignorable_tensors: Tuple[str, ...] = ()   # fnmatch patterns of tensors that may be present unused


def default_order(num_layers: int) -> Tuple[LayerCall, ...]:
    return tuple(LayerCall(layer=i, cache=i) for i in range(num_layers))
