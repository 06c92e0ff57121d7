"""Pre-norm residual block: ``h += mixer(norm1(h)); h += ffn(norm2(h))``
(reference: ``base/src/engine.cu:639-859``).

The sums are made in fp32 and rounded to the storage type.  A branch output is handed on as
``delta`` and added inside the next norm kernel, which sees exactly the rounded sum a separate
residual kernel would have produced.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..config.registry import BLOCKS
from .base import Block, BranchTail, MixerContext, Norm, NormedRows


@BLOCKS.register("pre_norm")
class PreNormBlock(Block):
    graph_safe = True
    NORM_NAMES = ("mixer", "feed_forward")

    def __init__(self, mixer, feed_forward, norms):
        super().__init__(mixer, feed_forward, norms)
        self.mixer_norm, self.ffn_norm = self.norms["mixer"], self.norms["feed_forward"]

    def first_norm(self) -> Norm:
        return self.mixer_norm

    def forward(self, hidden: torch.Tensor, delta, ctx: MixerContext, next_norm: Optional[Norm] = None):
        # first norm: already prepared by the previous product, or add-and-normalise here
        if isinstance(delta, NormedRows):
            x = delta if getattr(self.mixer, "fuses_tail", False) else delta.materialize()
        else:
            x = self.mixer_norm.forward(hidden, delta=delta)
        if getattr(self.mixer, "fuses_tail", False):
            a = self.mixer.forward(x, ctx, tail=BranchTail(hidden, self.ffn_norm))
        else:
            a = self.mixer.forward(x, ctx)
        if isinstance(a, NormedRows):               # hidden has taken the mixer's output already
            x = a if getattr(self.feed_forward, "fuses_tail", False) else a.materialize()
        else:
            x = self.ffn_norm.forward(hidden, delta=a)
        if getattr(self.feed_forward, "fuses_tail", False):
            f = self.feed_forward.forward(x, ctx, tail=BranchTail(hidden, next_norm))
        else:
            f = self.feed_forward.forward(x, ctx)
        return hidden, f
