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
from .base import Block, MixerContext


@BLOCKS.register("pre_norm")
class PreNormBlock(Block):
    graph_safe = True

    def forward(self, hidden: torch.Tensor, delta: Optional[torch.Tensor], ctx: MixerContext):
        x = self.mixer_norm.forward(hidden, delta=delta)
        a = self.mixer.forward(x, ctx)
        x = self.ffn_norm.forward(hidden, out=x, delta=a)
        f = self.feed_forward.forward(x, ctx)
        return hidden, f
