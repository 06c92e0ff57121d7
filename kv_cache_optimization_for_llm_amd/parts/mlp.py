"""SwiGLU feed-forward: ``down( silu(gate(x)) * up(x) )``, no biases
(reference: ``base/src/engine.cu:780-858``, ``siluKernel`` ``base/src/kernels.cu:45-52``).

Gate and up matrices are joined at load time into one ``[2 * intermediate, hidden]`` matrix.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..config.registry import FEED_FORWARDS
from ..models.spec import TensorSpec
from ..ops import kernels as K
from .base import FeedForward, MixerContext
from .linear import Linear


@FEED_FORWARDS.register("swiglu")
class SwiGLU(FeedForward):
    graph_safe = True

    def __init__(self, prefix: str, *, hidden_size: int, intermediate_size: int):
        super().__init__(prefix)
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.gate_up: Optional[Linear] = None
        self.down: Optional[Linear] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        p, h, i = self.prefix, self.hidden_size, self.intermediate_size
        return {
            p + "gate_proj.weight": TensorSpec((i, h)),
            p + "up_proj.weight": TensorSpec((i, h)),
            p + "down_proj.weight": TensorSpec((h, i)),
        }

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        p = self.prefix
        g, u = tensors[p + "gate_proj.weight"], tensors[p + "up_proj.weight"]
        if g.dtype != u.dtype:
            raise ValueError(f"{p}: gate and up projection weights are stored in different dtypes")
        self.gate_up = Linear(torch.cat([g, u], dim=0))
        self.down = Linear(tensors[p + "down_proj.weight"])

    def forward(self, x: torch.Tensor, ctx: MixerContext) -> torch.Tensor:
        act = torch.empty((x.shape[0], self.intermediate_size), dtype=x.dtype, device=x.device)
        w = self.gate_up.weight
        if x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 \
                and K.gemm_skinny_supported(x.shape[0], w.shape[0], w.shape[1]):
            K.gemm_skinny(x, w, act, swiglu=True)      # activation fused into the product
        else:
            K.silu_mul(self.gate_up(x), act)
        return self.down(act)
