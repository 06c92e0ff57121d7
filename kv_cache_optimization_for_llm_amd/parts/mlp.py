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
from .base import BranchTail, FeedForward, MixerContext, NormedRows
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
        self.gate_up = Linear(torch.cat([g, u], dim=0), halves=2)
        self.down = Linear(tensors[p + "down_proj.weight"])

    fuses_tail = True

    def activation_elements(self) -> int:
        # gate and up, their gated product, the down projection
        return 3 * self.intermediate_size + self.hidden_size

    def forward(self, x, ctx: MixerContext, tail: Optional[BranchTail] = None):
        """``x`` may be NormedRows; with a ``tail`` the down projection adds into the residual
        stream and prepares the next norm when the shapes allow (NormedRows are returned)."""
        rows = x.shape[0]
        up_kernel = self.gate_up.fused_kernel(rows, x.dtype)
        # Both products in their few-rows form and at most 16 rows: the activations go from one to
        # the other in the order the second one's lanes read them (ops.kernels.TiledRows).
        tiled = (up_kernel == Linear.FEW_ROWS and rows <= K.TiledRows.MAX_ROWS and self.intermediate_size % 8 == 0
                 and self.down.residual_kernel(rows, x.dtype, tail) == Linear.FEW_ROWS)
        if tiled:
            act = K.TiledRows(rows, self.intermediate_size, x.device)
        else:
            act = torch.empty((rows, self.intermediate_size), dtype=x.dtype, device=x.device)
        if up_kernel is not None:
            # activation fused into the product; an unfinished input norm is finished there too
            self.gate_up.gated(x, act)
        else:
            K.silu_mul(self.gate_up(x), act)
        if tail is not None:
            fused = self.down.into_residual(act, tail)
            if fused is not None:
                return fused
        if tiled:
            act = act.to_rows()
        return self.down(act)
