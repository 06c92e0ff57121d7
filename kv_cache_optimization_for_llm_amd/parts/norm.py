"""RMSNorm: ``y = x / sqrt(mean(x^2) + eps) * w`` (reference: ``base/src/kernels.cu:10-36``).

The weight multiplies as stored (no ``1 + w``).  ``forward`` can fuse the residual add that
comes before the norm (``delta``) and a gather of rows (``row_idx``).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..config.registry import NORMS
from ..models.spec import TensorSpec
from ..ops import kernels as K
from .base import Norm


@NORMS.register("rmsnorm")
class RMSNorm(Norm):
    graph_safe = True
    takes_partial_sums = True       # ``delta`` may be ops.kernels.PartialSums (bf16 streams)

    def __init__(self, prefix: str, *, width: int, eps: float, weight_name: str = "weight"):
        super().__init__(prefix)
        self.width, self.eps = int(width), float(eps)
        self.weight_name = prefix + weight_name
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {self.weight_name: TensorSpec((self.width,), init="norm", role="vector")}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.weight = tensors[self.weight_name].contiguous()

    def prepared_by_product(self):
        return (self.weight, self.width, self.eps)

    def activation_elements(self) -> int:
        return self.width

    def forward(self, x, out=None, delta=None, row_idx=None):
        if out is None:
            rows = x.shape[0] if row_idx is None else row_idx.shape[0]
            out = torch.empty((rows, self.width), dtype=x.dtype, device=x.device)
        if isinstance(delta, K.PartialSums) and (x.dtype != torch.bfloat16 or self.width % 8):
            delta = delta.materialize()
        return K.rmsnorm(x, self.weight, self.eps, out, delta=delta, row_idx=row_idx)
