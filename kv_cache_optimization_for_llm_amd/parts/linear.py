"""y = x @ W^T for a row-major ``[out, in]`` weight, without bias.

The reference calls cublasGemmEx for this (bf16 operands, fp32 accumulate,
``base/src/engine.cu:652-671``).  Here:

* bf16 weight, bf16 activations: hand-written MFMA kernels where they exist for the shape,
  otherwise the vendor GEMM library through ``torch.matmul`` (as the reference uses cuBLAS);
* fp32 weight: the true-fp32 kernel ``gemm_nt_f32``; bf16 activations are widened for it and
  the result is rounded back, so a tensor stored in 32-bit is used in 32-bit.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..ops import kernels as K


class Linear:
    def __init__(self, weight: torch.Tensor):
        if weight.dim() != 2:
            raise ValueError(f"Linear weight must be 2-D, got {tuple(weight.shape)}")
        self.weight = weight.contiguous()
        self.out_features, self.in_features = weight.shape

    def __call__(self, x: torch.Tensor, out: Optional[torch.Tensor] = None,
                 out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        w = self.weight
        rows = x.shape[0]
        want = out_dtype or (out.dtype if out is not None else x.dtype)
        if out is None:
            out = torch.empty((rows, self.out_features), dtype=want, device=x.device)
        if w.dtype == torch.float32:
            x32 = x if x.dtype == torch.float32 else K.cast(x, torch.empty_like(x, dtype=torch.float32))
            if out.dtype == torch.float32:
                K.gemm_nt_f32(x32, w, out)
            else:
                y32 = torch.empty((rows, self.out_features), dtype=torch.float32, device=x.device)
                K.gemm_nt_f32(x32, w, y32)
                K.cast(y32, out)
            return out
        # bf16 weight
        if x.dtype != torch.bfloat16:
            raise K.KernelError("Linear: a bfloat16 weight needs bfloat16 activations")
        from ..ops import gemm_bf16
        return gemm_bf16.linear_bf16(x, w, out)
