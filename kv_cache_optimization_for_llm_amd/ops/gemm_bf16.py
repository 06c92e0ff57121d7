"""bf16 matrix products: picks the kernel for a shape.

``linear_bf16(x, w, out)`` computes ``out = x @ w^T`` with fp32 accumulation.  ``out`` may be
bf16 or fp32.  Up to 16 rows (decode steps, short portions) take the hand-written matrix-core
kernel that streams a tiled copy of the weight once (``csrc/gemm_skinny.hip``).  Other shapes go to the vendor
GEMM library through ``torch.matmul``, which is where the reference's engine uses cuBLAS.
"""
from __future__ import annotations

import torch

from . import kernels as K


# Measured on MI355X at the Llama-3.2-1B shapes: up to 16 rows the few-rows kernel beats the vendor
# GEMM (weights streamed at 5+ TB/s, norms and activation fused); from 32 rows on the vendor
# GEMM's tiles win because the few-rows kernel re-reads X once per 16 rows of W.
SKINNY_MAX_ROWS = 16


def use_skinny(m: int, n: int, k: int) -> bool:
    return m <= SKINNY_MAX_ROWS and K.gemm_skinny_supported(m, n, k)


def linear_bf16(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, tiled=None) -> torch.Tensor:
    """``tiled`` is the weight's :class:`~.kernels.TiledWeight` when it has one."""
    if not (x.is_cuda and w.is_cuda and out.is_cuda):
        raise K.KernelError("linear_bf16: operands must be on the GPU")
    if x.shape[1] != w.shape[1] or out.shape != (x.shape[0], w.shape[0]):
        raise K.KernelError(f"linear_bf16: x {tuple(x.shape)} w {tuple(w.shape)} out "
                            f"{tuple(out.shape)} do not fit")
    if x.shape[0] == 0:
        return out
    if tiled is not None and use_skinny(x.shape[0], w.shape[0], w.shape[1]):
        return K.gemm_skinny(x, tiled, out)
    if out.dtype == torch.bfloat16:
        torch.matmul(x, w.t(), out=out)
    else:
        tmp = torch.matmul(x, w.t())
        K.cast(tmp, out)
    return out
