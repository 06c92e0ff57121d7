"""y = x @ W^T for a row-major ``[out, in]`` weight, without bias.

The reference calls cublasGemmEx for this (bf16 operands, fp32 accumulate,
``base/src/engine.cu:652-671``).  Here:

* bf16 weight, bf16 activations: hand-written MFMA kernels where they exist for the shape,
  otherwise the vendor GEMM library (``ops.kernels.gemm_vendor``, as the reference uses cuBLAS);
* fp32 weight: the true-fp32 kernel ``gemm_nt_f32``; bf16 activations are widened for it and
  the result is rounded back, so a tensor stored in 32-bit is used in 32-bit.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..ops import kernels as K
from .base import BranchTail, NormedRows


class Linear:
    def __init__(self, weight: torch.Tensor, halves: int = 1):
        """``halves=2``: the weight is two matrices joined along the rows (gate and up)."""
        if weight.dim() != 2:
            raise ValueError(f"Linear weight must be 2-D, got {tuple(weight.shape)}")
        self.weight = weight.contiguous()
        self.out_features, self.in_features = weight.shape
        self.halves = halves
        # a second, tiled copy for the few-rows kernel (decode); the plain layout serves prompts
        self.tiled = None
        if weight.is_cuda and weight.dtype == torch.bfloat16:
            K.gemm_vendor_init()            # the library's handle and workspace exist before any step
            if self.in_features % 32 == 0:
                self.tiled = K.TiledWeight(self.weight, halves)

    GEMV, FEW_ROWS = "gemv", "few_rows"
    # The matrix-vector product adds an attention output's partial results up itself only for up to
    # 2,048 inputs: beyond, the registers that hold them cost it more than the merge launch saved
    # (decode steps of one / two requests at 700 keys, 8 layers of the 3B sizes, 3,072 inputs of heads
    # of 128: 0.536 / 0.578 -> 0.537 / 0.609 ms; 8B sizes, 4,096 inputs: 0.862 / 0.906 -> 0.854 / 0.964;
    # 1B sizes, 2,048 inputs of heads of 64, 16 layers: 0.688 / 0.769 -> 0.660 / 0.741).
    MERGES_UP_TO_INPUTS = 2048

    def fused_kernel(self, rows: int, dtype, rotated: bool = False) -> Optional[str]:
        """The hand-written product that takes ``rows`` rows of ``dtype`` with a norm on its input
        and/or the residual stream in its epilogue: ``GEMV`` (one token: a matrix-vector product
        over the plain weight), ``FEW_ROWS`` (the matrix-core kernel over the tiled copy) or None.
        ``rotated``: the product asked about is the joined Q/K/V product with rotation and cache
        write in its epilogue."""
        from ..ops.gemm_bf16 import use_gemv, use_skinny
        if dtype != torch.bfloat16 or self.weight.dtype != torch.bfloat16 or not self.weight.is_cuda:
            return None
        if use_gemv(rows, self.out_features, self.in_features):
            return self.GEMV
        if self.tiled is not None and use_skinny(rows, self.out_features, self.in_features, self.halves == 2, rotated):
            return self.FEW_ROWS
        return None

    def fusable(self, x) -> bool:
        """Whether this product can finish a norm on its input and/or feed the residual stream
        in its epilogue for these rows (bf16 everywhere, few rows)."""
        return self.fused_kernel(x.shape[0], x.dtype) is not None

    def residual_kernel(self, rows: int, dtype, tail: Optional[BranchTail]) -> Optional[str]:
        """The kernel with which :meth:`into_residual` will fuse ``rows`` rows of ``dtype``, or None
        (with ``FEW_ROWS`` its input may come as ``ops.kernels.TiledRows``)."""
        prep = tail.norm.prepared_by_product() if tail is not None and tail.norm is not None else None
        if prep is None or prep[1] != self.out_features or tail.hidden.dtype != torch.bfloat16:
            return None
        return self.fused_kernel(rows, dtype)

    def takes_attention_partials(self, rows: int, dtype, tail: Optional[BranchTail], head_dim: int) -> int:
        """How many partial results a row (``ops.kernels.AttentionPartials``) :meth:`into_residual`
        can add up itself for ``rows`` rows of heads of ``head_dim``; 0: none, it wants the output."""
        if self.residual_kernel(rows, dtype, tail) != self.GEMV or self.in_features > self.MERGES_UP_TO_INPUTS:
            return 0
        most = K.gemv_merge_max_parts(rows)
        return most if K.gemv_merged_supported(rows, self.out_features, self.in_features, head_dim, most) else 0

    def into_residual(self, x, tail: BranchTail):
        """hidden += x @ W^T in place and the sum prepared for ``tail.norm`` (NormedRows); or, at
        17 to 64 rows of a matrix that the few-rows kernel does not take whole, the product as
        ``ops.kernels.PartialSums`` for a ``tail.norm`` that says it adds them up
        (``takes_partial_sums``); ``None`` when neither is possible (the caller then takes the
        plain product)."""
        kernel = self.residual_kernel(x.shape[0], x.dtype, tail)
        if kernel is None:
            return self._partial_sums(x, tail)
        next_w, width, eps = tail.norm.prepared_by_product()
        rows = x.shape[0]
        scaled = torch.empty((rows, self.out_features), dtype=torch.bfloat16, device=x.device)
        norm = {}
        if isinstance(x, NormedRows):
            norm = dict(sumsq=x.sumsq, norm_width=x.width, eps=x.eps)
            x = x.scaled
        if isinstance(x, K.AttentionPartials) and kernel != self.GEMV:
            raise K.KernelError("Linear.into_residual: partial results were left for a product that cannot add them up")
        if kernel == self.GEMV:
            if isinstance(x, K.TiledRows):
                x = x.to_rows()
            sumsq = torch.empty((rows, K.gemv_sumsq_parts(self.out_features, self.in_features)),
                                dtype=torch.float32, device=x.device)
            if isinstance(x, K.AttentionPartials):
                K.gemv_merged(x, self.weight, tail.hidden, next_w, scaled, sumsq)
            else:
                K.gemv(x, self.weight, None, hidden=tail.hidden, next_weight=next_w, scaled_out=scaled,
                       sumsq_out=sumsq, **norm)
        else:
            sumsq = torch.empty((rows, K.gemm_skinny_sumsq_parts(self.out_features)), dtype=torch.float32,
                                device=x.device)
            K.gemm_skinny(x, self.tiled, None, hidden=tail.hidden, next_weight=next_w, scaled_out=scaled,
                          sumsq_out=sumsq, x_tiled=isinstance(x, K.TiledRows), **norm)
        return NormedRows(scaled, sumsq, width, eps, tail.norm)

    def _partial_sums(self, x, tail: Optional[BranchTail]):
        from ..ops.gemm_bf16 import use_partial_sums
        if tail is None or not getattr(tail.norm, "takes_partial_sums", False) or self.tiled is None \
                or not isinstance(x, torch.Tensor) or x.dtype != torch.bfloat16 or tail.hidden.dtype != torch.bfloat16 \
                or self.out_features % 8 or not use_partial_sums(x.shape[0], self.out_features, self.in_features):
            return None
        return K.gemm_skinny_partials(x, self.tiled)

    def gated(self, x, out) -> None:
        """``out`` = silu(x gate^T) * (x up^T) for a joined [gate; up] weight whose rows
        :meth:`fusable` accepts; ``out`` is [rows, out_features / 2] or, for the few-rows kernel,
        an ``ops.kernels.TiledRows`` of that size."""
        norm = {}
        if isinstance(x, NormedRows):
            norm = dict(sumsq=x.sumsq, norm_width=x.width, eps=x.eps)
            x = x.scaled
        if self.fused_kernel(x.shape[0], x.dtype) == self.GEMV:
            K.gemv(x, self.weight, out, swiglu=True, **norm)
        else:
            K.gemm_skinny(x, self.tiled, out, swiglu=True, out_tiled=isinstance(out, K.TiledRows), **norm)

    def __call__(self, x, out: Optional[torch.Tensor] = None,
                 out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        if isinstance(x, NormedRows):
            kernel = self.fused_kernel(x.shape[0], x.dtype)
            if kernel is not None:
                if out is None:
                    out = torch.empty((x.shape[0], self.out_features), dtype=out_dtype or x.dtype,
                                      device=x.device)
                if kernel == self.GEMV:
                    return K.gemv(x.scaled, self.weight, out, sumsq=x.sumsq, norm_width=x.width, eps=x.eps)
                return K.gemm_skinny(x.scaled, self.tiled, out, sumsq=x.sumsq, norm_width=x.width, eps=x.eps)
            x = x.materialize()
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
        return gemm_bf16.linear_bf16(x, w, out, self.tiled)
