"""Chooses the attention kernel for a step's batch."""
from __future__ import annotations

import torch

from . import kernels as K


def paged_attention(qkv: torch.Tensor, out: torch.Tensor, kv, batch, num_q_heads: int,
                    num_kv_heads: int, head_dim: int, scale: float, window: int = 0) -> torch.Tensor:
    """Causal GQA attention of the step's tokens over the paged cache.  ``qkv`` is the fused
    projection output ``[T, (nq + 2 nkv) d]`` whose first ``nq * d`` columns are the (already
    position-encoded) queries; keys and values are read from ``kv``."""
    if kv is None:
        raise K.KernelError("paged_attention: the mixer has no cache view")
    return K.attention_rowwise(qkv, qkv.shape[1], out, kv.k_cache, kv.v_cache, kv.block_table,
                               batch.tok_seat, batch.positions, num_q_heads, num_kv_heads,
                               head_dim, scale, window)
