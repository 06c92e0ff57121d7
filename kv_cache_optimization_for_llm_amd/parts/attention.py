"""Grouped-query causal attention over the paged cache (the Llama mixer).

Per token (reference order, ``base/src/engine.cu:652-762``): Q, K, V projections without bias
-> position encoding of Q and K -> K and V written to the cache -> scores ``q.k * scale`` over
the request's keys up to the token's own position (optionally only the last ``window``),
softmax in fp32 -> ``P V`` -> output projection.  ``kv_head = q_head // (num_heads / num_kv_heads)``.

The three projection matrices are joined at load time into one ``[nq*d + 2*nkv*d, hidden]``
matrix, so the step runs one product instead of three.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..config.registry import MIXERS, POSITION_ENCODINGS
from ..models.spec import PartSpec, TensorSpec
from ..ops import attention as attn_ops
from ..ops import kernels as K
from ..ops.gemm_bf16 import SKINNY_MAX_ROWS
from .base import BranchTail, KVCacheSpec, Mixer, MixerContext, NormedRows, attention_cache_spec
from .linear import Linear


class EncodedQKV:
    """The joined Q/K/V projection with position encoding and cache write: what every mixer that
    attends over cached keys does first.  It owns the choice between one product that does all of
    it in its epilogue (few rows, an encoding that is a rotate-half rotation over the whole head,
    or none) and the product followed by the encoding's own kernel, so that a mixer - this one or
    another attention variant - only says ``qkv(x, batch, kv)``."""

    # Above 16 decoded tokens the library's product followed by the attention kernel that rotates and
    # caches inside is ahead of the few-rows product with that work in its epilogue, except for large
    # matrices at many rows.  Whole decode steps at 768 keys, ms, epilogue -> attention kernel:
    # 1B sizes (3,072 x 2,048) 17 / 24 / 32 requests 1.188 / 1.243 / 1.292 -> 1.133 / 1.194 / 1.245;
    # 8 layers of the 3B sizes (5,120 x 3,072) 17 / 32 / 48: 0.855 / 0.929 / 1.040 -> 0.838 / 0.927 / 1.007;
    # 8 layers of the 8B sizes (6,144 x 4,096) 17 / 24: 1.262 / 1.298 -> 1.259 / 1.281, but 32 / 40 / 48:
    # 1.288 / 1.386 / 1.374 -> 1.292 / 1.400 / 1.416.
    ROTATE_LATER_ROWS = 24
    ROTATE_LATER_ELEMENTS = 1 << 24

    def __init__(self, linear: Linear, position, hidden_size: int, num_heads: int, num_kv_heads: int,
                 head_dim: int):
        self.linear, self.position = linear, position
        self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim = hidden_size, num_heads, num_kv_heads, head_dim
        self.pending_rotation = None          # set by a call that left encoding and cache write to the attention kernel

    def __call__(self, x, batch, kv):
        """``x`` [T, hidden] (plain or NormedRows).  Returns a tensor whose first ``nq * d`` columns
        are the position-encoded queries; K (encoded) and V of the step's tokens are in the cache
        when ``kv`` allows writing.  Or, with ``self.pending_rotation`` set to the (cos, sin) tables
        (or (None, None)), the joined projection as the product left it: encoding and cache write
        are then the attention kernel's (``ops.attention.paged_attention(..., rope=...)``)."""
        self.pending_rotation = None
        tables, rows = None, x.shape[0]
        kernel = self.linear.fused_kernel(rows, x.dtype, rotated=True)
        if kernel == Linear.GEMV and not K.gemv_qkv_rope_supported(rows, self.hidden_size, self.head_dim):
            kernel = Linear.FEW_ROWS if self.linear.tiled is not None else None
        if kernel == Linear.FEW_ROWS and not K.gemm_skinny_qkv_rope_supported(rows, self.hidden_size, self.head_dim):
            kernel = None
        if (kernel == Linear.FEW_ROWS and rows > SKINNY_MAX_ROWS
                and (rows <= self.ROTATE_LATER_ROWS or self.linear.weight.numel() <= self.ROTATE_LATER_ELEMENTS)
                and attn_ops.rotates_in_kernel(batch, kv, self.num_heads, self.num_kv_heads, self.head_dim, x.dtype)):
            kernel = None
        if kernel is not None:
            tables = self.position.rotate_half_tables(x.device, self.head_dim)
        if tables is None:
            qkv = self.linear(x)
            # decoded tokens only: rotation and cache write go into the attention kernel, which
            # takes the product as it is (one launch less per layer where the product is the library's)
            later = self.position.rotate_half_tables(x.device, self.head_dim)
            if later is not None and attn_ops.rotates_in_kernel(batch, kv, self.num_heads, self.num_kv_heads,
                                                                self.head_dim, qkv.dtype):
                self.pending_rotation = later
                return qkv
            self.position.apply_and_cache(qkv, batch.positions, self.num_heads, self.num_kv_heads,
                                          self.head_dim, kv)
            return qkv
        write = kv is not None and kv.writes
        q = torch.empty((rows, self.num_heads * self.head_dim), dtype=torch.bfloat16, device=x.device)
        norm = {}
        if isinstance(x, NormedRows):
            norm = dict(sumsq=x.sumsq, norm_width=x.width, eps=x.eps)
            x = x.scaled
        product, weight = ((K.gemv_qkv_rope, self.linear.weight) if kernel == Linear.GEMV
                           else (K.gemm_skinny_qkv_rope, self.linear.tiled))
        product(x, weight, q, self.num_heads, self.num_kv_heads, self.head_dim,
                batch.positions, tables[0], tables[1],
                kv.k_cache if write else None, kv.v_cache if write else None,
                kv.slot_mapping if write else None, kv.page_size if kv is not None else 0, **norm)
        return q


@MIXERS.register("gqa_attention")
class GQAAttention(Mixer):
    graph_safe = True

    def __init__(self, prefix: str, *, hidden_size: int, num_heads: int, num_kv_heads: int,
                 head_dim: int, scale: float, position: PartSpec, window: int = 0):
        super().__init__(prefix)
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads is not a multiple of {num_kv_heads} kv heads")
        self.hidden_size, self.num_heads, self.num_kv_heads = hidden_size, num_heads, num_kv_heads
        self.head_dim, self.scale, self.window = head_dim, float(scale), int(window)
        self.position = POSITION_ENCODINGS.get(position.kind)(**position.params)
        self.qkv: Optional[EncodedQKV] = None
        self.o: Optional[Linear] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        p, d = self.prefix, self.head_dim
        return {
            p + "q_proj.weight": TensorSpec((self.num_heads * d, self.hidden_size)),
            p + "k_proj.weight": TensorSpec((self.num_kv_heads * d, self.hidden_size)),
            p + "v_proj.weight": TensorSpec((self.num_kv_heads * d, self.hidden_size)),
            p + "o_proj.weight": TensorSpec((self.hidden_size, self.num_heads * d)),
        }

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        p = self.prefix
        q, k, v = (tensors[p + n + "_proj.weight"] for n in "qkv")
        if not (q.dtype == k.dtype == v.dtype):
            raise ValueError(f"{p}: q/k/v projection weights are stored in different dtypes")
        self.qkv = EncodedQKV(Linear(torch.cat([q, k, v], dim=0)), self.position, self.hidden_size,
                              self.num_heads, self.num_kv_heads, self.head_dim)
        self.o = Linear(tensors[p + "o_proj.weight"])

    def kv_cache_spec(self) -> KVCacheSpec:
        return attention_cache_spec(self.num_kv_heads, self.head_dim,
                                    kind="window" if self.window > 0 else "full", window=self.window)

    fuses_tail = True

    def activation_elements(self) -> int:
        # the joined projection, the attention output and the output projection
        return (2 * self.num_heads + 2 * self.num_kv_heads) * self.head_dim + self.hidden_size

    def forward(self, x, ctx: MixerContext, tail: Optional[BranchTail] = None):
        """``x`` may be NormedRows (the input norm is then finished inside the QKV product); with
        a ``tail`` the output projection adds into the residual stream and prepares the next
        norm when the shapes allow, and NormedRows are returned instead of the plain output."""
        batch, kv = ctx.batch, ctx.kv
        qkv = self.qkv(x, batch, kv)
        out = torch.empty((x.shape[0], self.num_heads * self.head_dim), dtype=x.dtype, device=x.device)
        # an output projection that adds the key ranges' partial results up itself (one or two
        # decoded tokens) is told so: the attention kernel may then leave them unmerged
        max_parts = self.o.takes_attention_partials(x.shape[0], x.dtype, tail, self.head_dim) \
            if self.qkv.pending_rotation is None else 0
        out = attn_ops.paged_attention(qkv, out, kv, batch, self.num_heads, self.num_kv_heads,
                                       self.head_dim, self.scale, self.window, rope=self.qkv.pending_rotation,
                                       max_parts=max_parts)
        if tail is not None:
            fused = self.o.into_residual(out, tail)
            if fused is not None:
                return fused
        return self.o(out)
