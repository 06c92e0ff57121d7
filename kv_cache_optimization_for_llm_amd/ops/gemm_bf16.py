"""bf16 matrix products: picks the kernel for a shape.

``linear_bf16(x, w, out)`` computes ``out = x @ w^T`` with fp32 accumulation.  ``out`` may be
bf16 or fp32.  Few rows (decode steps, short portions; how few depends on the matrix, see
``use_skinny``) take the hand-written matrix-core kernel that streams a tiled copy of the weight
once (``csrc/gemm_skinny.hip``).  Other shapes go to the vendor GEMM library (hipBLASLt, called
directly with the algorithm of a shape looked up once: ``csrc/gemm_vendor.hip``), which is where
the reference's engine uses cuBLAS.
"""
from __future__ import annotations

import torch

from . import kernels as K


# Measured on MI355X at the Llama-3.2-1B shapes with weights that are not in any cache, whole
# decode steps timed:
# * up to 16 rows the few-rows kernel beats the vendor GEMM everywhere (weights streamed once at
#   5+ TB/s, norms, rotation, activation and residual fused);
# * up to 32 rows it still wins for small matrices (the Q/K/V and output projections), where a
#   launch costs more than the product and its epilogues replace 5 us kernels, and for matrices
#   with many more rows than columns (the joined gate/up matrix: many workgroups, SwiGLU fused);
#   not for the down projection (few row tiles, long K: the vendor GEMM's split wins), and at 64
#   rows the vendor GEMM wins everywhere because the few-rows kernel re-reads X once per 16 rows of W;
# * the vocabulary-sized product (4 row tiles of W per wave share each X fragment, fp32 output
#   without a cast) wins up to 48 rows.
# Where "small" ends, whole decode steps of 17 / 24 / 32 requests at the 3B and 8B layer sizes: the
# output projection by the few-rows kernel, 3,072 x 3,072: 2.80 / 2.94 / 3.04 -> 2.74 / 2.89 / 3.02
# ms; 4,096 x 4,096: 4.55 / 4.75 / 4.91 -> 4.62 / 4.82 / 5.03.  The Q/K/V product with rotation and
# cache write in its epilogue (it stands for the library's product and the rotation kernel) gains
# at both: 3B 2.80 -> 2.77 (5,120 x 3,072), 8B 4.55 -> 4.52 (6,144 x 4,096); for those larger
# matrices up to 48 rows (decode steps of 40 / 48 requests: 3B 3.26 / 3.25 -> 3.20 / 3.20 ms, 8B 5.17 /
# 5.16 -> 5.09 / 5.08; at 64 rows a tie at 8B and a loss at 3B; at the 1B sizes a tie at 48 already).
SKINNY_MAX_ROWS = 16            # every shape
SKINNY_MID_ROWS = 32            # small or tall matrices, and the Q/K/V product with its epilogue
SKINNY_MID_ELEMENTS = 3 << 22
# Small matrices whole (with their epilogue) only up to 20 rows since their partial products over
# ranges of K, added up by the norm kernel, exist: decode steps of 17 / 24 / 32 requests, output
# projection whole -> in ranges: 1B sizes 1.108 / 1.141 / 1.204 -> 1.125 / 1.126 / 1.176 ms, 8 layers
# of the 3B sizes 18 / 24 / 32 requests 0.806 / 0.834 / 0.881 -> 0.806 / 0.828 / 0.858.
SKINNY_SMALL_ROWS = 20
SKINNY_ROTATED_ROWS = 48        # the Q/K/V product with its epilogue, matrices above SKINNY_MID_ELEMENTS
SKINNY_WIDE_ROWS = 64           # matrices whose waves share X through LDS
SKINNY_WIDE_N = 32768


def use_skinny(m: int, n: int, k: int, gated: bool = False, rotated: bool = False) -> bool:
    """``gated``: the weight is a joined [gate; up] matrix whose product is taken with the
    activation fused; ``rotated``: a joined [q; k; v] matrix whose product is taken with rotation
    and cache write fused."""
    if not K.gemm_skinny_supported(m, n, k):
        return False
    if m <= SKINNY_MAX_ROWS:
        return True
    if m <= SKINNY_MID_ROWS and (rotated or (n * k <= SKINNY_MID_ELEMENTS and m <= SKINNY_SMALL_ROWS) or n >= 4 * k):
        return True
    if rotated and m <= SKINNY_ROTATED_ROWS and n * k > SKINNY_MID_ELEMENTS:
        return True
    return m <= SKINNY_WIDE_ROWS and (n >= SKINNY_WIDE_N or (gated and n >= 4 * k))


def use_partial_sums(m: int, n: int, k: int) -> bool:
    """17 to 64 rows of a product that goes into the residual stream and that the few-rows kernel
    does not take whole: its shared-X form over ranges of K (``kernels.gemm_skinny_partials``)
    instead of the vendor library, the norm kernel adding the ranges up."""
    return SKINNY_MAX_ROWS < m <= SKINNY_WIDE_ROWS and K.gemm_skinny_partial_ranges(m, n, k) >= 1


# One or two tokens go to the matrix-vector kernel over the plain weight (csrc/gemv.hip): measured
# inside a graph at the 1B sizes with the epilogues the model uses, one token, it takes 5.5 / 4.2 /
# 12.6 / 8.6 microseconds for Q/K/V, output, gate/up and down against the few-rows kernel's 7.3 /
# 5.8 / 13.5 / 13.1, and a decode step of one request 0.70 ms against 0.85 (two: 0.78 against 0.86).
GEMV_MAX_ROWS = 2
# From 5,120 inputs on a wavefront of that kernel has one row of W in flight, and with two tokens
# its dot products, not the stream, set its time; the few-rows kernel's time does not depend on
# one or two tokens.  Alone in a graph, residual epilogue, microseconds for one / two tokens,
# matrix-vector against few-rows kernel: [3072 x 5120] 7.6 / 10.4 against 9.8 / 9.8, [4096 x 7168]
# 12.4 / 17.4 against 13.1 / 13.1, [3072 x 8192] 12.8 / 15.5 against 11.9 / 11.9, [8192 x 8192]
# 26.6 / 33.4 against 24.6 / 24.7; with 2,048 rows of W the matrix-vector kernel wins at every K
# ([2048 x 8192]: 8.8 / 10.6 against 10.7 / 10.9), and at K up to 4,096 the two are within 4 %.
# Decode steps of one / two requests at the 3B sizes (8 layers; the down projection is
# [3072 x 8192]): 0.552 / 0.614 -> 0.535 / 0.577 ms.
GEMV_WIDE_N = 3072
GEMV_LONG_K = {1: 8192, 2: 5120}


def use_gemv(m: int, n: int, k: int) -> bool:
    if m > GEMV_MAX_ROWS or not K.gemv_supported(m, n, k):
        return False
    return not (n >= GEMV_WIDE_N and k >= GEMV_LONG_K[m] and K.gemm_skinny_supported(m, n, k))


def decode_tune_rows(max_rows: int) -> list:
    """Row counts for which a server with ``max_rows`` seats has the vendor library's algorithms
    timed at start-up: the powers of two from 32 and ``max_rows`` itself.  A row count that was not
    timed takes what was found for the nearest timed one above it, up to twice its size, so these
    cover every decode batch above the few-rows kernels' 16 (a shape costs a fraction of a second;
    decode steps of 17 / 24 / 32 requests at the 1B sizes: 1.22 / 1.27 / 1.36 ms with the library's
    own choice, 1.19 / 1.25 / 1.31 with 32 rows timed)."""
    rows, r = [], 32
    while r < max_rows:
        rows.append(r)
        r *= 2
    if max_rows > SKINNY_MAX_ROWS:
        rows.append(int(max_rows))
    return rows


def linear_bf16(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, tiled=None) -> torch.Tensor:
    """``tiled`` is the weight's :class:`~.kernels.TiledWeight` when it has one."""
    if not (x.is_cuda and w.is_cuda and out.is_cuda):
        raise K.KernelError("linear_bf16: operands must be on the GPU")
    if x.shape[1] != w.shape[1] or out.shape != (x.shape[0], w.shape[0]):
        raise K.KernelError(f"linear_bf16: x {tuple(x.shape)} w {tuple(w.shape)} out "
                            f"{tuple(out.shape)} do not fit")
    if x.shape[0] == 0:
        return out
    if use_gemv(x.shape[0], w.shape[0], w.shape[1]) and w.is_contiguous() and x.stride(1) == 1:
        return K.gemv(x, w, out)
    if tiled is not None and use_skinny(x.shape[0], w.shape[0], w.shape[1]):
        return K.gemm_skinny(x, tiled, out)
    if K.gemm_vendor(x, w, out):
        return out
    # a shape the library's heuristic has nothing for: the framework's route to the same library
    if out.dtype == torch.bfloat16:
        torch.matmul(x, w.t(), out=out)
    else:
        tmp = torch.matmul(x, w.t())
        K.cast(tmp, out)
    return out
