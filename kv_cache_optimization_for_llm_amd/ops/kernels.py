"""Tensor-level entry points of the HIP kernels.

Each function checks on the host that shapes, dtypes, devices and layouts are what the kernel
and its grid assume, then launches on torch's current HIP stream.  There is no other code path:
a tensor that is not on the GPU, or a missing kernel library, is an error.
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from .library import KernelError, check, hip_lib

F32, BF16 = 0, 1
_DTYPE_CODE = {torch.float32: F32, torch.bfloat16: BF16}


def dtype_code(dt: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dt]
    except KeyError:
        raise KernelError(f"unsupported dtype {dt}; kernels take float32 and bfloat16") from None


_RAW_STREAM = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_RAW_DEVICE = getattr(torch._C, "_cuda_getDevice", None) or torch.cuda.current_device


def _stream() -> int:
    """Handle of torch's current stream on the current device (also while a graph is captured).
    The raw accessor costs a fraction of a microsecond; ``torch.cuda.current_stream()`` some ten,
    once per launch."""
    if _RAW_STREAM is not None:
        return _RAW_STREAM(_RAW_DEVICE())
    return torch.cuda.current_stream().cuda_stream


def _dev(t: torch.Tensor, name: str, dtype: Optional[torch.dtype] = None, contiguous: bool = True):
    if not isinstance(t, torch.Tensor):
        raise KernelError(f"{name}: expected a tensor, got {type(t).__name__}")
    if not t.is_cuda:
        raise KernelError(f"{name}: tensor is on {t.device}; the kernels run on the GPU only")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name}: dtype {t.dtype}, expected {dtype}")
    if contiguous and not t.is_contiguous():
        raise KernelError(f"{name}: tensor must be contiguous")
    return t.data_ptr()


def _opt(t: Optional[torch.Tensor], name: str, dtype: Optional[torch.dtype] = None):
    return None if t is None else _dev(t, name, dtype)


def k_chunk(head_dim: int) -> int:
    """Elements of a key that lie next to each other inside a K page (``csrc/kv_layout.h``)."""
    return 4 if head_dim % 8 else 8


def k_page_shape(num_kv_heads: int, head_dim: int) -> tuple:
    """Per-token shape of the K cache array: a key as ``head_dim / C`` chunks of ``C`` elements; the
    page's token axis lies between the two (``[kv_heads, head_dim / C, page_size, C]``)."""
    c = k_chunk(head_dim)
    return (num_kv_heads, head_dim // c, c)


def keys_to_pages(k: torch.Tensor) -> torch.Tensor:
    """Keys ``[..., page_size, head_dim]`` (row by row) in the cache's layout
    ``[..., head_dim / C, page_size, C]``."""
    *lead, page, d = k.shape
    c = k_chunk(d)
    return k.reshape(*lead, page, d // c, c).transpose(-3, -2).contiguous()


def pages_to_keys(k: torch.Tensor) -> torch.Tensor:
    """The inverse of :func:`keys_to_pages`: ``[..., head_dim / C, page_size, C]`` to ``[..., page_size, head_dim]``."""
    *lead, chunks, page, c = k.shape
    return k.transpose(-3, -2).reshape(*lead, page, chunks * c)


def check_cache_shapes(what: str, k_cache: torch.Tensor, v_cache: torch.Tensor, num_kv_heads: int,
                       head_dim: int) -> int:
    """K pages are [kv_heads, head_dim / C, page_size, C] (a key in chunks of C = 8 elements, the chunks
    of a page's keys next to each other: ``csrc/kv_layout.h``); V pages are transposed, [kv_heads,
    head_dim, page_size].  Returns the page size."""
    if k_cache.dim() != 5 or v_cache.dim() != 4:
        raise KernelError(f"{what}: the K cache must be 5-D and the V cache 4-D")
    pages, nkv, chunks, ps, c = k_cache.shape
    if (nkv, chunks, c) != k_page_shape(num_kv_heads, head_dim) or tuple(v_cache.shape) != (pages, nkv, head_dim, ps):
        raise KernelError(f"{what}: K cache {tuple(k_cache.shape)} / V cache {tuple(v_cache.shape)} are "
                          f"not [pages, {num_kv_heads}, {head_dim} / C, page, C] / [pages, {num_kv_heads}, "
                          f"{head_dim}, page] with C = {k_chunk(head_dim)}")
    return int(ps)


# --------------------------------------------------------------------------------------
def embed_gather(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor,
                 feedback: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[t, :] = table[ids[t], :], converted to out's dtype.  A negative id ``-1 - r`` stands
    for ``feedback[r]`` (a token still on the device); the caller guarantees ``r`` is inside
    ``feedback`` and that no id is negative when there is none.  An id outside the table (only
    what a kernel left in ``feedback`` can be: the host checks the ids it uploads) reads the
    nearest row of it."""
    rows, width = out.shape
    if table.dim() != 2 or table.shape[1] != width or ids.shape != (rows,):
        raise KernelError(f"embed_gather: shapes table {tuple(table.shape)} ids {tuple(ids.shape)} "
                          f"out {tuple(out.shape)} do not fit")
    check(hip_lib().kva_embed_gather(_dev(out, "out"), _dev(table, "table"),
                                     _dev(ids, "ids", torch.int32),
                                     _opt(feedback, "feedback", torch.int32), rows, width, table.shape[0],
                                     dtype_code(table.dtype), dtype_code(out.dtype), _stream()),
          "embed_gather")
    return out


def embed_gather_prep(table: torch.Tensor, ids: torch.Tensor, hidden: torch.Tensor, scaled: torch.Tensor,
                      sumsq: torch.Tensor, norm_weight: torch.Tensor,
                      feedback: Optional[torch.Tensor] = None) -> torch.Tensor:
    """:func:`embed_gather` for a bf16 table and stream that prepares the first norm in the same
    pass: ``scaled = round(hidden * norm_weight)`` and ``sumsq[t, 0] = sum(hidden[t]^2)``."""
    rows, width = hidden.shape
    if table.dim() != 2 or table.shape[1] != width or ids.shape != (rows,) or scaled.shape != (rows, width) \
            or sumsq.shape != (rows, 1) or norm_weight.shape != (width,):
        raise KernelError(f"embed_gather_prep: shapes table {tuple(table.shape)} ids {tuple(ids.shape)} hidden "
                          f"{tuple(hidden.shape)} scaled {tuple(scaled.shape)} sumsq {tuple(sumsq.shape)} do not fit")
    if not (table.dtype == hidden.dtype == scaled.dtype == torch.bfloat16) or width % 8 \
            or norm_weight.dtype not in (torch.bfloat16, torch.float32):
        raise KernelError("embed_gather_prep: bf16 table and outputs, a width that is a multiple of 8")
    check(hip_lib().kva_embed_gather_prep(
        _dev(hidden, "hidden"), _dev(scaled, "scaled"), _dev(sumsq, "sumsq", torch.float32), _dev(table, "table"),
        _dev(ids, "ids", torch.int32), _opt(feedback, "feedback", torch.int32), _dev(norm_weight, "norm_weight"),
        1 if norm_weight.dtype == torch.float32 else 0, rows, width, table.shape[0], _stream()), "embed_gather_prep")
    return hidden


class PartialSums:
    """A branch output that has not been added up yet: ``parts`` fp32 ``[ranges, rows, width]``, the
    products of :func:`gemm_skinny_partials` over ranges of K.  It stands where a bf16 ``[rows,
    width]`` delta stands; the norm kernel that adds the delta to the stream adds the ranges first
    (and rounds their sum to bf16, as the whole product would have been).  ``materialize()`` gives
    the plain delta."""

    def __init__(self, parts: torch.Tensor):
        if parts.dim() != 3 or parts.dtype != torch.float32:
            raise KernelError("PartialSums: fp32 [ranges, rows, width] needed")
        self.parts = parts

    @property
    def shape(self):
        return self.parts.shape[1:]

    @property
    def dtype(self):
        return torch.bfloat16

    @property
    def device(self):
        return self.parts.device

    def materialize(self) -> torch.Tensor:
        total = self.parts[0].clone()           # the ranges in order, by element-wise kernels only
        for r in range(1, self.parts.shape[0]):
            total += self.parts[r]
        return total.to(torch.bfloat16)


class AttentionPartials:
    """An attention output that has not been added up yet: what :func:`attention_mfma` leaves per
    key range when it is told to (``leave_partials``): ``part_o`` fp32 ``[tokens * heads, parts,
    head_dim]`` and ``part_ml`` fp32 ``[tokens * heads, parts, 2]`` (maximum in the base-2 domain,
    sum of exponentials).  It stands where the bf16 ``[tokens, heads * head_dim]`` output stands,
    for a consumer that adds the ranges up itself (:func:`gemv_merged`)."""

    def __init__(self, part_o: torch.Tensor, part_ml: torch.Tensor, tokens: int, heads: int):
        if part_o.dim() != 3 or part_o.dtype != torch.float32 or part_o.shape[0] != tokens * heads \
                or part_ml.shape != (tokens * heads, part_o.shape[1], 2) or part_ml.dtype != torch.float32:
            raise KernelError("AttentionPartials: fp32 [tokens * heads, parts, head_dim] and [tokens * heads, parts, 2] needed")
        self.part_o, self.part_ml, self.tokens, self.heads = part_o, part_ml, tokens, heads

    @property
    def parts(self) -> int:
        return self.part_o.shape[1]

    @property
    def head_dim(self) -> int:
        return self.part_o.shape[2]

    @property
    def shape(self):
        return (self.tokens, self.heads * self.head_dim)

    @property
    def dtype(self):
        return torch.bfloat16

    @property
    def device(self):
        return self.part_o.device


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor,
            delta=None, row_idx: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out = rmsnorm(x) * weight.  With ``delta`` (a tensor like x, or :class:`PartialSums`): x +=
    delta first (in place, fp32 add).  With ``row_idx``: out[i] = rmsnorm(x[row_idx[i]])."""
    width = x.shape[-1]
    out_rows = out.shape[0]
    if x.dim() != 2 or out.dim() != 2 or out.shape[1] != width or weight.shape != (width,):
        raise KernelError(f"rmsnorm: shapes x {tuple(x.shape)} weight {tuple(weight.shape)} out "
                          f"{tuple(out.shape)} do not fit")
    if out.dtype != x.dtype:
        raise KernelError("rmsnorm: out must have x's dtype")
    if row_idx is None:
        if out_rows != x.shape[0]:
            raise KernelError("rmsnorm: out needs as many rows as x")
    elif row_idx.shape != (out_rows,):
        raise KernelError("rmsnorm: one row index per output row")
    parts = None
    if isinstance(delta, PartialSums):
        if tuple(delta.shape) != tuple(x.shape) or x.dtype != torch.bfloat16 or width % 8:
            raise KernelError("rmsnorm: partial sums stand in for a bf16 delta of x's shape, width a multiple of 8")
        parts, delta = delta.parts, None
    if delta is not None and (delta.shape != x.shape or delta.dtype != x.dtype):
        raise KernelError("rmsnorm: delta must match x")
    check(hip_lib().kva_rmsnorm(_dev(out, "out"), _dev(x, "x"), _opt(delta, "delta"),
                                _dev(weight, "weight"), _opt(row_idx, "row_idx", torch.int32),
                                out_rows, width, float(eps), dtype_code(x.dtype),
                                dtype_code(weight.dtype), _opt(parts, "partial sums", torch.float32),
                                parts.shape[0] if parts is not None else 0,
                                parts.shape[1] if parts is not None else 0, _stream()), "rmsnorm")
    return out


def residual_add(hidden: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
    if hidden.shape != delta.shape or hidden.dtype != delta.dtype:
        raise KernelError("residual_add: operands must match")
    check(hip_lib().kva_residual_add(_dev(hidden, "hidden"), _dev(delta, "delta"), hidden.numel(),
                                     dtype_code(hidden.dtype), _stream()), "residual_add")
    return hidden


def stream_read(x: torch.Tensor, workgroups: int, sink: torch.Tensor) -> None:
    """A probe: reads ``x`` once and stores nothing (``sink``: any int32 device tensor, practically
    never written).  Its time is the floor of any kernel that reads as many bytes."""
    check(hip_lib().kva_stream_read(_dev(x, "x"), x.numel() * x.element_size(), int(workgroups),
                                    _dev(sink, "sink", torch.int32), _stream()), "stream_read")


def stream_reread(x: torch.Tensor, workgroups: int, repeats: int, sink: torch.Tensor) -> None:
    """A probe: every one of ``workgroups`` workgroups reads all of ``x``, ``repeats`` times over,
    through the caches.  With an ``x`` that fits a die's L2: what a compute unit takes in from there."""
    check(hip_lib().kva_stream_reread(_dev(x, "x"), x.numel() * x.element_size(), int(workgroups), int(repeats),
                                      _dev(sink, "sink", torch.int32), _stream()), "stream_reread")


def stream_mixed(own: Optional[torch.Tensor], shared: Optional[torch.Tensor], workgroups: int,
                 sink: torch.Tensor) -> None:
    """A probe: half of each workgroup's wavefronts stream the workgroup's own 1/``workgroups`` of
    ``own`` from memory while the other half read all of ``shared`` (from L2); either may be None."""
    if int(workgroups) < 1:
        raise KernelError("stream_mixed: at least one workgroup")
    own_bytes = 0 if own is None else own.numel() * own.element_size() // int(workgroups) // 16 * 16
    shared_bytes = 0 if shared is None else shared.numel() * shared.element_size() // 16 * 16
    check(hip_lib().kva_stream_mixed(None if own is None else _dev(own, "own"), own_bytes,
                                     None if shared is None else _dev(shared, "shared"), shared_bytes,
                                     int(workgroups), _dev(sink, "sink", torch.int32), _stream()), "stream_mixed")


def probe_read_bandwidth(device, megabytes: int = 2048, workgroups: int = 2048, reps: int = 5) -> float:
    """GB/s of a plain read stream over a buffer far larger than every cache, best of ``reps``."""
    x = torch.empty(megabytes << 20, dtype=torch.uint8, device=device)
    x.zero_()
    sink = torch.zeros(4, dtype=torch.int32, device=device)
    stream_read(x, workgroups, sink)
    best = 0.0
    for _ in range(reps):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        stream_read(x, workgroups, sink)
        b.record()
        b.synchronize()
        best = max(best, x.numel() / (a.elapsed_time(b) * 1e-3) / 1e9)
    return best


def scale_softcap(x: torch.Tensor, scale: float, cap: float = 0.0) -> torch.Tensor:
    """In place: ``x *= scale``, then with ``cap > 0`` ``x = cap * tanh(x / cap)``."""
    if cap < 0:
        raise KernelError("scale_softcap: the cap must not be negative")
    check(hip_lib().kva_scale_softcap(_dev(x, "x"), x.numel(), float(scale), float(cap), dtype_code(x.dtype),
                                      _stream()), "scale_softcap")
    return x


def silu_mul(gate_up: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[t, i] = silu(gate_up[t, i]) * gate_up[t, I + i]."""
    rows, inter = out.shape
    if gate_up.shape != (rows, 2 * inter) or gate_up.dtype != out.dtype:
        raise KernelError(f"silu_mul: gate_up {tuple(gate_up.shape)} does not fit out {tuple(out.shape)}")
    check(hip_lib().kva_silu_mul(_dev(out, "out"), _dev(gate_up, "gate_up"), rows, inter,
                                 dtype_code(out.dtype), _stream()), "silu_mul")
    return out


def cast(src: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    if src.shape != out.shape:
        raise KernelError("cast: shapes differ")
    if src.dtype == out.dtype:
        raise KernelError("cast: same dtype on both sides")
    check(hip_lib().kva_cast(_dev(out, "out"), _dev(src, "src"), src.numel(), dtype_code(src.dtype),
                             dtype_code(out.dtype), _stream()), "cast")
    return out


def rope_kv_write(qkv: torch.Tensor, positions: torch.Tensor, num_q_heads: int, num_kv_heads: int,
                  head_dim: int, cos: Optional[torch.Tensor], sin: Optional[torch.Tensor],
                  k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                  slot_mapping: Optional[torch.Tensor], page_size: int) -> None:
    """Rotates the Q and K heads of ``qkv`` [T, (nq + 2 nkv) d] by the tokens' positions; Q in
    place, rotated K and plain V into the cache [pages, nkv, page_size, d] at ``slot_mapping``."""
    tokens = qkv.shape[0]
    if qkv.dim() != 2 or qkv.shape[1] != (num_q_heads + 2 * num_kv_heads) * head_dim:
        raise KernelError(f"rope_kv_write: qkv {tuple(qkv.shape)} is not [T, (nq + 2 nkv) * d]")
    if positions.shape != (tokens,):
        raise KernelError("rope_kv_write: one position per token")
    rot = 0
    if cos is not None:
        if sin is None or cos.shape != sin.shape or cos.dim() != 2:
            raise KernelError("rope_kv_write: cos and sin tables must be [positions, rot/2]")
        rot = 2 * cos.shape[1]
    write = k_cache is not None
    if write:
        if v_cache is None or slot_mapping is None:
            raise KernelError("rope_kv_write: K and V cache and a slot mapping are all needed")
        check_cache_shapes("rope_kv_write", k_cache, v_cache, num_kv_heads, head_dim)
        if k_cache.shape[3] != page_size:
            raise KernelError(f"rope_kv_write: cache pages hold {k_cache.shape[3]} tokens, not {page_size}")
        if k_cache.dtype != qkv.dtype or slot_mapping.shape != (tokens,):
            raise KernelError("rope_kv_write: cache dtype or slot mapping shape does not fit")
    check(hip_lib().kva_rope_kv_write(
        _dev(qkv, "qkv"), _opt(k_cache, "k_cache"), _opt(v_cache, "v_cache"),
        _opt(cos, "cos", torch.float32), _opt(sin, "sin", torch.float32),
        _dev(positions, "positions", torch.int32), _opt(slot_mapping, "slot_mapping", torch.int32),
        tokens, num_q_heads, num_kv_heads, head_dim, rot, page_size, 1 if write else 0,
        dtype_code(qkv.dtype), _stream()), "rope_kv_write")


def attention_rowwise(q: torch.Tensor, q_row_stride: int, out: torch.Tensor, k_cache: torch.Tensor,
                      v_cache: torch.Tensor, block_table: torch.Tensor, tok_seat: torch.Tensor,
                      tok_pos: torch.Tensor, num_q_heads: int, num_kv_heads: int, head_dim: int,
                      scale: float, window: int = 0) -> torch.Tensor:
    """Causal GQA attention of every token over its request's cached keys; ``q`` is a view whose
    rows are ``q_row_stride`` elements apart (the Q part of a fused QKV buffer)."""
    tokens = out.shape[0]
    if out.shape != (tokens, num_q_heads * head_dim):
        raise KernelError("attention: out must be [T, nq * d]")
    check_cache_shapes("attention", k_cache, v_cache, num_kv_heads, head_dim)
    if block_table.dim() != 2 or tok_seat.shape != (tokens,) or tok_pos.shape != (tokens,):
        raise KernelError("attention: block table [seats, blocks], one seat and position per token")
    if q.dtype != out.dtype or k_cache.dtype != out.dtype:
        raise KernelError("attention: q, cache and out must share a dtype")
    if q.data_ptr() % 16 or q_row_stride < num_q_heads * head_dim:
        raise KernelError("attention: q view is misaligned or its stride is too small")
    page_size = k_cache.shape[3]
    check(hip_lib().kva_attention_rowwise(
        _dev(out, "out"), _dev(q, "q", contiguous=False), q_row_stride, _dev(k_cache, "k_cache"),
        _dev(v_cache, "v_cache"), _dev(block_table, "block_table", torch.int32), block_table.shape[1],
        _dev(tok_seat, "tok_seat", torch.int32), _dev(tok_pos, "tok_pos", torch.int32), tokens,
        num_q_heads, num_kv_heads, head_dim, page_size, float(scale), int(window),
        dtype_code(out.dtype), _stream()), "attention_rowwise")
    return out


def gemm_nt_f32(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[M, N] = a[M, K] @ w[N, K]^T in true fp32."""
    m, k = a.shape
    n = w.shape[0]
    if w.shape != (n, k) or out.shape != (m, n):
        raise KernelError(f"gemm_f32: a {tuple(a.shape)} w {tuple(w.shape)} out {tuple(out.shape)} do not fit")
    check(hip_lib().kva_gemm_nt_f32(_dev(out, "out", torch.float32), _dev(a, "a", torch.float32),
                                    _dev(w, "w", torch.float32), m, n, k, k, k, n, _stream()),
          "gemm_nt_f32")
    return out


def host_memory_is_mapped(t: torch.Tensor) -> bool:
    """Whether a kernel may write into this host tensor (pinned memory mapped for the device)."""
    if t.is_cuda or not t.is_pinned():
        return False
    return bool(hip_lib().kva_host_memory_is_mapped(ctypes.c_void_p(t.data_ptr())))


def sample(logits: torch.Tensor, out_tokens: torch.Tensor, *, chunks: int = 128,
           inv_temperature: Optional[torch.Tensor] = None, seed: int = 0,
           rng_key: Optional[torch.Tensor] = None, rng_step: Optional[torch.Tensor] = None,
           penalty_mask: Optional[torch.Tensor] = None, row_seat: Optional[torch.Tensor] = None,
           penalty: float = 1.0, mark_mask: Optional[torch.Tensor] = None,
           mark_seat: Optional[torch.Tensor] = None, host_tokens: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Greedy (rows whose inv_temperature is 0 or absent) or temperature sampling per row.
    ``penalty_mask`` ``[seats, vocab]`` with ``row_seat`` (-1: none) names the logits that are
    penalised; ``mark_mask`` with ``mark_seat`` (-1: none) gets ``mark_mask[seat, token] = 1`` for
    every chosen token, in the same launch.  ``host_tokens``: a pinned host int32 tensor with a
    place per row that takes the tokens too, written by the kernel itself (valid once the stream
    has passed the launch)."""
    rows, vocab = logits.shape
    if out_tokens.shape != (rows,):
        raise KernelError("sample: one output token per row")
    any_sampled = inv_temperature is not None
    if any_sampled and (rng_key is None or rng_step is None or inv_temperature.shape != (rows,)
                        or rng_key.shape != (rows,) or rng_step.shape != (rows,)):
        raise KernelError("sample: inv_temperature, rng_key and rng_step are needed per row")
    if penalty_mask is not None:
        if row_seat is None or row_seat.shape != (rows,) or penalty_mask.dim() != 2 \
                or penalty_mask.shape[1] != vocab:
            raise KernelError("sample: penalty mask [seats, vocab] needs a seat per row")
    if (mark_mask is None) != (mark_seat is None) or (mark_mask is not None and (
            mark_seat.shape != (rows,) or mark_mask.dim() != 2 or mark_mask.shape[1] != vocab)):
        raise KernelError("sample: marking needs a mask [seats, vocab] and a seat per row")
    if host_tokens is not None and (host_tokens.is_cuda or not host_tokens.is_pinned() or host_tokens.dtype != torch.int32
                                    or host_tokens.dim() != 1 or host_tokens.shape[0] < rows
                                    or not host_tokens.is_contiguous()):
        raise KernelError("sample: host_tokens must be a pinned host int32 vector with a place per row")
    lib = hip_lib()
    ws = torch.empty(max(1, lib.kva_sample_workspace_bytes(rows, chunks) // 4), dtype=torch.float32,
                     device=logits.device)
    check(lib.kva_sample(
        _dev(out_tokens, "out_tokens", torch.int32), _dev(logits, "logits", torch.float32), rows, vocab,
        chunks, _opt(penalty_mask, "penalty_mask", torch.uint8), _opt(row_seat, "row_seat", torch.int32),
        float(penalty), _opt(inv_temperature, "inv_temperature", torch.float32), int(seed) & 0xFFFFFFFF,
        _opt(rng_key, "rng_key", torch.int32), _opt(rng_step, "rng_step", torch.int32),
        1 if any_sampled else 0, _dev(ws, "workspace"), _opt(mark_mask, "mark_mask", torch.uint8),
        _opt(mark_seat, "mark_seat", torch.int32),
        ctypes.c_void_p(host_tokens.data_ptr()) if host_tokens is not None else None, _stream()), "sample")
    return out_tokens


def mark_tokens(mask: torch.Tensor, seats: torch.Tensor, tokens: torch.Tensor) -> None:
    n = seats.shape[0]
    if tokens.shape != (n,) or mask.dim() != 2:
        raise KernelError("mark_tokens: one seat per token, mask [seats, vocab]")
    check(hip_lib().kva_mark_tokens(_dev(mask, "mask", torch.uint8), _dev(seats, "seats", torch.int32),
                                    _dev(tokens, "tokens", torch.int32), n, mask.shape[1], _stream()),
          "mark_tokens")


_MAX_SPLITS = None


def attention_max_splits() -> int:
    """Most key splits the matrix-core attention kernels and their merge take."""
    global _MAX_SPLITS
    if _MAX_SPLITS is None:
        _MAX_SPLITS = int(hip_lib().kva_attention_max_splits())
    return _MAX_SPLITS


def attention_mfma_supported(head_dim: int, page_size: int) -> bool:
    return bool(hip_lib().kva_attention_mfma_supported(int(head_dim), int(page_size)))


def attention_mfma_row_tiles(head_dim: int, wide: bool) -> int:
    """Row tiles (of 16 query rows) per work item the kernel offers for this head size."""
    return int(hip_lib().kva_attention_mfma_row_tiles(int(head_dim), 1 if wide else 0))


def attention_mfma(q: torch.Tensor, q_row_stride: int, out: torch.Tensor, k_cache: torch.Tensor,
                   v_cache: torch.Tensor, block_table: torch.Tensor, item_entry: torch.Tensor,
                   item_row0: torch.Tensor, entry_seat: torch.Tensor, entry_q_start: torch.Tensor,
                   entry_start_pos: torch.Tensor, num_q_heads: int, num_kv_heads: int, head_dim: int,
                   scale: float, window: int = 0, splits: int = 1, keys_per_split: int = 0,
                   row_tiles: int = 1, pair: bool = False,
                   item_meta: Optional[torch.Tensor] = None, covers_all_rows: bool = True,
                   keep_cached: bool = False, waves: int = 1, leave_partials: bool = False):
    """bf16 matrix-core attention over the paged cache.  Items are (entry, first query row) pairs
    of ``16 * row_tiles`` query rows each, row = token_in_step * (nq / nkv) + head_in_group.
    With ``pair`` one wavefront takes item i and item n-1-i of the list (give the list ordered by
    keys visited, most first, and every wavefront has about the same work).  ``item_meta``
    ``[items, 8]`` int32 (q_start, q_len, start_pos, seat, row0, 0, 0, 0 per item) saves the
    kernel the chain of lookups item -> entry -> entry arrays; it must say the same as they do.
    ``covers_all_rows=False``: the items are only some of the step's rows (the others belong to
    another launch) and a split merge must leave those alone.  ``keep_cached`` (items of one row
    tile): keys and values are loaded through the caches instead of past them - for the few
    short contexts that are still in the memory-side cache when the next step reads them.
    ``waves`` (1, 2 or 4; items of one row tile, head sizes up to 128): so many of the ``splits``
    key ranges go to the wavefronts of one workgroup, which adds their results up itself; only
    ``splits // waves`` partial results per row are left for the merge (none: no merge launch).
    ``leave_partials`` (the items cover every row of the step): where more than one partial result
    a row is left they are not merged into ``out`` but returned as :class:`AttentionPartials`."""
    tokens = out.shape[0]
    if out.dtype != torch.bfloat16 or q.dtype != torch.bfloat16 or k_cache.dtype != torch.bfloat16:
        raise KernelError("attention_mfma: bfloat16 only")
    if leave_partials and not covers_all_rows:
        raise KernelError("attention_mfma: partial results can only be left for a launch that covers every row")
    if waves < 1 or splits % waves:
        raise KernelError(f"attention_mfma: {waves} wavefronts per item do not divide {splits} key ranges")
    if out.shape != (tokens, num_q_heads * head_dim):
        raise KernelError("attention_mfma: out must be [T, nq * d]")
    check_cache_shapes("attention_mfma", k_cache, v_cache, num_kv_heads, head_dim)
    n_items = item_entry.shape[0]
    n_entries = entry_seat.shape[0]
    if item_row0.shape != (n_items,) or entry_q_start.shape != (n_entries + 1,) \
            or entry_start_pos.shape != (n_entries,) or block_table.dim() != 2:
        raise KernelError("attention_mfma: index arrays do not fit each other")
    if q.data_ptr() % 16 or q_row_stride < num_q_heads * head_dim:
        raise KernelError("attention_mfma: q view is misaligned or its stride is too small")
    if item_meta is not None and item_meta.shape != (n_items, 8):
        raise KernelError("attention_mfma: item_meta must be [items, 8]")
    part_o = part_ml = None
    if splits // waves > 1:
        part_o = torch.empty((tokens * num_q_heads, splits // waves, head_dim), dtype=torch.float32, device=out.device)
        part_ml = torch.empty((tokens * num_q_heads, splits // waves, 2), dtype=torch.float32, device=out.device)
    left = leave_partials and part_o is not None
    check(hip_lib().kva_attention_mfma(
        None if left else _dev(out, "out"), _opt(part_o, "part_o"), _opt(part_ml, "part_ml"),
        _dev(q, "q", contiguous=False), q_row_stride, _dev(k_cache, "k_cache"), _dev(v_cache, "v_cache"),
        _dev(block_table, "block_table", torch.int32), block_table.shape[1],
        _opt(item_meta, "item_meta", torch.int32),
        _dev(item_entry, "item_entry", torch.int32), _dev(item_row0, "item_row0", torch.int32), n_items,
        int(row_tiles), _dev(entry_seat, "entry_seat", torch.int32), _dev(entry_q_start, "entry_q_start", torch.int32),
        _dev(entry_start_pos, "entry_start_pos", torch.int32), tokens * num_q_heads, num_q_heads,
        num_kv_heads, head_dim, k_cache.shape[3], float(scale), int(window), int(splits),
        int(keys_per_split), 1 if pair else 0, 1 if covers_all_rows else 0, 1 if keep_cached else 0,
        int(waves), _stream()), "attention_mfma")
    return AttentionPartials(part_o, part_ml, tokens, num_q_heads) if left else out


def attention_mfma_rope_supported(head_dim: int, page_size: int, group: int) -> bool:
    """Whether the decode attention kernel that rotates and caches inside takes this geometry
    (``group``: query heads per kv head)."""
    return bool(hip_lib().kva_attention_mfma_rope_supported(int(head_dim), int(page_size), int(group)))


def attention_mfma_rope(qkv: torch.Tensor, out: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                        block_table: torch.Tensor, item_meta: torch.Tensor, num_q_heads: int, num_kv_heads: int,
                        head_dim: int, scale: float, cos: Optional[torch.Tensor], sin: Optional[torch.Tensor],
                        slot_mapping: Optional[torch.Tensor], window: int = 0, splits: int = 1,
                        keys_per_split: int = 0, keep_cached: bool = False, waves: int = 1) -> torch.Tensor:
    """bf16 matrix-core attention of decoded tokens (one token per item) straight from the joined
    Q/K/V projection ``qkv`` ``[T, (nq + 2 nkv) d]``, not yet rotated: the kernel rotates Q and the
    token's K by its position (``cos`` / ``sin`` ``[positions, d / 2]`` fp32, both None: no
    rotation), stores the rotated K and the V at ``slot_mapping[token]`` (None: the cache is only
    read) and attends, the token's own key and value taken from registers.  ``item_meta``
    ``[items, 8]`` int32: (token row, 1, position, seat, 0, 0, 0, 0).  ``waves``: as for
    :func:`attention_mfma`."""
    tokens = out.shape[0]
    if out.dtype != torch.bfloat16 or qkv.dtype != torch.bfloat16 or k_cache.dtype != torch.bfloat16:
        raise KernelError("attention_mfma_rope: bfloat16 only")
    if waves < 1 or splits % waves:
        raise KernelError(f"attention_mfma_rope: {waves} wavefronts per item do not divide {splits} key ranges")
    if out.shape != (tokens, num_q_heads * head_dim) or qkv.dim() != 2 or qkv.shape[0] != tokens \
            or qkv.shape[1] != (num_q_heads + 2 * num_kv_heads) * head_dim or not qkv.is_contiguous():
        raise KernelError("attention_mfma_rope: qkv must be [T, (nq + 2 nkv) d] and out [T, nq * d]")
    check_cache_shapes("attention_mfma_rope", k_cache, v_cache, num_kv_heads, head_dim)
    if item_meta.dim() != 2 or item_meta.shape[1] != 8 or block_table.dim() != 2:
        raise KernelError("attention_mfma_rope: item_meta must be [items, 8] and the block table [seats, blocks]")
    if (cos is None) != (sin is None) or (cos is not None and (cos.shape != sin.shape or cos.dim() != 2
                                                               or cos.shape[1] != head_dim // 2)):
        raise KernelError("attention_mfma_rope: cos and sin tables must both be [positions, d / 2]")
    if slot_mapping is not None and slot_mapping.shape != (tokens,):
        raise KernelError("attention_mfma_rope: one cache slot per token")
    part_o = part_ml = None
    if splits // waves > 1:
        part_o = torch.empty((tokens * num_q_heads, splits // waves, head_dim), dtype=torch.float32, device=out.device)
        part_ml = torch.empty((tokens * num_q_heads, splits // waves, 2), dtype=torch.float32, device=out.device)
    check(hip_lib().kva_attention_mfma_rope(
        _dev(out, "out"), _opt(part_o, "part_o"), _opt(part_ml, "part_ml"), _dev(qkv, "qkv"), qkv.shape[1],
        _dev(k_cache, "k_cache"), _dev(v_cache, "v_cache"), _dev(block_table, "block_table", torch.int32),
        block_table.shape[1], _dev(item_meta, "item_meta", torch.int32), item_meta.shape[0], tokens * num_q_heads,
        num_q_heads, num_kv_heads, head_dim, k_cache.shape[3], float(scale), int(window), int(splits),
        int(keys_per_split), 1 if keep_cached else 0, _opt(cos, "cos", torch.float32), _opt(sin, "sin", torch.float32),
        _opt(slot_mapping, "slot_mapping", torch.int32), int(waves), _stream()), "attention_mfma_rope")
    return out


def attention_lds_supported(head_dim: int, page_size: int) -> bool:
    return bool(hip_lib().kva_attention_lds_supported(int(head_dim), int(page_size)))


def attention_lds(q: torch.Tensor, q_row_stride: int, out: torch.Tensor, k_cache: torch.Tensor,
                  v_cache: torch.Tensor, block_table: torch.Tensor, item_meta: torch.Tensor,
                  num_q_heads: int, num_kv_heads: int, head_dim: int, scale: float, window: int = 0,
                  pair: bool = False, splits: int = 1, keys_per_split: int = 0,
                  covers_all_rows: bool = True) -> torch.Tensor:
    """bf16 matrix-core attention for prompt portions: a workgroup of four wavefronts per 128
    query rows (row = token_in_step * (nq / nkv) + head_in_group) shares every key and value
    block through LDS.  ``item_meta`` ``[items, 8]`` int32: (q_start, q_len, start_pos, seat,
    row0, 0, 0, 0) with ``row0`` a multiple of 128.  With ``pair`` a workgroup takes item i and
    item n-1-i of the list.  With ``splits`` > 1 the keys are cut into ranges of
    ``keys_per_split`` (a multiple of 32), one workgroup each, and merged afterwards
    (``covers_all_rows=False``: only over the items' rows, the others belong to another launch)."""
    tokens = out.shape[0]
    if out.dtype != torch.bfloat16 or q.dtype != torch.bfloat16 or k_cache.dtype != torch.bfloat16:
        raise KernelError("attention_lds: bfloat16 only")
    if out.shape != (tokens, num_q_heads * head_dim):
        raise KernelError("attention_lds: out must be [T, nq * d]")
    check_cache_shapes("attention_lds", k_cache, v_cache, num_kv_heads, head_dim)
    if item_meta.dim() != 2 or item_meta.shape[1] != 8 or block_table.dim() != 2:
        raise KernelError("attention_lds: item_meta must be [items, 8] and the block table [seats, blocks]")
    if q.data_ptr() % 16 or q_row_stride < num_q_heads * head_dim:
        raise KernelError("attention_lds: q view is misaligned or its stride is too small")
    part_o = part_ml = None
    if splits > 1:
        part_o = torch.empty((tokens * num_q_heads, splits, head_dim), dtype=torch.float32, device=out.device)
        part_ml = torch.empty((tokens * num_q_heads, splits, 2), dtype=torch.float32, device=out.device)
    check(hip_lib().kva_attention_lds(
        _dev(out, "out"), _opt(part_o, "part_o"), _opt(part_ml, "part_ml"),
        _dev(q, "q", contiguous=False), q_row_stride, _dev(k_cache, "k_cache"),
        _dev(v_cache, "v_cache"), _dev(block_table, "block_table", torch.int32), block_table.shape[1],
        _dev(item_meta, "item_meta", torch.int32), item_meta.shape[0], 1 if pair else 0, num_q_heads,
        num_kv_heads, head_dim, k_cache.shape[3], float(scale), int(window), int(splits), int(keys_per_split),
        tokens * num_q_heads, 1 if covers_all_rows else 0, _stream()), "attention_lds")
    return out


def gemm_vendor_init() -> None:
    """Makes the vendor GEMM library's handle and workspace on the current device; called when a
    weight is loaded, so that no product makes them in the middle of a graph capture."""
    check(hip_lib().kva_gemm_vendor_init(), "gemm_vendor_init")


def gemm_vendor(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> bool:
    """out = x @ w^T by the vendor GEMM library (bf16 operands, fp32 accumulation, bf16 or fp32
    result).  False when the library has no algorithm for the shape: nothing was launched."""
    m, k = x.shape
    n = w.shape[0]
    if w.shape[1] != k or out.shape != (m, n) or x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 \
            or out.dtype not in (torch.bfloat16, torch.float32):
        raise KernelError(f"gemm_vendor: x {tuple(x.shape)} {x.dtype}, w {tuple(w.shape)} {w.dtype}, out "
                          f"{tuple(out.shape)} {out.dtype} do not fit")
    code = hip_lib().kva_gemm_vendor(_dev(out, "out"), _dev(x, "x"), _dev(w, "w"), m, n, k, k, n,
                                     1 if out.dtype == torch.float32 else 0, _stream())
    if code == 1:
        return False
    check(code, "gemm_vendor")
    return True


def gemm_vendor_tune(rows: int, weights, out_dtype: torch.dtype = torch.bfloat16) -> tuple:
    """Finds the vendor library's fastest algorithm for products of ``rows`` rows with weights of
    the shape of ``weights`` (bf16 matrices of one shape, e.g. the same projection of every
    layer; they are used in turn so that each comes from memory) and keeps it for later
    :func:`gemm_vendor` calls of that shape.  Runs every algorithm the library has for the shape:
    seconds, at start-up, never inside a graph capture.  A winner whose product differs from the
    heuristic's choice by more than rounding is dropped again.  Returns (microseconds of the
    heuristic's choice, microseconds of the one kept, algorithms run)."""
    import ctypes
    weights = list(weights)
    if not weights or rows < 1:
        raise KernelError("gemm_vendor_tune: needs at least one weight and one row")
    n, k = weights[0].shape
    for w in weights:
        if w.shape != (n, k) or w.dtype != torch.bfloat16 or not w.is_cuda or not w.is_contiguous():
            raise KernelError("gemm_vendor_tune: weights must be contiguous bf16 matrices of one shape on the GPU")
    dev = weights[0].device
    x = (torch.randn((rows, k), device=dev, dtype=torch.float32) * 0.5).to(torch.bfloat16)
    out = torch.empty((rows, n), dtype=out_dtype, device=dev)
    if not gemm_vendor(x, weights[0], out):
        return (-1.0, -1.0, 0)
    before = out.float()
    ptrs = (ctypes.c_void_p * len(weights))(*[w.data_ptr() for w in weights])
    first, best, tried = ctypes.c_float(), ctypes.c_float(), ctypes.c_int()
    check(hip_lib().kva_gemm_vendor_tune(_dev(out, "out"), _dev(x, "x"), ptrs, len(weights), rows, n, k, k, n,
                                         1 if out_dtype == torch.float32 else 0, _stream(),
                                         ctypes.byref(first), ctypes.byref(best), ctypes.byref(tried)),
          "gemm_vendor_tune")
    gemm_vendor(x, weights[0], out)
    scale = float(before.abs().max())
    if not float((out.float() - before).abs().max()) <= 0.02 * scale:
        check(hip_lib().kva_gemm_vendor_forget(rows, n, k, k, n, 1 if out_dtype == torch.float32 else 0),
              "gemm_vendor_forget")
        return (first.value, first.value, tried.value)
    return (first.value, best.value, tried.value)


def gemm_skinny_supported(m: int, n: int, k: int) -> bool:
    return bool(hip_lib().kva_gemm_skinny_supported(int(m), int(n), int(k)))


class TiledWeight:
    """A bf16 ``[N, K]`` weight re-laid for the few-rows product: ``[n-tile][K/32][4][16][8]``
    (tile of 16 rows, step of 32 of K, quarter of the step, row, 8 of K), rows padded with zeros
    to a multiple of 16, so that the 1 KiB a wavefront needs per step is contiguous and in the
    order of its lanes.  With ``halves=2`` (a joined ``[gate; up]`` matrix) each half is tiled on its own
    and the gate tiles come first."""

    def __init__(self, weight: torch.Tensor, halves: int = 1):
        n, k = weight.shape
        if weight.dtype != torch.bfloat16 or k % 32 or n % halves:
            raise KernelError(f"TiledWeight: bf16 [N, K] with K % 32 == 0 needed, got {tuple(weight.shape)} {weight.dtype}")
        self.n, self.k, self.halves = n, k, halves
        parts = []
        for h in weight.view(halves, n // halves, k):
            rows = h.shape[0]
            pad = (-rows) % 16
            if pad:
                h = torch.cat([h, torch.zeros((pad, k), dtype=h.dtype, device=h.device)])
            # [tile][row 16][step][g 4][8] -> [tile][step][g][row][8]: the 16 bytes of lane r + 16 g
            # of a wavefront lie at byte 16 (r + 16 g) of the step's 1 KiB, so neighbouring lanes
            # read neighbouring memory (four lanes per 64-byte access instead of one)
            parts.append(h.view((rows + pad) // 16, 16, k // 32, 4, 8).permute(0, 2, 3, 1, 4).contiguous())
        self.data = torch.cat(parts).contiguous()


class TiledRows:
    """At most 64 rows of ``width`` bf16 columns laid out ``[width / 8, R, 8]`` with ``R`` the row
    count rounded up to a multiple of 16, or 8 for up to 8 rows (the library says which:
    ``kva_tiled_rows``): element (m, c) at ``[c // 8, m, c % 8]``, rows past ``rows`` unwritten.  It is the order in which the lanes of a few-rows product read X (sixteen
    neighbouring lanes take the same 8 columns of sixteen neighbouring rows: 256 contiguous bytes
    instead of sixteen pieces a row apart), so a product that feeds another can leave its result
    like this.  ``to_rows()`` gives the plain ``[rows, width]``."""

    MAX_ROWS = 64

    def __init__(self, rows: int, width: int, device):
        if not (1 <= rows <= self.MAX_ROWS) or width % 8:
            raise KernelError(f"TiledRows: 1..{self.MAX_ROWS} rows and a multiple of 8 columns, not {rows} x {width}")
        self.rows, self.width = rows, width
        self.padded = int(hip_lib().kva_tiled_rows(int(rows)))
        self.data = torch.empty((width // 8, self.padded, 8), dtype=torch.bfloat16, device=device)

    @classmethod
    def from_rows(cls, x: torch.Tensor) -> "TiledRows":
        t = cls(x.shape[0], x.shape[1], x.device)
        t.data[:, :t.rows, :] = x.view(t.rows, t.width // 8, 8).permute(1, 0, 2)
        return t

    @property
    def shape(self):
        return (self.rows, self.width)

    @property
    def dtype(self):
        return self.data.dtype

    @property
    def device(self):
        return self.data.device

    def to_rows(self) -> torch.Tensor:
        return self.data.permute(1, 0, 2).reshape(self.padded, self.width)[:self.rows].contiguous()


def gemm_skinny(x: torch.Tensor, w: TiledWeight, out: Optional[torch.Tensor], swiglu: bool = False, *,
                sumsq: Optional[torch.Tensor] = None, norm_width: int = 0, eps: float = 0.0,
                hidden: Optional[torch.Tensor] = None, next_weight: Optional[torch.Tensor] = None,
                scaled_out: Optional[torch.Tensor] = None, sumsq_out: Optional[torch.Tensor] = None,
                x_tiled: bool = False, out_tiled: bool = False):
    """out = x @ W^T for at most 64 rows of x (bf16 operands, fp32 accumulation); ``w`` is the
    :class:`TiledWeight` of W.

    * ``out`` bf16 or fp32 ``[M, N]``; with ``swiglu`` the weight is a joined ``[gate; up]``
      matrix (tiled with ``halves=2``) and ``out`` is bf16 ``[M, N / 2]`` = silu(x gate^T) * (x up^T).
    * ``sumsq`` ``[M, parts]`` fp32: the rows of ``x`` are un-normalised norm inputs
      (``round(h * w_norm)``) and the product is scaled per token by
      ``rsqrt(sum(sumsq[m]) / norm_width + eps)``.
    * ``hidden`` (instead of ``out``): ``hidden += x @ W^T`` in place (fp32 add, rounded), plus
      ``scaled_out = round(hidden * next_weight)`` and ``sumsq_out[M, ceil(N / 16)]``.
    * ``out_tiled`` (gated product): ``out`` is ``[N / 2 / 8, R, 8]`` (``R``: see :class:`TiledRows`), element
      (m, c) at ``[c // 8, m, c % 8]`` - the order in which the lanes of a following few-rows
      product read it (a :class:`TiledRows`); such a result is given to that product as ``x``
      with ``x_tiled``."""
    if not isinstance(w, TiledWeight):
        raise KernelError("gemm_skinny: the weight must be a TiledWeight")
    if x_tiled:
        if not isinstance(x, TiledRows):
            raise KernelError("gemm_skinny: x_tiled needs a TiledRows")
        m, k, x = x.rows, x.width, x.data
    else:
        m, k = x.shape
    n = w.n
    if x.dtype != torch.bfloat16 or k != w.k or (swiglu != (w.halves == 2)):
        raise KernelError(f"gemm_skinny: bf16 x {tuple(x.shape)} does not fit weight [{w.n}, {w.k}] "
                          f"(halves {w.halves})")
    lib = hip_lib()
    if sumsq is not None and (sumsq.dim() != 2 or sumsq.shape[0] != m or norm_width <= 0):
        raise KernelError("gemm_skinny: sumsq must be [M, parts] and norm_width positive")
    parts = sumsq.shape[1] if sumsq is not None else 0
    if hidden is not None:
        if swiglu or out is not None:
            raise KernelError("gemm_skinny: the residual epilogue has no other output")
        p_out = lib.kva_gemm_skinny_sumsq_parts(n)
        if hidden.shape != (m, n) or hidden.dtype != torch.bfloat16 or scaled_out is None \
                or scaled_out.shape != (m, n) or scaled_out.dtype != torch.bfloat16 \
                or sumsq_out is None or sumsq_out.shape != (m, p_out):
            raise KernelError("gemm_skinny: hidden / scaled_out [M, N] bf16 and sumsq_out [M, ceil(N/16)] needed")
        if next_weight is not None and next_weight.shape != (n,):
            raise KernelError("gemm_skinny: the next norm's weight must be [N]")
        check(lib.kva_gemm_skinny(
            None, _dev(x, "x"), _dev(w.data, "w"), m, n, k, k, n, 3, _opt(sumsq, "sumsq", torch.float32), parts,
            int(norm_width), float(eps), _dev(hidden, "hidden"), _opt(next_weight, "next_weight"),
            1 if next_weight is not None and next_weight.dtype == torch.float32 else 0,
            _dev(scaled_out, "scaled_out"), _dev(sumsq_out, "sumsq_out", torch.float32),
            1 if x_tiled else 0, 0, _stream()),
            "gemm_skinny")
        return hidden
    cols = n // 2 if swiglu else n
    out_t = out
    if out_tiled:
        if not (isinstance(out, TiledRows) and swiglu and out.rows == m and out.width == cols):
            raise KernelError("gemm_skinny: out_tiled needs the gated product and a TiledRows of its size")
        out_t = out.data
    elif out.shape != (m, cols) or (swiglu and out.dtype != torch.bfloat16) \
            or out.dtype not in (torch.bfloat16, torch.float32):
        raise KernelError(f"gemm_skinny: out {tuple(out.shape)} {out.dtype} does not fit")
    mode = 2 if swiglu else (1 if out_t.dtype == torch.float32 else 0)
    check(lib.kva_gemm_skinny(_dev(out_t, "out"), _dev(x, "x"), _dev(w.data, "w"), m, n, k, k, cols, mode,
                              _opt(sumsq, "sumsq", torch.float32), parts, int(norm_width), float(eps),
                              None, None, 0, None, None, 1 if x_tiled else 0, 1 if out_tiled else 0, _stream()),
          "gemm_skinny")
    return out


def gemm_skinny_partial_ranges(m: int, n: int, k: int) -> int:
    """Into how many ranges of K :func:`gemm_skinny_partials` cuts an [n, k] product of ``m`` rows;
    0: it does not take the shape (it takes 17 to 64 rows, K a multiple of 128)."""
    return int(hip_lib().kva_gemm_skinny_partial_slices(int(m), int(n), int(k)))


def gemm_skinny_partials(x: torch.Tensor, w: "TiledWeight") -> PartialSums:
    """x @ W^T for 17 to 64 rows as fp32 partial products over ranges of K, one per group of
    workgroups, so that a matrix with few rows of tiles still fills the chip while the rows of x go
    through LDS; whoever takes the :class:`PartialSums` adds them up."""
    if not isinstance(w, TiledWeight) or w.halves != 1:
        raise KernelError("gemm_skinny_partials: the weight must be a plain TiledWeight")
    m, k = x.shape
    if x.dtype != torch.bfloat16 or k != w.k:
        raise KernelError(f"gemm_skinny_partials: bf16 x {tuple(x.shape)} does not fit weight [{w.n}, {w.k}]")
    ranges = gemm_skinny_partial_ranges(m, w.n, k)
    if ranges < 1:
        raise KernelError(f"gemm_skinny_partials: {m} rows of a [{w.n}, {k}] product are not taken (17..64 rows, K % 128 == 0)")
    parts = torch.empty((ranges, m, w.n), dtype=torch.float32, device=x.device)
    check(hip_lib().kva_gemm_skinny_partials(_dev(parts, "parts"), _dev(x, "x"), _dev(w.data, "w"), m, w.n, k, k,
                                             ranges, _stream()), "gemm_skinny_partials")
    return PartialSums(parts)


def gemm_skinny_qkv_rope_supported(m: int, k: int, head_dim: int) -> bool:
    return bool(hip_lib().kva_gemm_skinny_qkv_rope_supported(int(m), int(k), int(head_dim)))


def gemm_skinny_qkv_rope(x: torch.Tensor, w: TiledWeight, q_out: torch.Tensor, num_q_heads: int,
                         num_kv_heads: int, head_dim: int, positions: torch.Tensor,
                         cos: Optional[torch.Tensor], sin: Optional[torch.Tensor],
                         k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                         slot_mapping: Optional[torch.Tensor], page_size: int, *,
                         sumsq: Optional[torch.Tensor] = None, norm_width: int = 0, eps: float = 0.0):
    """The joined Q/K/V projection of at most 64 rows with rotation and cache write in its
    epilogue: ``q_out`` [M, nq*d] takes the rotated Q heads, the cache takes rotated K and plain V
    at ``slot_mapping`` (``k_cache`` None: nothing is cached).  ``cos``/``sin`` are the full
    tables [positions, d/2], or both None for no rotation.  ``sumsq`` as in :func:`gemm_skinny`."""
    if not isinstance(w, TiledWeight) or w.halves != 1:
        raise KernelError("gemm_skinny_qkv_rope: the weight must be a plain TiledWeight")
    m, k = x.shape
    if x.dtype != torch.bfloat16 or k != w.k or w.n != (num_q_heads + 2 * num_kv_heads) * head_dim:
        raise KernelError(f"gemm_skinny_qkv_rope: bf16 x {tuple(x.shape)} does not fit weight [{w.n}, {w.k}] "
                          f"for {num_q_heads}+2*{num_kv_heads} heads of {head_dim}")
    if q_out.shape != (m, num_q_heads * head_dim) or q_out.dtype != torch.bfloat16:
        raise KernelError("gemm_skinny_qkv_rope: q_out must be bf16 [M, nq * d]")
    if positions.shape != (m,):
        raise KernelError("gemm_skinny_qkv_rope: one position per row")
    if (cos is None) != (sin is None) or (cos is not None and (
            cos.shape != sin.shape or cos.dim() != 2 or cos.shape[1] * 2 != head_dim)):
        raise KernelError("gemm_skinny_qkv_rope: cos and sin tables must both be [positions, d/2]")
    if sumsq is not None and (sumsq.dim() != 2 or sumsq.shape[0] != m or norm_width <= 0):
        raise KernelError("gemm_skinny_qkv_rope: sumsq must be [M, parts] and norm_width positive")
    write = k_cache is not None
    if write:
        if v_cache is None or slot_mapping is None or slot_mapping.shape != (m,):
            raise KernelError("gemm_skinny_qkv_rope: K and V cache and one slot per row are all needed")
        check_cache_shapes("gemm_skinny_qkv_rope", k_cache, v_cache, num_kv_heads, head_dim)
        if k_cache.shape[3] != page_size or k_cache.dtype != torch.bfloat16:
            raise KernelError("gemm_skinny_qkv_rope: cache page size or dtype does not fit")
    check(hip_lib().kva_gemm_skinny_qkv_rope(
        _dev(q_out, "q_out"), q_out.shape[1], _dev(x, "x"), _dev(w.data, "w"), m, k, k, num_q_heads,
        num_kv_heads, head_dim, _opt(sumsq, "sumsq", torch.float32), sumsq.shape[1] if sumsq is not None else 0,
        int(norm_width), float(eps), _opt(cos, "cos", torch.float32), _opt(sin, "sin", torch.float32),
        _dev(positions, "positions", torch.int32),
        _dev(slot_mapping, "slot_mapping", torch.int32) if write else None,
        _opt(k_cache, "k_cache") if write else None, _opt(v_cache, "v_cache") if write else None,
        int(page_size), _stream()), "gemm_skinny_qkv_rope")
    return q_out


def gemm_skinny_sumsq_parts(n: int) -> int:
    return int(hip_lib().kva_gemm_skinny_sumsq_parts(int(n)))


def gemv_supported(m: int, n: int, k: int) -> bool:
    return bool(hip_lib().kva_gemv_supported(int(m), int(n), int(k)))


def gemv_sumsq_parts(n: int, k: int) -> int:
    """Partial sums of squares per token that :func:`gemv` writes with its residual epilogue."""
    return int(hip_lib().kva_gemv_sumsq_parts(int(n), int(k)))


def gemv(x: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor], swiglu: bool = False, *,
         sumsq: Optional[torch.Tensor] = None, norm_width: int = 0, eps: float = 0.0,
         hidden: Optional[torch.Tensor] = None, next_weight: Optional[torch.Tensor] = None,
         scaled_out: Optional[torch.Tensor] = None, sumsq_out: Optional[torch.Tensor] = None):
    """out = x @ W^T for one or two rows of x over the plain row-major bf16 weight ``w`` [N, K]
    (fp32 accumulation).  The options are :func:`gemm_skinny`'s: ``swiglu`` for a joined
    ``[gate; up]`` matrix, ``sumsq`` to finish the input's norm, ``hidden`` / ``next_weight`` /
    ``scaled_out`` / ``sumsq_out`` [M, :func:`gemv_sumsq_parts`] for the residual epilogue."""
    if x.dim() != 2 or w.dim() != 2 or x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 \
            or x.shape[1] != w.shape[1] or not w.is_contiguous() or x.stride(1) != 1:
        raise KernelError(f"gemv: bf16 x {tuple(x.shape)} does not fit a row-major bf16 weight {tuple(w.shape)}")
    m, k = x.shape
    n = w.shape[0]
    lib = hip_lib()
    if sumsq is not None and (sumsq.dim() != 2 or sumsq.shape[0] != m or norm_width <= 0):
        raise KernelError("gemv: sumsq must be [M, parts] and norm_width positive")
    parts = sumsq.shape[1] if sumsq is not None else 0
    norm = (_opt(sumsq, "sumsq", torch.float32), parts, int(norm_width), float(eps))
    if hidden is not None:
        if swiglu or out is not None:
            raise KernelError("gemv: the residual epilogue has no other output")
        p_out = gemv_sumsq_parts(n, k)
        if hidden.shape != (m, n) or hidden.dtype != torch.bfloat16 or scaled_out is None \
                or scaled_out.shape != (m, n) or scaled_out.dtype != torch.bfloat16 \
                or sumsq_out is None or sumsq_out.shape != (m, p_out):
            raise KernelError(f"gemv: hidden / scaled_out [M, N] bf16 and sumsq_out [M, {p_out}] needed")
        if next_weight is not None and next_weight.shape != (n,):
            raise KernelError("gemv: the next norm's weight must be [N]")
        check(lib.kva_gemv(None, _dev(x, "x", contiguous=False), _dev(w, "w"), m, n, k, x.stride(0), n, 3, *norm,
                           _dev(hidden, "hidden"), _opt(next_weight, "next_weight"),
                           1 if next_weight is not None and next_weight.dtype == torch.float32 else 0,
                           _dev(scaled_out, "scaled_out"), _dev(sumsq_out, "sumsq_out", torch.float32), _stream()),
              "gemv")
        return hidden
    cols = n // 2 if swiglu else n
    if out.shape != (m, cols) or (swiglu and out.dtype != torch.bfloat16) \
            or out.dtype not in (torch.bfloat16, torch.float32) or not out.is_contiguous():
        raise KernelError(f"gemv: out {tuple(out.shape)} {out.dtype} does not fit")
    mode = 2 if swiglu else (1 if out.dtype == torch.float32 else 0)
    check(lib.kva_gemv(_dev(out, "out"), _dev(x, "x", contiguous=False), _dev(w, "w"), m, n, k, x.stride(0), cols, mode, *norm,
                       None, None, 0, None, None, _stream()), "gemv")
    return out


def gemv_merged_supported(m: int, n: int, k: int, head_dim: int, parts: int) -> bool:
    """Whether :func:`gemv_merged` takes ``m`` tokens of ``k / head_dim`` heads with ``parts``
    partial results each."""
    return bool(hip_lib().kva_gemv_merged_supported(int(m), int(n), int(k), int(head_dim), int(parts)))


def gemv_merge_max_parts(m: int = 2) -> int:
    """Partial results a row that :func:`gemv_merged` adds up for ``m`` tokens."""
    return int(hip_lib().kva_gemv_merge_max_parts(int(m)))


def gemv_merged(x: AttentionPartials, w: torch.Tensor, hidden: torch.Tensor, next_weight: Optional[torch.Tensor],
                scaled_out: torch.Tensor, sumsq_out: torch.Tensor) -> torch.Tensor:
    """:func:`gemv` with its residual epilogue over an attention output that is still in partial
    results per key range: the kernel adds them up (as the merge kernel would, rounded to bf16)
    where it would have read the tokens."""
    m, k = x.shape
    n = w.shape[0]
    if w.dim() != 2 or w.dtype != torch.bfloat16 or w.shape[1] != k or not w.is_contiguous():
        raise KernelError(f"gemv_merged: partial results of {tuple(x.shape)} do not fit a row-major bf16 weight {tuple(w.shape)}")
    if not gemv_merged_supported(m, n, k, x.head_dim, x.parts):
        raise KernelError(f"gemv_merged: {m} tokens, weight {tuple(w.shape)}, heads of {x.head_dim}, {x.parts} partial results: not supported")
    p_out = gemv_sumsq_parts(n, k)
    if hidden.shape != (m, n) or hidden.dtype != torch.bfloat16 or scaled_out.shape != (m, n) \
            or scaled_out.dtype != torch.bfloat16 or sumsq_out.shape != (m, p_out):
        raise KernelError(f"gemv_merged: hidden / scaled_out [M, N] bf16 and sumsq_out [M, {p_out}] needed")
    if next_weight is not None and next_weight.shape != (n,):
        raise KernelError("gemv_merged: the next norm's weight must be [N]")
    check(hip_lib().kva_gemv_merged(
        _dev(x.part_o, "part_o", torch.float32), _dev(x.part_ml, "part_ml", torch.float32), x.parts, x.head_dim,
        _dev(w, "w"), m, n, k, _dev(hidden, "hidden"), _opt(next_weight, "next_weight"),
        1 if next_weight is not None and next_weight.dtype == torch.float32 else 0,
        _dev(scaled_out, "scaled_out"), _dev(sumsq_out, "sumsq_out", torch.float32), _stream()), "gemv_merged")
    return hidden


def gemv_qkv_rope_supported(m: int, k: int, head_dim: int) -> bool:
    return bool(hip_lib().kva_gemv_qkv_rope_supported(int(m), int(k), int(head_dim)))


def gemv_qkv_rope(x: torch.Tensor, w: torch.Tensor, q_out: torch.Tensor, num_q_heads: int,
                  num_kv_heads: int, head_dim: int, positions: torch.Tensor,
                  cos: Optional[torch.Tensor], sin: Optional[torch.Tensor],
                  k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                  slot_mapping: Optional[torch.Tensor], page_size: int, *,
                  sumsq: Optional[torch.Tensor] = None, norm_width: int = 0, eps: float = 0.0):
    """:func:`gemm_skinny_qkv_rope` for one or two rows, over the plain row-major weight."""
    m, k = x.shape
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or not w.is_contiguous() \
            or w.shape != ((num_q_heads + 2 * num_kv_heads) * head_dim, k):
        raise KernelError(f"gemv_qkv_rope: bf16 x {tuple(x.shape)} does not fit weight {tuple(w.shape)} "
                          f"for {num_q_heads}+2*{num_kv_heads} heads of {head_dim}")
    if q_out.shape != (m, num_q_heads * head_dim) or q_out.dtype != torch.bfloat16 or not q_out.is_contiguous():
        raise KernelError("gemv_qkv_rope: q_out must be bf16 [M, nq * d]")
    if positions.shape != (m,):
        raise KernelError("gemv_qkv_rope: one position per row")
    if (cos is None) != (sin is None) or (cos is not None and (
            cos.shape != sin.shape or cos.dim() != 2 or cos.shape[1] * 2 != head_dim)):
        raise KernelError("gemv_qkv_rope: cos and sin tables must both be [positions, d/2]")
    if sumsq is not None and (sumsq.dim() != 2 or sumsq.shape[0] != m or norm_width <= 0):
        raise KernelError("gemv_qkv_rope: sumsq must be [M, parts] and norm_width positive")
    write = k_cache is not None
    if write:
        if v_cache is None or slot_mapping is None or slot_mapping.shape != (m,):
            raise KernelError("gemv_qkv_rope: K and V cache and one slot per row are all needed")
        check_cache_shapes("gemv_qkv_rope", k_cache, v_cache, num_kv_heads, head_dim)
        if k_cache.shape[3] != page_size or k_cache.dtype != torch.bfloat16:
            raise KernelError("gemv_qkv_rope: cache page size or dtype does not fit")
    check(hip_lib().kva_gemv_qkv_rope(
        _dev(q_out, "q_out"), q_out.shape[1], _dev(x, "x"), _dev(w, "w"), m, k, x.stride(0), num_q_heads,
        num_kv_heads, head_dim, _opt(sumsq, "sumsq", torch.float32), sumsq.shape[1] if sumsq is not None else 0,
        int(norm_width), float(eps), _opt(cos, "cos", torch.float32), _opt(sin, "sin", torch.float32),
        _dev(positions, "positions", torch.int32),
        _dev(slot_mapping, "slot_mapping", torch.int32) if write else None,
        _opt(k_cache, "k_cache") if write else None, _opt(v_cache, "v_cache") if write else None,
        int(page_size), _stream()), "gemv_qkv_rope")
    return q_out


def normed_rows_finish(scaled: torch.Tensor, sumsq: torch.Tensor, norm_width: int, eps: float,
                       out: torch.Tensor, row_idx: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[i] = scaled[row] * rsqrt(sum(sumsq[row]) / norm_width + eps), row = row_idx[i] or i."""
    rows, width = out.shape
    if scaled.dim() != 2 or scaled.shape[1] != width or sumsq.shape[0] != scaled.shape[0] \
            or scaled.dtype != torch.bfloat16 or out.dtype != torch.bfloat16:
        raise KernelError("normed_rows_finish: bf16 scaled [T, H], sumsq [T, parts], out [rows, H]")
    if row_idx is None and rows != scaled.shape[0]:
        raise KernelError("normed_rows_finish: out needs as many rows as scaled")
    check(hip_lib().kva_normed_rows_finish(
        _dev(out, "out"), _dev(scaled, "scaled"), _dev(sumsq, "sumsq", torch.float32), sumsq.shape[1],
        rows, _opt(row_idx, "row_idx", torch.int32), width, float(eps), _stream()), "normed_rows_finish")
    return out


# --------------------------------------------------------------------------------------
# Measurement: device time per class of kernel, from events around every launch.
KERNEL_CLASSES = {
    "embed_gather": "embedding", "embed_gather_prep": "embedding", "rmsnorm": "norm", "normed_rows_finish": "norm",
    "residual_add": "elementwise", "scale_softcap": "elementwise", "cast": "elementwise",
    "silu_mul": "activation", "rope_kv_write": "rope + cache write",
    "attention_rowwise": "attention", "attention_mfma": "attention", "attention_lds": "attention",
    "attention_mfma_rope": "attention",
    "gemm_nt_f32": "gemm fp32", "gemm_vendor": "gemm (vendor library)",
    "gemm_skinny": "gemm (few rows)", "gemm_skinny_qkv_rope": "gemm (few rows)",
    "gemv": "gemm (few rows)", "gemv_qkv_rope": "gemm (few rows)", "gemv_merged": "gemm (few rows)",
    "sample": "sampling", "mark_tokens": "sampling",
}


class KernelClassTimer:
    """``with KernelClassTimer() as t: ...`` brackets every kernel entry point of this module
    with a pair of events on the current stream; ``t.milliseconds()`` then gives the device time
    per class of kernel (the reference times its attention micro-benchmark the same way,
    ``micro/main_paged.cu:102-114``).  Launches one by one - a step replayed from a graph shows
    nothing here - so a class's time includes the gaps between its launches and their
    predecessors; it tells where a step's time goes, not how fast a kernel can be."""

    def __init__(self):
        self._marks = []
        self._saved = {}

    def __enter__(self):
        module = globals()
        for name, cls in KERNEL_CLASSES.items():
            fn = module[name]
            self._saved[name] = fn
            module[name] = self._wrap(fn, cls)
        return self

    def _wrap(self, fn, cls):
        marks = self._marks

        def timed(*args, **kwargs):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            try:
                return fn(*args, **kwargs)
            finally:
                b.record()
                marks.append((cls, a, b))
        return timed

    def __exit__(self, *exc):
        globals().update(self._saved)
        self._saved = {}
        return False

    def milliseconds(self) -> dict:
        torch.cuda.synchronize()
        out: dict = {}
        for cls, a, b in self._marks:
            out[cls] = out.get(cls, 0.0) + a.elapsed_time(b)
        return {k: round(v, 4) for k, v in sorted(out.items(), key=lambda kv: -kv[1])}
