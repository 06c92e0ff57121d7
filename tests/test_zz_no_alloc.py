"""The attention entry point that allocates nothing (``kva_attention_mfma_static``, declared in
``csrc/attention_static.h``), called through ctypes as a caller without an allocator would: its
output must be the existing entry point's, bit for bit, on two calls in a row, the second with a
smaller input (the static scratch array still holds the first call's partial results then)."""
import ctypes
import math

import numpy as np
import pytest
import torch

from kv_cache_optimization_for_llm_amd.ops import kernels as K

pytestmark = pytest.mark.gpu

P, I, F = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
STATIC_ARGS = [P, P, I, P, P, P, I, P, P, P, I, I, P, P, P, I, I, I, I, I, F, I, I, I, I, I, P]


def case(batch, context, nq, nkv, d, page, seed, gpu):
    """``batch`` decoding requests with ``context`` keys each in a shuffled paged cache."""
    g = torch.Generator().manual_seed(seed)
    blocks = (context + page - 1) // page
    pages = batch * blocks + 5
    kc = K.keys_to_pages(torch.randn(pages, nkv, page, d, generator=g).to(torch.bfloat16)).to(gpu)
    vc = torch.randn(pages, nkv, d, page, generator=g).to(torch.bfloat16).to(gpu)
    table = torch.randperm(pages, generator=g)[:batch * blocks].view(batch, blocks).to(torch.int32).to(gpu)
    q = (torch.randn(batch, nq * d, generator=g) * 1.5).to(torch.bfloat16).to(gpu)
    ar = torch.arange(batch, dtype=torch.int32, device=gpu)
    return dict(q=q, kc=kc, vc=vc, table=table, item_entry=ar.clone(), item_row0=torch.zeros_like(ar),
                entry_seat=ar.clone(), q_start=torch.arange(batch + 1, dtype=torch.int32, device=gpu),
                start_pos=torch.full((batch,), context - 1, dtype=torch.int32, device=gpu))


def test_static_attention_equals_the_allocating_entry_point_twice_in_a_row(gpu):
    from kv_cache_optimization_for_llm_amd.ops import kernels as K
    from kv_cache_optimization_for_llm_amd.ops.library import hip_lib
    lib = hip_lib()
    fn = lib.kva_attention_mfma_static
    fn.argtypes, fn.restype = STATIC_ARGS, ctypes.c_int
    lib.kva_attention_mfma_static_scratch_bytes.argtypes = [I, I, I]
    lib.kva_attention_mfma_static_scratch_bytes.restype = ctypes.c_longlong
    nq, nkv, d, page = 8, 2, 64, 16
    scale = 1.0 / math.sqrt(d)
    stream = torch.cuda.current_stream().cuda_stream
    # the first call is the larger one: 6 requests x 1,000 keys in 8 splits; the second, 2 requests x
    # 300 keys in 3 splits, finds the first call's partial results in the scratch array
    for batch, context, splits, seed in ((6, 1000, 8, 1), (2, 300, 3, 2)):
        c = case(batch, context, nq, nkv, d, page, seed, gpu)
        per = ((context + splits - 1) // splits + 31) // 32 * 32
        want = torch.full((batch, nq * d), float("nan"), dtype=torch.bfloat16, device=gpu)
        K.attention_mfma(c["q"], nq * d, want, c["kc"], c["vc"], c["table"], c["item_entry"], c["item_row0"],
                         c["entry_seat"], c["q_start"], c["start_pos"], nq, nkv, d, scale, 0, splits, per)
        got = torch.full_like(want, float("nan"))
        assert 0 < lib.kva_attention_mfma_static_scratch_bytes(batch * nq, d, splits) <= 16 << 20
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated(gpu)
        rc = fn(got.data_ptr(), c["q"].data_ptr(), nq * d, c["kc"].data_ptr(), c["vc"].data_ptr(),
                c["table"].data_ptr(), c["table"].shape[1], None, c["item_entry"].data_ptr(),
                c["item_row0"].data_ptr(), batch, 1, c["entry_seat"].data_ptr(), c["q_start"].data_ptr(),
                c["start_pos"].data_ptr(), batch * nq, nq, nkv, d, page, scale, 0, splits, per, 0, 1, stream)
        assert rc == 0, lib.kva_last_error()
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated(gpu) == before
        assert not torch.isnan(got.float()).any()
        assert torch.equal(got, want), f"batch {batch}, context {context}, {splits} splits"
    # one split needs no scratch at all and gives the same as the existing entry point too
    c = case(3, 200, nq, nkv, d, page, 3, gpu)
    want = torch.empty((3, nq * d), dtype=torch.bfloat16, device=gpu)
    K.attention_mfma(c["q"], nq * d, want, c["kc"], c["vc"], c["table"], c["item_entry"], c["item_row0"],
                     c["entry_seat"], c["q_start"], c["start_pos"], nq, nkv, d, scale)
    got = torch.empty_like(want)
    assert fn(got.data_ptr(), c["q"].data_ptr(), nq * d, c["kc"].data_ptr(), c["vc"].data_ptr(),
              c["table"].data_ptr(), c["table"].shape[1], None, c["item_entry"].data_ptr(),
              c["item_row0"].data_ptr(), 3, 1, c["entry_seat"].data_ptr(), c["q_start"].data_ptr(),
              c["start_pos"].data_ptr(), 3 * nq, nq, nkv, d, page, scale, 0, 1, 0, 0, 1, stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    # a call beyond the array's size is refused with a message and launches nothing
    big_rows, big_splits = 64 * 32, 64
    assert lib.kva_attention_mfma_static_scratch_bytes(big_rows, 128, big_splits) > 16 << 20
    rc = fn(got.data_ptr(), c["q"].data_ptr(), nq * d, c["kc"].data_ptr(), c["vc"].data_ptr(),
            c["table"].data_ptr(), c["table"].shape[1], None, c["item_entry"].data_ptr(),
            c["item_row0"].data_ptr(), 3, 1, c["entry_seat"].data_ptr(), c["q_start"].data_ptr(),
            c["start_pos"].data_ptr(), big_rows, nq, nkv, 128, page, scale, 0, big_splits, 32, 0, 1, stream)
    assert rc != 0 and b"static array holds" in lib.kva_last_error()
    torch.cuda.synchronize()
