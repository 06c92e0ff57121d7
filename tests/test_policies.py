"""Host-side decisions that need no GPU: how attention keys are cut into splits, and how large a
cache pool is made from leftover device memory."""
import pytest

from kv_cache_optimization_for_llm_amd.engine.engine import EngineError, pool_pages_from_memory
from kv_cache_optimization_for_llm_amd.ops.attention import (choose_decode_ranges, choose_left_ranges, choose_lds_splits, choose_splits,
                                                             use_lds_kernel)

KERNEL_MAX_SPLITS = 256         # what the kernels and their merge take (kva_attention_max_splits)


@pytest.mark.parametrize("nkv", [1, 2, 4, 8])
@pytest.mark.parametrize("items", [1, 2, 3])
@pytest.mark.parametrize("context", [4096, 32768, 65536, 100000, 131072])
def test_key_splits_never_exceed_what_the_kernels_take(nkv, items, context):
    """Few kv heads, one or two decoding requests and a long context ask for many splits; the
    policy must stop at the kernels' limit, and its ranges must still cover every key."""
    for splits, per in (choose_splits(items, nkv, context, KERNEL_MAX_SPLITS),
                        choose_splits(items, nkv, context, KERNEL_MAX_SPLITS, decoding=True),
                        choose_lds_splits(items * nkv, context, KERNEL_MAX_SPLITS),
                        choose_lds_splits(items * nkv, context, KERNEL_MAX_SPLITS, head_dim=128)):
        assert 1 <= splits <= KERNEL_MAX_SPLITS
        if splits > 1:
            assert per % 32 == 0 and splits * per >= context and (splits - 1) * per < context


def test_the_clamp_is_what_bites_for_few_kv_heads():
    # one request on one kv head at 131,072 keys would ask for 1,024 ranges of 128 keys
    assert choose_splits(1, 1, 131072, 4096)[0] == 1024
    assert choose_splits(1, 1, 131072, KERNEL_MAX_SPLITS) == (256, 512)
    assert choose_splits(1, 4, 65536, KERNEL_MAX_SPLITS) == (256, 256)
    assert choose_splits(4096, 8, 2048, KERNEL_MAX_SPLITS) == (1, 0)      # a big prompt fills the GPU by itself
    assert choose_splits(1, 8, 100, KERNEL_MAX_SPLITS) == (1, 0)          # too short to split


@pytest.mark.parametrize("nkv", [1, 2, 5, 8])
@pytest.mark.parametrize("items", [1, 2, 8, 17, 31, 48, 64, 100, 128, 300])
@pytest.mark.parametrize("context", [1, 40, 200, 768, 4096, 8192, 131072])
@pytest.mark.parametrize("head_dim", [64, 128, 256])
def test_key_ranges_of_decoded_tokens_and_the_wavefronts_that_share_them(nkv, items, context, head_dim):
    """Whatever the batch: the ranges cover every key, there are no more of them than the kernels
    take, the wavefronts of a workgroup divide them, and head sizes above 128 get one."""
    splits, per, waves = choose_decode_ranges(items, nkv, context, head_dim, KERNEL_MAX_SPLITS)
    assert 1 <= splits <= KERNEL_MAX_SPLITS and waves in (1, 2, 4) and splits % waves == 0
    if splits > 1:
        # every key in a range, and no workgroup (of `waves` neighbouring ranges) without a key
        assert per % 32 == 0 and splits * per >= context and (splits - waves) * per < context
    if head_dim > 128:
        assert waves == 1


def test_where_decoded_tokens_need_no_merge_launch():
    # 17 to 63 requests of 8 kv heads: four ranges, all in one workgroup
    for items in (17, 24, 32, 48, 63):
        assert choose_decode_ranges(items, 8, 768, 64, KERNEL_MAX_SPLITS) == (4, 192, 4)
    assert choose_decode_ranges(64, 8, 768, 64, KERNEL_MAX_SPLITS) == (1, 0, 1)          # enough wavefronts as they are
    assert choose_decode_ranges(64, 8, 8192, 64, KERNEL_MAX_SPLITS) == (4, 2048, 4)      # but not for long contexts
    assert choose_decode_ranges(20, 8, 100, 64, KERNEL_MAX_SPLITS) == (2, 64, 2)
    # many ranges share a workgroup only where the merge has much to read
    assert choose_decode_ranges(8, 8, 8192, 64, KERNEL_MAX_SPLITS) == (16, 512, 4)
    assert choose_decode_ranges(8, 8, 768, 64, KERNEL_MAX_SPLITS) == (4, 192, 4)
    # three to fifteen requests above 2,048 keys (from six requests on above 1,024): four ranges to a
    # workgroup, and no more workgroups than compute units
    assert choose_decode_ranges(8, 8, 4096, 64, KERNEL_MAX_SPLITS) == (16, 256, 4)
    assert choose_decode_ranges(3, 8, 8192, 64, KERNEL_MAX_SPLITS) == (40, 224, 4)
    assert choose_decode_ranges(7, 8, 8192, 64, KERNEL_MAX_SPLITS) == (16, 512, 4)          # 224 workgroups, not 280
    assert choose_decode_ranges(12, 8, 2048, 64, KERNEL_MAX_SPLITS) == (8, 256, 4)
    assert choose_decode_ranges(5, 8, 2048, 64, KERNEL_MAX_SPLITS)[2] == 1 and choose_decode_ranges(6, 8, 2048, 64, KERNEL_MAX_SPLITS)[2] == 4
    assert choose_decode_ranges(5, 8, 768, 64, KERNEL_MAX_SPLITS)[2] == 1
    assert choose_decode_ranges(16, 8, 4096, 64, KERNEL_MAX_SPLITS) == (8, 512, 1)
    assert choose_decode_ranges(5, 8, 8192, 128, KERNEL_MAX_SPLITS)[2] == 1                 # head size 128: not measured
    assert choose_decode_ranges(1, 8, 8192, 64, KERNEL_MAX_SPLITS) == (64, 128, 4)
    assert choose_decode_ranges(1, 8, 768, 64, KERNEL_MAX_SPLITS) == (12, 64, 1)
    # short contexts: four ranges from 8 requests of 8 kv heads on
    assert choose_decode_ranges(8, 8, 768, 64, KERNEL_MAX_SPLITS) == (4, 192, 4)
    assert choose_decode_ranges(7, 8, 768, 64, KERNEL_MAX_SPLITS)[2] == 1
    assert choose_decode_ranges(8, 8, 2048, 64, KERNEL_MAX_SPLITS) == (16, 128, 4)
    assert choose_decode_ranges(32, 8, 768, 256, KERNEL_MAX_SPLITS)[2] == 1               # head size 256: one wavefront
    # one request and a long context: twice the ranges the merge kernel is given otherwise, four to a
    # workgroup, so that there is still a workgroup for every compute unit
    assert choose_decode_ranges(1, 8, 32768, 64, KERNEL_MAX_SPLITS) == (128, 256, 4)
    assert choose_decode_ranges(1, 8, 131072, 64, KERNEL_MAX_SPLITS) == (128, 1024, 4)
    assert choose_decode_ranges(1, 1, 65536, 64, KERNEL_MAX_SPLITS) == (256, 256, 1)      # 64 workgroups would be too few
    assert choose_decode_ranges(16, 8, 8192, 64, KERNEL_MAX_SPLITS) == (8, 1024, 1)
    # head size 128: four ranges up to 256 pairs only, and many ranges keep a wavefront each
    assert choose_decode_ranges(32, 8, 768, 128, KERNEL_MAX_SPLITS) == (4, 192, 4)
    assert choose_decode_ranges(33, 8, 768, 128, KERNEL_MAX_SPLITS) == (1, 0, 1)
    assert choose_decode_ranges(47, 8, 2048, 128, KERNEL_MAX_SPLITS) == (1, 0, 1)
    assert choose_decode_ranges(33, 8, 768, 64, KERNEL_MAX_SPLITS) == (4, 192, 4)
    # ... and from 128 pairs on, where head size 64 shares from 64
    assert choose_decode_ranges(8, 8, 768, 64, KERNEL_MAX_SPLITS) == (4, 192, 4)
    assert choose_decode_ranges(12, 8, 768, 128, KERNEL_MAX_SPLITS) == (8, 96, 1)
    assert choose_decode_ranges(16, 8, 768, 128, KERNEL_MAX_SPLITS) == (4, 192, 4)
    assert choose_decode_ranges(48, 8, 768, 128, KERNEL_MAX_SPLITS) == (1, 0, 1)
    assert choose_decode_ranges(64, 8, 8192, 128, KERNEL_MAX_SPLITS) == (1, 0, 1)
    assert choose_decode_ranges(8, 8, 8448, 128, KERNEL_MAX_SPLITS)[2] == 1


def test_which_prompt_rows_go_to_the_workgroup_kernel():
    """Workgroups (128 query rows x kv heads) and mean keys a row decide; head size 128 goes there
    earlier, and with shorter key ranges."""
    # a 2,048-token prompt from position 0 on 8 kv heads, 4 query heads each: 512 workgroups, 1,024 keys a row
    assert not use_lds_kernel(512, 1024.5, 64) and use_lds_kernel(512, 1024.5, 128)
    assert use_lds_kernel(1024, 2048.5, 64) and use_lds_kernel(1024, 2048.5, 96)
    assert use_lds_kernel(768, 10, 64)                       # three workgroups per compute unit: whatever they visit
    assert use_lds_kernel(576, 1152.5, 64) and not use_lds_kernel(576, 500, 64)      # a 2,304-token prompt; many short ones
    # a 256-token portion at position 4,096: 64 workgroups
    assert not use_lds_kernel(64, 4224.5, 64) and use_lds_kernel(64, 4224.5, 128)
    assert not use_lds_kernel(64, 1152.5, 128)               # the same portion at position 1,024
    # head size 128, 24 heads on 8 kv heads: a 2,048-token prompt (384 workgroups) and one of 2,560 (480)
    # stay with the one-wavefront kernel, 3,072 tokens (576) do not; nor does a portion whose rows visit 2,048 keys
    assert not use_lds_kernel(384, 1024.5, 128) and not use_lds_kernel(480, 1280.5, 128)
    assert use_lds_kernel(576, 1536.5, 128) and use_lds_kernel(192, 2560.5, 128)
    assert not use_lds_kernel(8, 8000, 128)                  # a 32-token portion: too few rows to share a key block
    assert choose_lds_splits(64, 4352, KERNEL_MAX_SPLITS, head_dim=128) == (8, 544)
    assert choose_lds_splits(128, 4608, KERNEL_MAX_SPLITS, head_dim=64) == (4, 1152)
    assert choose_lds_splits(512, 2048, KERNEL_MAX_SPLITS, head_dim=128) == (1, 0)


def test_pool_from_leftover_memory():
    GiB = 1 << 30
    # Llama-3.2-1B: 16 layers x 2 x 8 heads x 64 x 16 tokens x 2 bytes = 512 KiB a page
    page_bytes = 16 * 2 * 8 * 64 * 16 * 2
    # config.json says 131,072 positions and the server has 64 seats: every seat at its longest
    # would be 256 GiB; the pool takes what is free instead
    pages = pool_pages_from_memory(200 * GiB, page_bytes, page_size=16, max_seqs=64, max_seq_len=131072,
                                   margin_bytes=2 * GiB, step_bytes=4 * GiB)
    assert pages == (200 - 2 - 4) * GiB // page_bytes
    assert pages * page_bytes <= 194 * GiB < 64 * 131072 // 16 * page_bytes
    # a small model on a big device: never more than every seat at its longest
    assert pool_pages_from_memory(200 * GiB, 4096, page_size=16, max_seqs=8, max_seq_len=100,
                                  margin_bytes=GiB) == 8 * 7
    with pytest.raises(EngineError) as e:
        pool_pages_from_memory(3 * GiB, page_bytes, page_size=16, max_seqs=8, max_seq_len=8192,
                               margin_bytes=2 * GiB, step_bytes=2 * GiB)
    assert "no room for a cache pool" in str(e.value)


def test_row_counts_timed_for_decode_batches_cover_every_batch_above_the_few_rows_kernels():
    """Every batch from 17 seats up to the largest has a timed row count at or above it and at
    most twice its size (the sharing rule of the vendor product's plans)."""
    from kv_cache_optimization_for_llm_amd.ops.gemm_bf16 import decode_tune_rows
    assert decode_tune_rows(1) == [] and decode_tune_rows(16) == []
    assert decode_tune_rows(17) == [17] and decode_tune_rows(32) == [32]
    assert decode_tune_rows(64) == [32, 64] and decode_tune_rows(100) == [32, 64, 100]
    for seats in (17, 40, 64, 200, 384):
        rows = decode_tune_rows(seats)
        for batch in range(17, seats + 1):
            assert any(batch <= r <= 2 * batch for r in rows), (seats, batch)


def test_which_products_of_one_or_two_tokens_take_the_matrix_vector_kernel():
    from kv_cache_optimization_for_llm_amd.ops.gemm_bf16 import use_gemv
    # the four products of a layer and the head at the 1B and 8B sizes: every one the kernel has an instance for
    for n, k in ((3072, 2048), (2048, 2048), (16384, 2048), (2048, 8192), (128256, 2048),
                 (6144, 4096), (4096, 4096), (28672, 4096), (128256, 4096)):
        assert use_gemv(1, n, k) and use_gemv(2, n, k), (n, k)
    assert not use_gemv(1, 4096, 14336)                 # no instance for that K
    assert not use_gemv(3, 2048, 2048)
    # the 3B sizes: all but the down projection, whose rows are long and many
    for n, k in ((5120, 3072), (3072, 3072), (16384, 3072), (128256, 3072)):
        assert use_gemv(1, n, k) and use_gemv(2, n, k), (n, k)
    assert not use_gemv(1, 3072, 8192) and not use_gemv(2, 3072, 8192)
    # long rows cost a second token more than a first one
    assert use_gemv(1, 4096, 5120) and not use_gemv(2, 4096, 5120)
    assert use_gemv(1, 2048, 8192) and use_gemv(2, 2048, 8192)


@pytest.mark.parametrize("context", [512, 513, 600, 768, 769, 1000, 1024, 1500, 2048])
@pytest.mark.parametrize("items", [1, 2])
def test_key_ranges_left_for_an_output_projection_that_adds_them_up(items, context, ):
    ranges, per, waves = choose_left_ranges(items, context, 64, 4)
    assert waves == 4 and ranges % 4 == 0 and 2 <= ranges // 4 <= 4          # what the consumer takes
    assert per % 32 == 0 and per >= 64 and ranges * per >= context           # every key in a range
    assert (ranges - 4) * per < context                                     # no workgroup without a key


def test_where_no_key_ranges_are_left_to_the_output_projection():
    assert choose_left_ranges(3, 768, 64, 4) is None            # the matrix-vector kernel takes two tokens
    assert choose_left_ranges(1, 300, 64, 4) is None            # too short for two workgroups of four ranges
    assert choose_left_ranges(1, 4096, 64, 4) is None           # too long for 16 ranges
    assert choose_left_ranges(1, 768, 128, 4) is None           # measured at head sizes up to 64
    assert choose_left_ranges(1, 768, 64, 1) is None and choose_left_ranges(1, 768, 64, 0) is None
    assert choose_left_ranges(1, 768, 64, 2) == (8, 96, 4)


def test_workgroups_a_pair_at_long_contexts_even_out_the_compute_units():
    """17 to 63 requests on 8 kv heads at 4,096 keys or more: one workgroup of four ranges a pair
    where that fills the compute units' turns well (192, 448 of 256), two or three where it
    leaves most units idle in the last turn (264, 320 of 512)."""
    from kv_cache_optimization_for_llm_amd.ops.attention import _workgroups_a_pair
    assert [_workgroups_a_pair(p, 8192) for p in (136, 160, 176, 192, 264, 320, 384, 448, 504)] == [3, 3, 1, 1, 3, 3, 2, 1, 1]
    assert [_workgroups_a_pair(p, 4096) for p in (136, 192, 264, 320, 384, 448)] == [1, 1, 2, 2, 2, 1]
    assert choose_decode_ranges(33, 8, 8192, 64, KERNEL_MAX_SPLITS) == (12, 704, 4)
    assert choose_decode_ranges(48, 8, 8192, 64, KERNEL_MAX_SPLITS) == (8, 1024, 4)
    assert choose_decode_ranges(56, 8, 8192, 64, KERNEL_MAX_SPLITS) == (4, 2048, 4)
    assert choose_decode_ranges(40, 8, 4096, 64, KERNEL_MAX_SPLITS) == (8, 512, 4)
    assert choose_decode_ranges(40, 8, 2048, 64, KERNEL_MAX_SPLITS) == (4, 512, 4)          # shorter contexts: as before
    assert choose_decode_ranges(40, 8, 131072, 64, KERNEL_MAX_SPLITS) == (12, 10944, 4)
