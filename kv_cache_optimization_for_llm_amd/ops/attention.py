"""Chooses the attention kernel for a step's batch.

float32 always takes the plain kernel (true fp32 arithmetic, fixed key order).  bfloat16 takes
the matrix-core kernel when the head size and page size allow it, and splits the keys of long
contexts over several wavefronts when the batch alone would leave most of the GPU idle.
"""
from __future__ import annotations

import torch

from . import kernels as K

# Wavefronts wanted in flight when keys are split.  Prompt portions (two row tiles per wavefront,
# keys shared through L2): a few per compute unit.  Decoded tokens stream their keys once and pay
# 4-5 us for the merge kernel as soon as there is more than one split: with three wavefronts for
# every two compute units they are not split at all, below that until there are four per unit,
# in ranges of at least 64 keys (128 for long contexts).  Whole decode steps of the 1B shape
# (8 kv heads, head size 64) in one process, ms per step, old rule (2,048 wavefronts, ranges of at
# least 128 keys) against this one:
#   contexts of 768: batch 1 0.890 -> 0.845, batch 8 0.915 -> 0.911, batch 32 1.384 -> 1.370,
#   batch 64 1.583 -> 1.510 (one range, no merge); contexts of 8,192: batch 1 0.919 -> 0.919,
#   batch 8 1.298 -> 1.269 (16 ranges instead of 32), batch 64 4.13 -> 4.10
_TARGET_WAVES = 2048
_MIN_KEYS_PER_SPLIT = 128
_TARGET_WAVES_DECODE = 1024
_UNSPLIT_WAVES_DECODE = 384
_MIN_KEYS_PER_SPLIT_DECODE = 64
_LONG_CONTEXT_DECODE = 2048         # above it a range holds at least _MIN_KEYS_PER_SPLIT keys
# The merge kernel walks the ranges of a row one after the other, so one request alone with a long
# context is not cut as far as the wavefront count asks: its attention at 32,768 keys takes 24.6 /
# 18.6 / 22.0 / 28.4 us in 32 / 64 / 128 / 256 ranges, at 131,072 keys 76.0 / 50.0 / 49.6 / 56.7.
# (8 kv heads: 512 wavefronts; with fewer heads the ranges go on until there are that many.)
_MAX_SPLITS_DECODE = 64
_MIN_WAVES_DECODE = 512
_KEEP_CACHED_BYTES = 64 << 20       # keys and values of one call (one layer) that may stay in the caches

# wide items (two row tiles per wave) are used when they alone give this many waves
_WIDE_MIN_WAVES = 1024
_PAIR_MIN_WAVES = 2048      # two items per wavefront once that still leaves a wavefront per SIMD
# The workgroup kernel (128 query rows share each key block through LDS) pays one barrier per key
# block: it wins once there are three workgroups per compute unit, or one per two units when the
# rows visit thousands of keys each (measured: 2,048-token prompt from position 0 a tie, 4,096 1.5x;
# portions of 512 tokens of an 8,192-token prompt, 128 workgroups, 5 % faster, and 25 % faster with
# their keys cut into ranges so that about a thousand workgroups run; portions of 256 tokens no faster).
_LDS_MIN_GROUPS = 128
_LDS_MANY_GROUPS = 768
_LDS_MIN_MEAN_KEYS = 2048
_LDS_SOME_GROUPS = 576
_LDS_SOME_GROUPS_MEAN_KEYS = 1024
# Head sizes above 96 do twice the matrix-core work per key and row for the same vector work, and
# one wavefront with two row tiles of them fills its SIMD's registers alone.  With keys laid out in
# chunks of 8 elements across a page (one run of bytes per operand load) the one-wavefront kernel
# holds out longer than it did: head size 128, one prompt from position 0, 24 heads, one-wavefront
# against workgroup kernel: 1,024 tokens 31 against 36 us, 2,048 (384 workgroups) 61 against 71,
# 2,560 (480) 80 against 91, but 3,072 (576) 163 against 112 and 4,096 221 against 161; 32 heads,
# 2,560 tokens (640 workgroups) 142 against 97.  So: from 512 workgroups on, or where rows visit
# 2,048 keys or more on average - with the keys cut into shorter ranges also for short portions deep
# in a context (256 tokens at position 4,096: 48 us in 8 ranges against 71 for the one-wavefront
# kernel at its best split; 128 at 8,192: 47 against 64; 64 at 8,192: 35 against 41).
_LDS_MIN_MEAN_KEYS_WIDE_HEADS = 2048
_LDS_MANY_GROUPS_WIDE_HEADS = 512
_LDS_MIN_GROUPS_WIDE_HEADS = 16
_LDS_TARGET_GROUPS_WIDE_HEADS = 512
_LDS_MIN_KEYS_PER_SPLIT_WIDE_HEADS = 256
# where the choice can change (a step shape that has a graph is told apart by these too)
LDS_MEAN_KEYS_STEPS = tuple(sorted({_LDS_MIN_MEAN_KEYS_WIDE_HEADS, _LDS_SOME_GROUPS_MEAN_KEYS, _LDS_MIN_MEAN_KEYS}))
# few workgroups that each walk thousands of keys: the keys are cut into ranges, one workgroup each
_LDS_TARGET_GROUPS = 1024
_LDS_MIN_KEYS_PER_SPLIT = 1024


def use_lds_kernel(groups: int, mean_keys: float, head_dim: int) -> bool:
    """Whether prompt rows that make ``groups`` workgroups of 128 rows (over all kv heads) and visit
    ``mean_keys`` keys each on average go to the workgroup kernel."""
    if groups >= _LDS_MANY_GROUPS:
        return True
    if head_dim > 96:
        if groups >= _LDS_MANY_GROUPS_WIDE_HEADS:
            return True
        if groups >= _LDS_MIN_GROUPS:
            return mean_keys >= _LDS_MIN_MEAN_KEYS_WIDE_HEADS
        return groups >= _LDS_MIN_GROUPS_WIDE_HEADS and mean_keys >= _LDS_MIN_MEAN_KEYS
    if groups >= _LDS_MIN_GROUPS and mean_keys >= _LDS_MIN_MEAN_KEYS:
        return True
    # Between 512 and 768 workgroups, whole prefill passes at the 1B sizes (one prompt from position 0):
    # 2,048 tokens (512 workgroups) 5.74 ms with the one-wavefront kernel against 6.03, but 2,304 tokens
    # 7.15 against 6.90, 2,560 7.66 against 7.36, 2,816 8.58 against 8.08.
    return groups >= _LDS_SOME_GROUPS and mean_keys >= _LDS_SOME_GROUPS_MEAN_KEYS


def _cut_keys(want: int, max_context: int, max_splits: int) -> tuple:
    """``max_context`` keys in at most ``min(want, max_splits)`` ranges of a multiple of 32 keys."""
    splits = min(want, max_splits)
    if splits <= 1:
        return 1, 0
    per = ((max_context + splits - 1) // splits + 31) // 32 * 32
    splits = (max_context + per - 1) // per      # rounding up the range never adds a range
    return (splits, per) if splits > 1 else (1, 0)


def _cut_keys_by_fours(want: int, max_context: int):
    """``max_context`` keys in at most ``want`` (a multiple of four) ranges of a multiple of 32
    keys, their number a multiple of four: the last three at most hold no key, never a whole
    workgroup of four.  None below 8 ranges."""
    per = ((max_context + want - 1) // want + 31) // 32 * 32
    n = ((max_context + per - 1) // per + 3) // 4 * 4
    return (n, per) if n >= 8 else None


def choose_splits(num_items: int, num_kv_heads: int, max_context: int, max_splits: int = None,
                  decoding: bool = False, merged_by_fours: bool = False) -> tuple:
    """(splits, keys_per_split) for the matrix-core kernel; never more splits than the kernels
    and their merge take (``max_splits``, by default what the library says).  ``decoding``: the
    items are decoded tokens (one row tile each); ``merged_by_fours``: four ranges at a time are
    added up by their own workgroup, so the merge kernel's limit of ranges a row does not hold."""
    if max_splits is None:
        max_splits = K.attention_max_splits()
    waves = max(1, num_items * num_kv_heads)
    target, least = _TARGET_WAVES, _MIN_KEYS_PER_SPLIT
    if decoding:
        if waves >= _UNSPLIT_WAVES_DECODE:
            return 1, 0
        target = _TARGET_WAVES_DECODE
        least = _MIN_KEYS_PER_SPLIT_DECODE if max_context <= _LONG_CONTEXT_DECODE else _MIN_KEYS_PER_SPLIT
    want = max(1, target // waves)
    if decoding:
        if not merged_by_fours:
            want = min(want, max(_MAX_SPLITS_DECODE, _MIN_WAVES_DECODE // waves))
    most = max(1, (max_context + least - 1) // least)
    return _cut_keys(min(want, most), max_context, max_splits)


# Wavefronts of one workgroup that take neighbouring key ranges of a decoded token and add their
# results up themselves (ops.kernels.attention_mfma, ``waves``).  Where two or four ranges are all
# there are, no partial result is written and no merge kernel runs: whole decode steps at 768 keys,
# 1B sizes, 32 requests (four ranges) 1.246 -> 1.188 ms, 48 requests (unsplit before) 1.293 -> 1.259;
# 17 / 24 / 56 requests 1.125 / 1.192 / 1.381 -> 1.098 / 1.139 / 1.356, 20 requests at 200 keys 1.061 ->
# 1.018, 24 at 4,096 keys 1.568 -> 1.503, 48 at 2,048 / 8,192 keys (unsplit before, one wavefront on
# all keys of a request) 1.722 / 3.709 -> 1.631 / 3.229; so between 128 and 512 (item, kv head) pairs
# the keys go in four ranges, whatever the wavefront count asked for, and from 4,096 keys on up to
# 1,100 pairs (64 requests at 4,096 / 8,192 keys 2.57 / 4.08 -> 2.52 / 3.86 ms, 128 at 4,096 4.32 ->
# 4.27; but 128 at 768 keys 2.03 -> 2.11).  With more ranges than four it pays only where the merge kernel has much to
# read: 8 requests at 8,192 / 32,768 keys (16 ranges of 512 / 2,048 keys) 1.156 / 2.167 -> 1.135 /
# 2.134 ms, one request at 8,192 keys (64 ranges) 0.755 -> 0.740; but 8 requests at 768 / 2,048 /
# 4,096 keys 0.846 / 0.932 / 1.024 -> 0.852 / 0.942 / 1.037 and one request at 768 keys 0.688 -> 0.705.
# (Eight requests at 2,048 / 4,096 keys were measured again after the kernels had changed, together with
# three to fifteen requests: see _SHARED_FEW_FROM.)
_SHARED_MAX_HEAD_DIM = 128
# Head size 128 (8 layers of the 8B sizes, ms a step, one wavefront a range -> this rule): 24 / 32
# requests at 768 keys 1.194 / 1.213 -> 1.147 / 1.177 and 24 at 8,448 keys 2.281 -> 2.161, but 48
# requests (384 pairs, unsplit before) 1.324 -> 1.373 and 3.109 -> 3.176, and 8 requests at 8,448 keys
# in 16 ranges, four to a workgroup, 1.319 -> 1.337: there the four ranges ended at 384 pairs and many
# ranges keep a wavefront each.  Measured again from 20 to 47 requests (8 layers of the 3B / 8B sizes,
# four ranges in a workgroup against what else is chosen - two ranges in a workgroup or three with
# the merge kernel): up to 24 requests the four win (3B, 20 / 24 requests at 700 keys 0.848 / 0.869
# -> 0.821 / 0.831 ms, at 2,000 keys 1.010 / 1.060 -> 0.972 / 1.009), at 28 and 32 a tie, from 33 on
# they lose (3B, 36 / 44 requests at 700 keys 0.974 / 1.001 -> 0.954 / 0.952, 33 / 40 / 47 at 2,000 keys
# 1.287 / 1.320 / 1.365 -> 1.211 / 1.268 / 1.331, at 8,100 keys 2.21 / 2.38 / 2.50 -> 2.08 / 2.32 / 2.47;
# 8B 1-4 % alike): they end at 256 pairs.  What followed them there was three ranges and the merge
# kernel, or two ranges in a workgroup; a wavefront on all keys of its pair, as from 384 pairs on, is
# ahead of both (33 / 40 / 47 requests, three or two ranges -> one: 3B at 700 keys 0.940 / 0.972 / 0.966 ->
# 0.904 / 0.925 / 0.961, at 2,000 keys 1.217 / 1.275 / 1.346 -> 1.223 / 1.247 / 1.318, at 8,100 keys
# 2.09 / 2.31 / 2.48 -> 2.13 / 2.26 / 2.40; 8B 1.27 / 1.30 / 1.27 -> 1.21 / 1.26 / 1.26, 1.49 / 1.54 / 1.63
# -> 1.47 / 1.49 / 1.62, 2.46 / 2.59 / 2.79 -> 2.41 / 2.54 / 2.70).
_SHARED_TUNED_HEAD_DIM = 64
_SHARED_FOUR_BELOW_WIDE = 257
# ... and at short contexts they begin at 128 pairs, not at 64: 8 / 12 / 16 requests at 700 keys, 16-8
# ranges with the merge kernel -> four in a workgroup, 3B 0.635 / 0.667 / 0.701 -> 0.639 / 0.676 / 0.694,
# 8B 0.953 / 1.024 / 1.113 -> 0.960 / 1.040 / 1.095 ms
_SHARED_FOUR_FROM_SHORT_WIDE = 127
_SHARED_FOUR_FROM = 128             # more (item, kv head) pairs than this ...
_SHARED_FOUR_BELOW = 512            # ... and fewer than this: four ranges in one workgroup
_SHARED_SHORT_CONTEXT = 1024        # up to this many keys already from ...
_SHARED_FOUR_FROM_SHORT = 63        # ... this many pairs (8 / 12 / 16 requests at 768 keys 0.854 / 0.912 / 0.959 ->
                                    # 0.852 / 0.900 / 0.945 ms; but 8 at 2,048 keys 0.930 -> 0.978, 16 at 8,192 1.56 -> 1.73)
_SHARED_LONG_CONTEXT = 4096         # from this many keys on ...
_SHARED_FOUR_BELOW_LONG = 1100      # ... up to this many pairs
_SHARED_MIN_KEYS = 512              # many ranges: wavefronts share a workgroup from this many keys a range ...
_SHARED_MIN_SPLITS = 64             # ... or from this many ranges
_SHARED_MANY = 16                   # (8 ranges in two workgroups of four: 16 requests at 8,192 keys 1.550 -> 1.561 ms)
_SHARED_MIN_WORKGROUPS = 192
_SHARED_FEW_BYTES_CONTEXT = 8192
# Between 16 and 128 pairs (three to fifteen requests on 8 kv heads) at contexts above 2,048 keys, and from
# 48 pairs on above 1,024: four ranges to a workgroup and one workgroup per compute unit at most (a
# 257th waits for a unit to come free: 7 requests at 8,100 keys in 20 ranges, 280 workgroups, 1.134
# -> 1.237 ms; in 16 ranges, 224 workgroups, 1.111).  Whole decode steps, a wavefront a range -> this,
# 3 / 4 / 5 / 6 / 7 requests: at 8,100 keys 1.008 / 1.034 / 1.047 / 1.087 / 1.134 -> 0.962 / 1.010 / 1.047 /
# 1.086 / 1.111 ms, at 4,000 keys 0.884 / 0.924 / 0.947 / 0.984 / 1.000 -> 0.880 / 0.908 / 0.927 / 0.971 /
# 0.982, at 2,000 keys 0.844 / 0.855 / 0.874 / 0.900 / 0.915 -> 0.850 / 0.867 / 0.886 / 0.884 / 0.894 (so
# from 6 requests there), at 768 keys 0.825 / 0.828 / 0.830 / 0.837 / 0.845 -> 0.836 / 0.848 / 0.847 /
# 0.848 / 0.851 (so not there).  The same up to 127 pairs (8 / 10 / 12 / 14 requests: at 2,000 keys 0.927 /
# 0.982 / 1.025 / 1.044 -> 0.906 / 0.970 / 0.998 / 1.026, at 4,000 keys 1.025 / 1.088 / 1.126 / 1.185 -> 1.001 /
# 1.094 / 1.117 / 1.164, at 8,100 keys 12 / 14 requests 1.369 / 1.471 -> 1.359 / 1.445); at 128 pairs (16
# requests) 1.079 -> 1.063 at 2,000 keys but 1.204 / 1.530 -> 1.215 / 1.538 at 4,000 / 8,100: not there.
_COMPUTE_UNITS = 256
_SHARED_FEW_FROM = 16
_SHARED_FEW_BELOW = 128
_SHARED_FEW_CONTEXT = 2048
_SHARED_FEW_PAIRS_MID = 48


# Long contexts, 17 to 63 requests on 8 kv heads: a workgroup of four ranges per (request, kv head)
# pair is 136-504 workgroups, and the step waits for the compute units that got one more than the
# others (264 workgroups: 8 units stream two pairs' keys while 248 stream one).  Two or three
# workgroups a pair even that out at the price of partial results and the merge kernel.  Whole
# decode steps at 8,100 keys, ms, one / two / three workgroups a pair: 17 requests 1.872 / 2.004 /
# 1.800, 24: 1.974 / 2.100 / 2.180, 33: 2.914 / 2.720 / 2.640, 40: 3.045 / 2.840 / 2.808, 48: 3.170 /
# 3.136 / 3.190, 56: 3.404 / 3.560 / 3.630; at 4,000 keys 17: 1.425 / 1.522 / 1.454, 33: 1.997 / 1.944 /
# 1.984, 40: 2.062 / 2.021 / 2.104, 48: 2.140 / 2.139 / 2.305.  What fits them: the share of compute
# units' turns that are used, workgroups / (256 * turns), divided by a price of 1 / 1.25 / 1.4 (up to
# 4,096 keys, where the rest of the step weighs more: 1 / 1.3 / 1.6); the largest wins.  Checked at
# batch sizes that were not used for it, four ranges a pair -> this: 18 / 36 / 44 requests at 8,100 keys
# 1.866 / 2.965 / 3.135 -> 1.823 / 2.716 / 2.938 ms (20: 1.893 -> 1.909), at 16,000 keys 18 / 20 / 36 / 44:
# 2.761 / 2.828 / 4.920 / 5.312 -> 2.559 / 2.705 / 4.316 / 4.762, at 4,000 keys 36 / 44: 2.025 / 2.125 ->
# 1.988 / 2.075; 22, 28 and 52 requests keep one workgroup a pair.
# Below 4,096 keys one workgroup a pair stays: two / three at 768 keys took 33-56 requests from 1.22-1.35
# to 1.28-1.45 / 1.30-1.52 ms, at 2,000 keys from 1.51-1.71 to 1.52-1.81 / 1.50-1.83.
# From 512 pairs on (64 requests and more) two workgroups a pair at 8,100 keys: 72 / 104 requests 4.73 /
# 6.12 -> 4.54 / 5.98 ms, 80 a tie, 64 / 88 / 120 slower by 2-3 %; at 4,000 keys nothing gained: one stays.
_GROUP_PRICE_LONG = (1.0, 1.25, 1.4)
_GROUP_PRICE = (1.0, 1.3, 1.6)


def _workgroups_a_pair(pairs: int, max_context: int) -> int:
    price = _GROUP_PRICE if max_context <= _SHARED_LONG_CONTEXT else _GROUP_PRICE_LONG
    best, best_score = 1, 0.0
    for groups, cost in enumerate(price, start=1):
        workgroups = pairs * groups
        turns = (workgroups + _COMPUTE_UNITS - 1) // _COMPUTE_UNITS
        score = workgroups / (turns * _COMPUTE_UNITS) / cost
        if score > best_score * 1.0001:
            best, best_score = groups, score
    return best


def choose_decode_ranges(num_items: int, num_kv_heads: int, max_context: int, head_dim: int,
                         max_splits: int = None) -> tuple:
    """(key ranges, keys per range, wavefronts per workgroup) for decoded tokens."""
    pairs = max(1, num_items * num_kv_heads)
    below = _SHARED_FOUR_BELOW if max_context < _SHARED_LONG_CONTEXT else _SHARED_FOUR_BELOW_LONG
    wide = head_dim > _SHARED_TUNED_HEAD_DIM
    if wide:
        below = _SHARED_FOUR_BELOW_WIDE
    frm = _SHARED_FOUR_FROM_SHORT if max_context <= _SHARED_SHORT_CONTEXT else _SHARED_FOUR_FROM
    if wide and frm < _SHARED_FOUR_FROM_SHORT_WIDE:
        frm = _SHARED_FOUR_FROM_SHORT_WIDE
    if not wide and _SHARED_FOUR_FROM < pairs < _SHARED_FOUR_BELOW and max_context >= _SHARED_LONG_CONTEXT:
        groups = _workgroups_a_pair(pairs, max_context)
        cut = _cut_keys_by_fours(4 * groups, max_context) if groups > 1 else None
        if cut is not None:
            return cut[0], cut[1], 4
    if head_dim <= _SHARED_MAX_HEAD_DIM and frm < pairs < below \
            and max_context >= 4 * _MIN_KEYS_PER_SPLIT_DECODE:
        splits, per = _cut_keys(4, max_context, 4)
        if splits in (2, 4):
            return splits, per, splits
    if not wide and _SHARED_FEW_FROM < pairs < _SHARED_FEW_BELOW and (
            max_context > _SHARED_FEW_CONTEXT or (max_context > _SHARED_SHORT_CONTEXT and pairs >= _SHARED_FEW_PAIRS_MID)):
        # three to fifteen requests: as many workgroups of four ranges as there are compute units, no more
        parts = min(_COMPUTE_UNITS // pairs, max_context // _MIN_KEYS_PER_SPLIT_DECODE // 4)
        cut = _cut_keys_by_fours(4 * parts, max_context) if parts >= 2 else None
        if cut is not None:
            return cut[0], cut[1], 4
    if head_dim <= _SHARED_MAX_HEAD_DIM and not wide:
        # many ranges, four to a workgroup - if that still leaves a workgroup for most compute units
        # (one request at 32,768 / 131,072 keys: 64 ranges in 128 workgroups 0.979 / 1.616 ms, 128
        # ranges in 256 workgroups 0.918 / 1.344, 64 ranges of one wavefront each 0.950 / 1.427) or the
        # context is short enough for its bytes not to matter (one request at 8,192 keys, 64 ranges:
        # 0.755 -> 0.740)
        splits, per = choose_splits(num_items, num_kv_heads, max_context, max_splits, decoding=True,
                                    merged_by_fours=True)
        if splits % 4 == 0 and splits >= _SHARED_MANY and (per >= _SHARED_MIN_KEYS or splits >= _SHARED_MIN_SPLITS) \
                and (pairs * (splits // 4) >= _SHARED_MIN_WORKGROUPS or max_context <= _SHARED_FEW_BYTES_CONTEXT):
            return splits, per, 4
    if wide and head_dim <= _SHARED_MAX_HEAD_DIM and pairs >= _SHARED_FOUR_BELOW_WIDE:
        return 1, 0, 1
    splits, per = choose_splits(num_items, num_kv_heads, max_context, max_splits, decoding=True)
    waves = splits if splits in (2, 4) and head_dim <= _SHARED_MAX_HEAD_DIM else 1
    return splits, per, waves


# One or two decoded tokens whose output projection adds partial results up itself
# (ops.kernels.gemv_merged): four ranges to a workgroup and one partial result per workgroup, so the
# merge kernel (3.7 us a layer for kilobytes) is not launched.  Whole decode steps at the 1B sizes,
# ms, merge kernel -> this: one request at 400 / 768 / 1,900 keys 0.686 / 0.688 / 0.703 -> 0.667 / 0.660 /
# 0.681, two requests at 768 / 1,900 keys 0.769 / 0.783 -> 0.741 / 0.766.  Up to 2,048 keys (contexts are
# rounded up to a power of two when a step is captured): with at most 4 partial results a row 4,096
# keys are 16 ranges of 256, and one request at 3,000 / 8,000 keys went 0.719 / 0.741 -> 0.722 / 0.805.
# With 8 partial results a row, which the consumer has room for with one token only, 2,049-4,096 keys are
# 32 ranges of 128: one request at 3,000 keys 0.720 -> 0.698 (two: 0.797 -> 0.798; 8,000 keys: 0.742 -> 0.746).
# Head sizes up to 64, where it was measured (at 128, with wider output projections: parts/linear.py).
_LEFT_MAX_ITEMS = 2
_LEFT_MIN_KEYS = 64
_LEFT_MAX_CONTEXT = 2048
_LEFT_PARTS_SHORT = 4             # up to 2,048 keys: at most 16 ranges
_LEFT_MAX_CONTEXT_ONE = 4096      # one token, a consumer that takes 8 partial results: 32 ranges up to here


def choose_left_ranges(num_items: int, max_context: int, head_dim: int, max_parts: int):
    """(key ranges, keys per range, 4) for decoded tokens whose consumer takes up to ``max_parts``
    partial results a row, or None where the ordinary choice stands."""
    if num_items > _LEFT_MAX_ITEMS or head_dim > _SHARED_TUNED_HEAD_DIM or max_parts < 2:
        return None
    if max_context <= _LEFT_MAX_CONTEXT:
        max_parts = min(max_parts, _LEFT_PARTS_SHORT)
    elif num_items > 1 or max_context > _LEFT_MAX_CONTEXT_ONE or max_parts <= _LEFT_PARTS_SHORT:
        return None
    # a multiple of four ranges whatever the context: the last ones may hold few keys or none (a
    # range without a key weighs nothing when the results are added up)
    want = min(4 * max_parts, max_context // _LEFT_MIN_KEYS) // 4 * 4
    if want < 8:
        return None
    per = ((max_context + want - 1) // want + 31) // 32 * 32
    return want, per, 4


def choose_lds_splits(groups: int, max_context: int, max_splits: int = None, head_dim: int = 64) -> tuple:
    """(splits, keys_per_split) for the workgroup kernel, under the same limit."""
    if max_splits is None:
        max_splits = K.attention_max_splits()
    wide = head_dim > 96
    want = max(1, (_LDS_TARGET_GROUPS_WIDE_HEADS if wide else _LDS_TARGET_GROUPS) // max(1, groups))
    min_keys = _LDS_MIN_KEYS_PER_SPLIT_WIDE_HEADS if wide else _LDS_MIN_KEYS_PER_SPLIT
    return _cut_keys(min(want, max(1, max_context // min_keys)), max_context, max_splits)


def _plan_for(batch, kv, num_q_heads: int, num_kv_heads: int, head_dim: int, max_parts: int = 0) -> list:
    plans = batch.attention_plans
    key = (num_q_heads, num_kv_heads, head_dim, kv.page_size, max_parts)
    plan = plans.get(key)
    if plan is None:
        plan = plans[key] = _plan(batch, num_q_heads // num_kv_heads, num_kv_heads, head_dim, kv.page_size, max_parts)
    return plan


def rotates_in_kernel(batch, kv, num_q_heads: int, num_kv_heads: int, head_dim: int, dtype) -> bool:
    """Whether :func:`paged_attention` can take the joined projection as the product left it and
    do rotation and cache write itself (``rope=...``): a bfloat16 step of decoded tokens only, a
    geometry the kernel takes, every token one work item whose record the host could make."""
    if kv is None or dtype != torch.bfloat16 or batch.max_q_len != 1 or num_q_heads % num_kv_heads:
        return False
    if not K.attention_mfma_rope_supported(head_dim, kv.page_size, num_q_heads // num_kv_heads):
        return False
    plan = _plan_for(batch, kv, num_q_heads, num_kv_heads, head_dim)
    return len(plan) == 1 and plan[0][0] == "wave" and plan[0][1][2] is not None


def paged_attention(qkv: torch.Tensor, out: torch.Tensor, kv, batch, num_q_heads: int,
                    num_kv_heads: int, head_dim: int, scale: float, window: int = 0, rope=None,
                    max_parts: int = 0):
    """Causal GQA attention of the step's tokens over the paged cache.  ``qkv`` is the fused
    projection output ``[T, (nq + 2 nkv) d]`` (or just its Q part) whose first ``nq * d`` columns
    are the (already position-encoded) queries; keys and values are read from ``kv``.

    bf16 runs on the matrix cores.  Decoded tokens (at most 16 query rows per kv head) take the
    one-wavefront kernel with their keys split over wavefronts; prompt portions take the
    workgroup kernel that shares key blocks through LDS when there is enough of them to fill the
    chip, else the one-wavefront kernel with two row tiles.  A step that holds both is two
    launches, each over its own entries.  Which kernels, over which work items and key splits, is
    decided once per step and geometry (every layer of a model asks the same) and kept with the
    batch.

    ``max_parts`` > 0: the caller can take the output of one or two decoded tokens as up to so
    many partial results a row (``ops.kernels.AttentionPartials``, returned instead of ``out``,
    which is then not written) - where the keys are cut that way no merge kernel runs."""
    if kv is None:
        raise K.KernelError("paged_attention: the mixer has no cache view")
    if rope is not None:
        # decoded tokens whose rotation and cache write are still to be done: ``rope`` = (cos, sin)
        # tables or (None, None); only where rotates_in_kernel() said yes
        if not rotates_in_kernel(batch, kv, num_q_heads, num_kv_heads, head_dim, qkv.dtype):
            raise K.KernelError("paged_attention: this step cannot rotate inside the attention kernel")
        (_, (_, _, meta), _, splits, per, _, _, keep_cached, waves), = _plan_for(batch, kv, num_q_heads, num_kv_heads, head_dim)
        return K.attention_mfma_rope(qkv, out, kv.k_cache, kv.v_cache, kv.block_table, meta, num_q_heads,
                                     num_kv_heads, head_dim, scale, rope[0], rope[1],
                                     kv.slot_mapping if kv.writes else None, window, splits, per, keep_cached, waves)
    if not (qkv.dtype == torch.bfloat16 and K.attention_mfma_supported(head_dim, kv.page_size)
            and qkv.shape[1] % 8 == 0):
        return K.attention_rowwise(qkv, qkv.shape[1], out, kv.k_cache, kv.v_cache, kv.block_table,
                                   batch.tok_seat, batch.positions, num_q_heads, num_kv_heads,
                                   head_dim, scale, window)
    plan = _plan_for(batch, kv, num_q_heads, num_kv_heads, head_dim, max_parts)
    stride = qkv.shape[1]
    for launch in plan:
        if launch[0] == "wave":
            _, (item_entry, item_row0, meta), tiles, splits, per, pair, covers_all, keep_cached, waves = launch
            left = max_parts > 0 and len(plan) == 1 and covers_all and 2 <= splits // waves <= max_parts
            got = K.attention_mfma(qkv, stride, out, kv.k_cache, kv.v_cache, kv.block_table, item_entry, item_row0,
                                   batch.entry_seat, batch.entry_q_start, batch.entry_start_pos, num_q_heads,
                                   num_kv_heads, head_dim, scale, window, splits, per, tiles, pair, meta,
                                   covers_all_rows=covers_all, keep_cached=keep_cached, waves=waves,
                                   leave_partials=left)
            if left:
                return got
        else:
            _, meta, splits, per, covers_all = launch
            K.attention_lds(qkv, stride, out, kv.k_cache, kv.v_cache, kv.block_table, meta, num_q_heads,
                            num_kv_heads, head_dim, scale, window, False, splits, per, covers_all_rows=covers_all)
    return out


def _plan(batch, group: int, num_kv_heads: int, head_dim: int, page_size: int, max_parts: int = 0) -> list:
    """The launches of one attention call over ``batch``: ("wave", items, row tiles, splits, keys per
    split, pair, covers all rows, keep cached, wavefronts of a workgroup that share an item) and
    ("lds", item records, splits, keys per split, covers all rows)."""
    plan = []

    def decoded(which):
        items = batch.attention_items(group, 1, which)
        n = items[0].shape[0]
        # a few short contexts: what this call reads is small enough to still be in the
        # memory-side cache at the next step if it is let in (whole steps of the 1B shape, 8 requests
        # of 768 keys, 12.6 MB a layer: 0.913 -> 0.902 ms; 8 of 8,192, 134 MB a layer: 1.27 -> 1.30,
        # so only the small ones)
        small = n * batch.max_context * num_kv_heads * head_dim * 4 <= _KEEP_CACHED_BYTES
        splits, per, waves = choose_decode_ranges(n, num_kv_heads, batch.max_context, head_dim)
        if max_parts > 0 and which == "all":
            splits, per, waves = choose_left_ranges(batch.num_tokens, batch.max_context, head_dim, max_parts) \
                or (splits, per, waves)
        # (not where wavefronts share a workgroup: 8 / 16 / 32 requests of 768 keys in four ranges
        # 0.854 / 0.942 / 1.154 ms through the caches, 0.848 / 0.938 / 1.124 past them; 4 requests of
        # 2,048 keys, a wavefront a range, 0.863 against 0.875)
        small = small and waves == 1
        plan.append(("wave", items, 1, splits, per, False, which == "all", small, waves))

    if batch.max_q_len * group <= 16:
        decoded("all")
        return plan
    mixed = batch.min_q_len * group <= 16
    which = "long" if mixed else "all"
    done = False
    if K.attention_lds_supported(head_dim, page_size):
        items = batch.attention_items(group, 8, which)
        groups = items[0].shape[0] * num_kv_heads
        if items[2] is not None and use_lds_kernel(groups, batch.mean_keys_of_long_entries(), head_dim):
            splits, per = choose_lds_splits(groups, batch.max_context, head_dim=head_dim)
            plan.append(("lds", items[2], splits, per, which == "all"))
            done = True
    if not done:
        # two row tiles per wave, so each key and value loaded serves 32 query rows; whole key
        # ranges as long as that gives a wave per SIMD
        tiles = K.attention_mfma_row_tiles(head_dim, True)
        items = batch.attention_items(group, tiles, which)
        waves = items[0].shape[0] * num_kv_heads
        if waves >= _WIDE_MIN_WAVES:
            # items come ordered by work: a wavefront that takes the i-th and the i-th last does
            # about the average; worth it while every SIMD still gets a wavefront
            plan.append(("wave", items, tiles, 1, 0, waves >= _PAIR_MIN_WAVES, which == "all", False, 1))
        else:
            # too few items to fill the chip: the keys are split over wavefronts as well (portions
            # of 256 tokens late in an 8,192-token prompt: 16 % faster than one row tile per wave)
            splits, per = choose_splits(items[0].shape[0], num_kv_heads, batch.max_context)
            plan.append(("wave", items, tiles, splits, per, False, which == "all", False, 1))
    if mixed:
        decoded("short")
    return plan
