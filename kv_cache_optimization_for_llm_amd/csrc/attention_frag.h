// Register fragments of the bf16 matrix-core attention kernels (gfx950).
#pragma once
#include "common.h"

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 b16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 b16x2 __attribute__((ext_vector_type(2)));

// 8 bf16 = one operand of mfma_f32_16x16x32_bf16
union Frag8 {
    b16x8 v;
    uint4 u4;
    uint2 u2[2];
    uint16_t h[8];
    b16x2 p2[4];
};

// 4 bf16 = one operand of mfma_f32_16x16x16bf16_1k
union Frag4 {
    s16x4 v;
    uint2 u2;
    uint16_t h[4];
};

// two floats -> two bf16, round to nearest even (one v_cvt_pk_bf16_f32)
__device__ inline b16x2 pack_bf16(float a, float b) {
    return __builtin_convertvector(f32x2{a, b}, b16x2);
}

// The values of a lane's four keys (4 bf16 = 8 bytes of a V^T operand), of which only the first
// `n` hold something this request wrote: the others are set to zero.  A position past a request's
// newest token belongs to the page but was written by the page's previous owner, or never; its
// probability is exactly zero, and zero times whatever lies there must stay zero (0 x NaN is not).
__device__ inline uint2 keep_first_keys(uint2 v, int n) {
    const uint64_t mask = n >= 4 ? ~0ull : (n <= 0 ? 0ull : ((1ull << (16 * n)) - 1ull));
    return make_uint2(v.x & (uint32_t)mask, v.y & (uint32_t)(mask >> 32));
}

// Most key splits the attention kernels and their merge take (the merge keeps one weight per
// split in LDS).  The host's split policy asks kva_attention_max_splits() for it.
#define MERGE_MAX_SPLITS 256

// attention_mfma.hip: merge of key-split partials (see there)
int kva_attention_merge_launch(void *out, const float *part_o, const float *part_ml, int head_dim, int splits,
                               const int *item_meta, const int *item_entry, const int *item_row0,
                               const int *entry_q_start, int num_items, int rows_per_item, int total_rows,
                               int num_q_heads, int num_kv_heads, int all_rows, hipStream_t stream);
