// Causal grouped-query attention over the paged cache on the matrix cores (bf16, gfx950).
//
// One kernel serves prompt portions and decoded tokens.  Work is cut into ITEMS: an item is 16
// consecutive "query rows" of one request and one kv head, where row = token_in_step * G + g
// enumerates (token, query head of the kv head's group) pairs, G = num_q_heads / num_kv_heads.
// A decoded token of a model with G <= 16 is one item; a prompt portion of n tokens is
// ceil(n * G / 16) items.  One 64-lane wavefront runs one (item, kv head, key split).
//
// Everything is computed transposed so that no operand ever has to change layout:
//     S^T = K  * Q^T     A = K rows (16 keys x head-dim slice), B = Q^T  -> lane holds, for its
//                        own query row (lane % 16), 4 keys (4 * (lane / 16) + i) of the key tile
//     O^T = V^T * P^T    A = V^T (16 value dims x 32 keys), B = P^T taken straight from the
//                        registers S^T came out in
// The matrix-core k index of the second product is a permutation of the 32 keys of a block
// (lane group g, element j <-> key (j / 4) * 16 + 4 g + j % 4); it is applied to V^T's loads,
// which is free because V pages are stored transposed ([kv_head, head_dim, page_size]) and a
// lane's 4 keys are 8 contiguous bytes.  K is loaded straight from the page
// ([kv_head, page_size, head_dim]) in operand layout too, so there is no LDS and no barrier.
//
// Softmax is online in fp32 per query row (running max m, denominator l), scores scaled after
// the product; P is rounded to bf16 for the second product, the accumulator stays fp32.  Keys
// are visited in blocks of 32 aligned to absolute positions.  With `splits` > 1 each split
// writes an un-normalised partial (o, m, l) and attention_merge combines them (flash-decoding);
// with one split the normalised result is written directly.
//
// Reference: same recurrence as paged_attention/src/kernels.cu:150-219 and the tiled prefill
// kernel base/src/kernels.cu:361-466, which work one key at a time on CUDA cores.
#include "common.h"
#include <math.h>

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 b16x8 __attribute__((ext_vector_type(8)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

union Frag8 {
    b16x8 v;
    s16x8 s;
    uint4 u4;
    uint2 u2[2];
    uint16_t h[8];
};
union Frag4 {
    s16x4 v;
    uint2 u2;
    uint16_t h[4];
};

template <int D>
__global__ void __launch_bounds__(KVA_WAVE)
attention_mfma_kernel(bf16_t *__restrict__ out, float *__restrict__ part_o, float *__restrict__ part_ml,
                      const bf16_t *__restrict__ q, int q_row_stride,
                      const bf16_t *__restrict__ k_cache, const bf16_t *__restrict__ v_cache,
                      const int *__restrict__ block_table, int max_blocks,
                      const int *__restrict__ item_entry, const int *__restrict__ item_row0,
                      const int *__restrict__ entry_seat, const int *__restrict__ entry_q_start,
                      const int *__restrict__ entry_start_pos, int num_q_heads, int num_kv_heads,
                      int page_size, float scale, int window, int splits, int keys_per_split) {
    constexpr int KSTEP = (D % 32 == 0) ? 32 : 16;   // head-dim slice per S^T product
    constexpr int NKS = D / KSTEP;
    constexpr int NDT = D / 16;                      // 16-wide tiles of the value dimension

    const int item = blockIdx.x, kvh = blockIdx.y, split = blockIdx.z;
    const int lane = threadIdx.x, r = lane & 15, g = lane >> 4;
    const int G = num_q_heads / num_kv_heads;

    const int e = item_entry[item];
    const int row0 = item_row0[item];
    const int q_start = entry_q_start[e];
    const int q_len = entry_q_start[e + 1] - q_start;
    const int start_pos = entry_start_pos[e];
    const int *bt = block_table + (size_t)entry_seat[e] * max_blocks;
    const int M = q_len * G;

    const int row = row0 + r;
    const bool row_valid = row < M;
    const int tq = row_valid ? row / G : 0;
    const int hg = row_valid ? row % G : 0;
    const int head = kvh * G + hg;
    const int my_pos = start_pos + tq;
    const int my_lo = (window > 0 && my_pos - window + 1 > 0) ? my_pos - window + 1 : 0;

    // keys any row of this item may see
    const int last_row = (row0 + 15 < M - 1) ? row0 + 15 : M - 1;
    const int item_hi = start_pos + last_row / G;                       // inclusive
    const int item_pos_lo = start_pos + row0 / G;
    const int item_lo = (window > 0 && item_pos_lo - window + 1 > 0) ? item_pos_lo - window + 1 : 0;
    int k_begin = item_lo & ~31;
    int k_end = item_hi + 1;                                            // exclusive
    if (splits > 1) {
        const int s_lo = split * keys_per_split, s_hi = s_lo + keys_per_split;
        if (s_lo > k_begin) k_begin = s_lo;
        if (s_hi < k_end) k_end = s_hi;
    }

    // Q^T operand: lane (r, g) holds Q[row r][ks * KSTEP + g * KSTEP/4 ...]
    Frag8 qf8[NKS];
    Frag4 qf4[NKS];
    {
        const bf16_t *qrow = q + (size_t)(q_start + tq) * q_row_stride + (size_t)head * D;
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
            if (KSTEP == 32) {
                qf8[ks].u4 = row_valid ? *reinterpret_cast<const uint4 *>(qrow + ks * 32 + g * 8)
                                       : make_uint4(0, 0, 0, 0);
            } else {
                qf4[ks].u2 = row_valid ? *reinterpret_cast<const uint2 *>(qrow + ks * 16 + g * 4)
                                       : make_uint2(0, 0);
            }
        }
    }

    float m = -INFINITY, l = 0.f;
    f32x4 o[NDT];
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};

    // K operand of one 32-key block: lane (r, g) holds K[key kstart + t*16 + r][ks*KSTEP + g*KSTEP/4 ..]
    Frag8 kf8[2][NKS];
    Frag4 kf4[2][NKS];
    auto load_k = [&](int kstart) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int key = kstart + t * 16 + r;
            const bool kvalid = key <= item_hi && key >= item_lo;   // pages outside may be unmapped
            const bf16_t *krow = k_cache;
            if (kvalid) {
                const int page = bt[key / page_size];
                krow += (((size_t)page * num_kv_heads + kvh) * page_size + key % page_size) * D;
            }
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) {
                if (KSTEP == 32)
                    kf8[t][ks].u4 = kvalid ? *reinterpret_cast<const uint4 *>(krow + ks * 32 + g * 8)
                                           : make_uint4(0, 0, 0, 0);
                else
                    kf4[t][ks].u2 = kvalid ? *reinterpret_cast<const uint2 *>(krow + ks * 16 + g * 4)
                                           : make_uint2(0, 0);
            }
        }
    };
    if (k_begin < k_end) load_k(k_begin);

    for (int kstart = k_begin; kstart < k_end; kstart += 32) {
        // ---- V^T operand of this block, issued early so the loads overlap the first product:
        // lane (r, g) supplies V^T[dt * 16 + r][keys kstart + 4g .. +3] and [kstart + 16 + 4g .. +3]
        Frag8 vf[NDT];
        {
            size_t vbase[2];
            bool vvalid[2];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const int key0 = kstart + t * 16 + 4 * g;
                vvalid[t] = key0 <= item_hi && key0 + 3 >= item_lo;
                vbase[t] = 0;
                if (vvalid[t]) {
                    const int page = bt[key0 / page_size];
                    vbase[t] = ((size_t)page * num_kv_heads + kvh) * D * page_size + key0 % page_size;
                }
            }
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
                for (int t = 0; t < 2; ++t)
                    vf[dt].u2[t] = vvalid[t] ? *reinterpret_cast<const uint2 *>(
                                                   v_cache + vbase[t] + (size_t)(dt * 16 + r) * page_size)
                                             : make_uint2(0, 0);
        }
        // ---- S^T for two 16-key tiles
        f32x4 s[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            s[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) {
                if (KSTEP == 32)
                    s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf8[t][ks].v, qf8[ks].v, s[t], 0, 0, 0);
                else
                    s[t] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(kf4[t][ks].v, qf4[ks].v, s[t], 0, 0, 0);
            }
        }
        // the next block's K, in flight during the softmax and the second product
        if (kstart + 32 < k_end) load_k(kstart + 32);
        // ---- mask, scale, online softmax for query row r (its keys are spread over 4 lane groups)
        float sv[8];
        float mloc = -INFINITY;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int key = kstart + t * 16 + 4 * g + i;
                const bool vis = row_valid && key <= my_pos && key >= my_lo;
                const float x = vis ? s[t][i] * scale : -INFINITY;
                sv[t * 4 + i] = x;
                mloc = fmaxf(mloc, x);
            }
        mloc = fmaxf(mloc, __shfl_xor(mloc, 16, KVA_WAVE));
        mloc = fmaxf(mloc, __shfl_xor(mloc, 32, KVA_WAVE));
        const float m_new = fmaxf(m, mloc);
        const float corr = (m_new == -INFINITY) ? 1.f : __expf(m - m_new);
        float lsum = 0.f;
        Frag8 pf;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float p = (sv[j] == -INFINITY) ? 0.f : __expf(sv[j] - m_new);
            lsum += p;
            pf.h[j] = float_to_bf16_bits(p);
        }
        lsum += __shfl_xor(lsum, 16, KVA_WAVE);
        lsum += __shfl_xor(lsum, 32, KVA_WAVE);
        l = l * corr + lsum;
        m = m_new;

        // ---- O^T += V^T * P^T
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) {
            f32x4 acc = o[dt];
            acc[0] *= corr; acc[1] *= corr; acc[2] *= corr; acc[3] *= corr;
            o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dt].v, pf.v, acc, 0, 0, 0);
        }
    }

    // lane (r, g) holds O[row r][dt * 16 + 4g + i]
    if (!row_valid) return;
    const size_t orow = (size_t)(q_start + tq) * num_q_heads + head;
    if (splits == 1) {
        const float inv = 1.f / l;
        bf16_t *dst = out + orow * D;
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) {
            Frag4 w;
#pragma unroll
            for (int i = 0; i < 4; ++i) w.h[i] = float_to_bf16_bits(o[dt][i] * inv);
            *reinterpret_cast<uint2 *>(dst + dt * 16 + 4 * g) = w.u2;
        }
    } else {
        float *dst = part_o + (orow * splits + split) * D;
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt)
            *reinterpret_cast<float4 *>(dst + dt * 16 + 4 * g) =
                make_float4(o[dt][0], o[dt][1], o[dt][2], o[dt][3]);
        if (g == 0) {
            part_ml[(orow * splits + split) * 2] = m;
            part_ml[(orow * splits + split) * 2 + 1] = l;
        }
    }
}

// out[row, :] = sum_s o_s * exp(m_s - M) / sum_s l_s * exp(m_s - M),  M = max_s m_s.
// One wavefront per row: lanes first own splits (max and denominator by wave reduction, the
// weights go to LDS), then own value dimensions and add the weighted partials.
#define MERGE_MAX_SPLITS 256
__global__ void __launch_bounds__(KVA_WAVE)
attention_merge_kernel(bf16_t *__restrict__ out, const float *__restrict__ part_o,
                       const float *__restrict__ part_ml, int head_dim, int splits) {
    __shared__ float w_s[MERGE_MAX_SPLITS];
    const size_t row = blockIdx.x;
    const int lane = threadIdx.x;
    const float2 *ml = reinterpret_cast<const float2 *>(part_ml) + row * splits;
    float M = -INFINITY;
    for (int s = lane; s < splits; s += KVA_WAVE) M = fmaxf(M, ml[s].x);
    M = wave_max(M);
    float denom = 0.f;
    for (int s = lane; s < splits; s += KVA_WAVE) {
        const float2 v = ml[s];
        const float w = (v.x == -INFINITY) ? 0.f : __expf(v.x - M);
        w_s[s] = w;
        denom += v.y * w;
    }
    denom = wave_sum(denom);
    __syncthreads();
    const float inv = 1.f / denom;
    const float *po = part_o + row * splits * head_dim;
    for (int j = lane; j < head_dim; j += KVA_WAVE) {
        float acc = 0.f;
#pragma unroll 8
        for (int s = 0; s < splits; ++s) acc += po[(size_t)s * head_dim + j] * w_s[s];
        out[row * head_dim + j].bits = float_to_bf16_bits(acc * inv);
    }
}

extern "C" int kva_attention_mfma_supported(int head_dim, int page_size) {
    switch (head_dim) {
    case 16: case 32: case 48: case 64: case 80: case 96: case 112: case 128: case 160: case 192:
    case 224: case 256:
        return page_size % 4 == 0 ? 1 : 0;
    default:
        return 0;
    }
}

extern "C" int kva_attention_mfma(void *out, float *part_o, float *part_ml, const void *q,
                                  int q_row_stride, const void *k_cache, const void *v_cache,
                                  const int *block_table, int max_blocks, const int *item_entry,
                                  const int *item_row0, int num_items, const int *entry_seat,
                                  const int *entry_q_start, const int *entry_start_pos, int total_rows,
                                  int num_q_heads, int num_kv_heads, int head_dim, int page_size,
                                  float scale, int window, int splits, int keys_per_split,
                                  hipStream_t stream) {
    KVA_REQUIRE(num_items >= 0 && num_q_heads > 0 && num_kv_heads > 0 && max_blocks > 0,
                "attention_mfma: bad sizes");
    KVA_REQUIRE(num_q_heads % num_kv_heads == 0, "attention_mfma: %d query heads is not a multiple of %d kv heads",
                num_q_heads, num_kv_heads);
    KVA_REQUIRE(kva_attention_mfma_supported(head_dim, page_size),
                "attention_mfma: head_dim %d / page_size %d not supported (head_dim a multiple of 16 up "
                "to 128 or 160/192/224/256, page_size a multiple of 4)", head_dim, page_size);
    KVA_REQUIRE(q_row_stride % 8 == 0, "attention_mfma: query row stride %d must be a multiple of 8", q_row_stride);
    KVA_REQUIRE(splits >= 1 && splits <= MERGE_MAX_SPLITS && num_kv_heads <= 65535,
                "attention_mfma: at most %d splits and 65535 kv heads", MERGE_MAX_SPLITS);
    KVA_REQUIRE(splits == 1 || (keys_per_split > 0 && keys_per_split % 32 == 0 && part_o && part_ml),
                "attention_mfma: splits need a key count that is a multiple of 32 and a workspace");
    KVA_REQUIRE(window >= 0, "attention_mfma: negative window");
    if (num_items == 0) return KVA_OK;
    dim3 grid(num_items, num_kv_heads, splits), block(KVA_WAVE);
#define LAUNCH(DD)                                                                              \
    hipLaunchKernelGGL((attention_mfma_kernel<DD>), grid, block, 0, stream, (bf16_t *)out, part_o, \
                       part_ml, (const bf16_t *)q, q_row_stride, (const bf16_t *)k_cache,        \
                       (const bf16_t *)v_cache, block_table, max_blocks, item_entry, item_row0,  \
                       entry_seat, entry_q_start, entry_start_pos, num_q_heads, num_kv_heads,    \
                       page_size, scale, window, splits, keys_per_split)
    switch (head_dim) {
    case 16: LAUNCH(16); break;
    case 32: LAUNCH(32); break;
    case 48: LAUNCH(48); break;
    case 64: LAUNCH(64); break;
    case 80: LAUNCH(80); break;
    case 96: LAUNCH(96); break;
    case 112: LAUNCH(112); break;
    case 128: LAUNCH(128); break;
    case 160: LAUNCH(160); break;
    case 192: LAUNCH(192); break;
    case 224: LAUNCH(224); break;
    case 256: LAUNCH(256); break;
    default: KVA_REQUIRE(false, "attention_mfma: head_dim %d", head_dim);
    }
#undef LAUNCH
    KVA_CHECK_LAUNCH("attention_mfma");
    if (splits > 1) {
        hipLaunchKernelGGL(attention_merge_kernel, dim3(total_rows), dim3(64), 0, stream, (bf16_t *)out,
                           part_o, part_ml, head_dim, splits);
        KVA_CHECK_LAUNCH("attention_merge");
    }
    return KVA_OK;
}
