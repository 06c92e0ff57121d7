// Causal grouped-query attention over the paged cache: the plain kernel.
//
// One wavefront per (token, query head).  The query at absolute position p of its request
// attends to keys lo..p of the same request (lo = 0, or p - window + 1 with a window), all read
// from the cache through the request's block-table row - the step has already written this
// step's K and V there (the reference also scatters before it attends,
// base/src/engine.cu:726-737).  Same recurrence as the reference's decode kernel
// (paged_attention/src/kernels.cu:150-219): fp32 dot product, score scaled, running max m,
// denominator l and accumulator acc in fp32, out = acc / l.  GQA: kv_head = q_head / (nq / nkv).
//
// K pages are [kv_head, page_size, head_dim]; V pages are stored transposed,
// [kv_head, head_dim, page_size].
//
// Keys are taken in blocks of 64 aligned to absolute positions (0..63, 64..127, ...): lane i of
// the wavefront owns key 64*b + i.  Because the blocks do not depend on where a step starts
// or on what else is in the batch, the fp32 result for a (request, position) is bit-identical
// however the tokens were cut into steps.
//
// This kernel serves the fp32 path and every shape (head_dim any multiple of 4 up to 256);
// the bf16 path uses it where the MFMA kernels do not apply.
#include "common.h"
#include "kv_layout.h"
#include <math.h>

#define ATTN_MAX_HEAD_DIM 256

template <typename T> struct Vec4;
template <> struct Vec4<float> {
    static __device__ inline void load(const float *p, float (&o)[4]) {
        const float4 v = *reinterpret_cast<const float4 *>(p);
        o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
    }
};
template <> struct Vec4<bf16_t> {
    static __device__ inline void load(const bf16_t *p, float (&o)[4]) {
        const uint2 v = *reinterpret_cast<const uint2 *>(p);
        o[0] = bf16_bits_to_float((uint16_t)(v.x & 0xffff));
        o[1] = bf16_bits_to_float((uint16_t)(v.x >> 16));
        o[2] = bf16_bits_to_float((uint16_t)(v.y & 0xffff));
        o[3] = bf16_bits_to_float((uint16_t)(v.y >> 16));
    }
};

template <typename T>
__global__ void __launch_bounds__(KVA_WAVE)
attention_rowwise_kernel(T *__restrict__ out, const T *__restrict__ q, int q_row_stride,
                         const T *__restrict__ k_cache, const T *__restrict__ v_cache,
                         const int *__restrict__ block_table, int max_blocks,
                         const int *__restrict__ tok_seat, const int *__restrict__ tok_pos,
                         int num_q_heads, int num_kv_heads, int head_dim, int page_size,
                         float scale, int window) {
    __shared__ float q_s[ATTN_MAX_HEAD_DIM];
    __shared__ float p_s[KVA_WAVE];
    __shared__ long long voff_s[KVA_WAVE];

    const int t = blockIdx.x;
    const int qh = blockIdx.y;
    const int lane = threadIdx.x;
    const int kvh = qh / (num_q_heads / num_kv_heads);
    const int pos = tok_pos[t];
    const int *bt = block_table + (size_t)tok_seat[t] * max_blocks;

    const T *qrow = q + (size_t)t * q_row_stride + (size_t)qh * head_dim;
    for (int j = lane; j < head_dim; j += KVA_WAVE) q_s[j] = to_float(qrow[j]);
    __syncthreads();

    const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
    float m = -INFINITY, l = 0.f;
    float acc[ATTN_MAX_HEAD_DIM / KVA_WAVE] = {0.f, 0.f, 0.f, 0.f};

    for (int kb = lo / KVA_WAVE; kb <= pos / KVA_WAVE; ++kb) {
        const int key = kb * KVA_WAVE + lane;
        const bool valid = key >= lo && key <= pos;
        float s = -INFINITY;
        long long row_off = 0;
        if (valid) {
            const int page = bt[key / page_size];
            row_off = ((long long)page * num_kv_heads + kvh) * page_size * (long long)head_dim;
            const T *kpage = k_cache + row_off;
            const int krow = key % page_size, kc = kva_k_chunk(head_dim);
            float dot = 0.f;
            for (int j = 0; j < head_dim; j += 4) {
                float kv[4];
                Vec4<T>::load(kpage + kva_k_at(krow, j, page_size, kc), kv);     // (4 elements never straddle a chunk)
                dot += q_s[j] * kv[0];
                dot += q_s[j + 1] * kv[1];
                dot += q_s[j + 2] * kv[2];
                dot += q_s[j + 3] * kv[3];
            }
            s = dot * scale;
        }
        const float m_new = fmaxf(m, wave_max(s));
        const float corr = (m == -INFINITY) ? 0.f : expf(m - m_new);
        const float p = valid ? expf(s - m_new) : 0.f;
        l = l * corr + wave_sum(p);
        m = m_new;
        __syncthreads();  // the previous block's p_s / voff_s have been consumed
        p_s[lane] = p;
        // V is stored transposed inside a page: [page, kv_head, head_dim, page_size]
        voff_s[lane] = valid ? ((long long)bt[key / page_size] * num_kv_heads + kvh) *
                                       (long long)head_dim * page_size + key % page_size
                             : 0;
        __syncthreads();
        const int first = (kb * KVA_WAVE >= lo) ? 0 : lo - kb * KVA_WAVE;
        const int last = (pos - kb * KVA_WAVE < KVA_WAVE - 1) ? pos - kb * KVA_WAVE : KVA_WAVE - 1;
#pragma unroll
        for (int c = 0; c < ATTN_MAX_HEAD_DIM / KVA_WAVE; ++c) {
            const int j = lane + c * KVA_WAVE;
            if (j < head_dim) {
                float a = acc[c] * corr;
                for (int i = first; i <= last; ++i)
                    a += p_s[i] * to_float(v_cache[voff_s[i] + (long long)j * page_size]);
                acc[c] = a;
            }
        }
    }
    T *orow = out + (size_t)t * num_q_heads * head_dim + (size_t)qh * head_dim;
#pragma unroll
    for (int c = 0; c < ATTN_MAX_HEAD_DIM / KVA_WAVE; ++c) {
        const int j = lane + c * KVA_WAVE;
        if (j < head_dim) orow[j] = from_float<T>(acc[c] / l);
    }
}

extern "C" int kva_attention_rowwise(void *out, const void *q, int q_row_stride, const void *k_cache,
                                     const void *v_cache, const int *block_table, int max_blocks,
                                     const int *tok_seat, const int *tok_pos, int tokens,
                                     int num_q_heads, int num_kv_heads, int head_dim, int page_size,
                                     float scale, int window, int dtype, hipStream_t stream) {
    KVA_REQUIRE(tokens >= 0 && num_q_heads > 0 && num_kv_heads > 0 && page_size > 0 && max_blocks > 0,
                "attention: bad sizes");
    KVA_REQUIRE(num_q_heads % num_kv_heads == 0, "attention: %d query heads is not a multiple of %d kv heads",
                num_q_heads, num_kv_heads);
    KVA_REQUIRE(head_dim % 4 == 0 && head_dim <= ATTN_MAX_HEAD_DIM,
                "attention: head_dim %d must be a multiple of 4 and at most %d", head_dim,
                ATTN_MAX_HEAD_DIM);
    KVA_REQUIRE(q_row_stride % 4 == 0, "attention: query row stride %d must be a multiple of 4", q_row_stride);
    KVA_REQUIRE(num_q_heads <= 65535, "attention: too many heads");
    KVA_REQUIRE(window >= 0, "attention: negative window");
    if (tokens == 0) return KVA_OK;
    dim3 grid(tokens, num_q_heads), block(KVA_WAVE);
    if (dtype == KVA_F32)
        hipLaunchKernelGGL(attention_rowwise_kernel<float>, grid, block, 0, stream, (float *)out,
                           (const float *)q, q_row_stride, (const float *)k_cache,
                           (const float *)v_cache, block_table, max_blocks, tok_seat, tok_pos,
                           num_q_heads, num_kv_heads, head_dim, page_size, scale, window);
    else if (dtype == KVA_BF16)
        hipLaunchKernelGGL(attention_rowwise_kernel<bf16_t>, grid, block, 0, stream, (bf16_t *)out,
                           (const bf16_t *)q, q_row_stride, (const bf16_t *)k_cache,
                           (const bf16_t *)v_cache, block_table, max_blocks, tok_seat, tok_pos,
                           num_q_heads, num_kv_heads, head_dim, page_size, scale, window);
    else KVA_REQUIRE(false, "attention: unsupported dtype %d", dtype);
    KVA_CHECK_LAUNCH("attention_rowwise");
    return KVA_OK;
}
