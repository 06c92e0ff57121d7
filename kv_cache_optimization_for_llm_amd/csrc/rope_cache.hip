// Rotary position encoding of Q and K fused with the write of K and V into the paged cache.
//
// The reference does this in three launches per layer: ropePackedKernel on Q, on K
// (base/src/kernels.cu:289-319) and scatterKVPackedKernel
// (paged_attention/src/kernels.cu:335-363).  Pairing is rotate-half: inside a head, element j
// pairs with j + rot/2 and both use angle index j:
//     out[j]         = x[j] * cos - x[j + rot/2] * sin
//     out[j + rot/2] = x[j] * sin + x[j + rot/2] * cos
// cos and sin come from fp32 tables [max_positions, rot/2] built once on the host.
// K is rotated BEFORE it is cached, V is cached as it is.
//
// Cache layout: K is [num_pages, num_kv_heads, head_dim / 8, page_size, 8] (kv_layout.h: a key's
// elements in chunks of 8, the chunks of all keys of a page next to each other); V is stored transposed
// inside a page, [num_pages, num_kv_heads, head_dim, page_size], so that the attention kernels
// can load "several keys of one value dimension" as one vector (the matrix-core operand layout
// of P*V).  Slot s of the slot mapping is page s / page_size, row s % page_size.  A negative
// slot skips the write.
#include "common.h"
#include "kv_layout.h"

template <typename T>
__global__ void rope_kv_write_kernel(T *__restrict__ qkv, T *__restrict__ k_cache,
                                     T *__restrict__ v_cache, const float *__restrict__ cos_table,
                                     const float *__restrict__ sin_table,
                                     const int *__restrict__ positions,
                                     const int *__restrict__ slot_mapping, int num_q_heads,
                                     int num_kv_heads, int head_dim, int rot_dim, int page_size,
                                     int write_cache) {
    const int t = blockIdx.x;
    const int row_width = (num_q_heads + 2 * num_kv_heads) * head_dim;
    T *row = qkv + (size_t)t * row_width;
    const int pos = positions[t];
    const int half = rot_dim / 2;
    const float *cs = cos_table ? cos_table + (size_t)pos * half : nullptr;
    const float *sn = sin_table ? sin_table + (size_t)pos * half : nullptr;

    int slot = -1;
    if (write_cache) slot = slot_mapping[t];
    const int page = slot >= 0 ? slot / page_size : 0;
    const int off = slot >= 0 ? slot % page_size : 0;

    // work item = (head among q and k heads, pair index in [0, head_dim/2)); pairs beyond the
    // rotated part (partial rotary) pass two plain elements through
    const int pairs_per_head = head_dim / 2;
    const int qk_heads = num_q_heads + num_kv_heads;
    for (int w = threadIdx.x; w < qk_heads * pairs_per_head; w += blockDim.x) {
        const int head = w / pairs_per_head;
        const int p = w % pairs_per_head;
        T *h = row + (size_t)head * head_dim;
        int i1, i2;
        float o1, o2;
        if (p < half) {
            i1 = p;
            i2 = p + half;
            const float x1 = to_float(h[i1]), x2 = to_float(h[i2]);
            if (cs) {
                const float c = cs[p], s = sn[p];
                o1 = x1 * c - x2 * s;
                o2 = x1 * s + x2 * c;
            } else {
                o1 = x1;
                o2 = x2;
            }
        } else {
            i1 = rot_dim + 2 * (p - half);
            i2 = i1 + 1;
            o1 = to_float(h[i1]);
            o2 = to_float(h[i2]);
        }
        const T r1 = from_float<T>(o1), r2 = from_float<T>(o2);
        if (head < num_q_heads) {
            h[i1] = r1;
            h[i2] = r2;
        } else if (slot >= 0) {
            const int kvh = head - num_q_heads;
            T *dst = k_cache + ((size_t)page * num_kv_heads + kvh) * page_size * head_dim;
            const int kc = kva_k_chunk(head_dim);
            dst[kva_k_at(off, i1, page_size, kc)] = r1;
            dst[kva_k_at(off, i2, page_size, kc)] = r2;
        }
    }
    if (slot >= 0) {
        const T *v = row + (size_t)(num_q_heads + num_kv_heads) * head_dim;
        for (int w = threadIdx.x; w < num_kv_heads * head_dim; w += blockDim.x) {
            const int kvh = w / head_dim, j = w % head_dim;
            v_cache[(((size_t)page * num_kv_heads + kvh) * head_dim + j) * page_size + off] = v[w];
        }
    }
}

// bf16, full rotary (rot_dim == head_dim), head_dim a multiple of 16: a thread rotates 8 pairs at a
// time with 16-byte loads and stores.
__device__ inline void rk_unpack8(const uint4 &v, float (&f)[8]) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        f[2 * i] = bf16_bits_to_float((uint16_t)(w[i] & 0xffffu));
        f[2 * i + 1] = bf16_bits_to_float((uint16_t)(w[i] >> 16));
    }
}

__device__ inline uint4 rk_pack8(const float (&f)[8]) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
        w[i] = (uint32_t)float_to_bf16_bits(f[2 * i]) | ((uint32_t)float_to_bf16_bits(f[2 * i + 1]) << 16);
    return make_uint4(w[0], w[1], w[2], w[3]);
}

__global__ void rope_kv_write_vec_kernel(bf16_t *__restrict__ qkv, bf16_t *__restrict__ k_cache,
                                         bf16_t *__restrict__ v_cache, const float *__restrict__ cos_table,
                                         const float *__restrict__ sin_table,
                                         const int *__restrict__ positions,
                                         const int *__restrict__ slot_mapping, int num_q_heads,
                                         int num_kv_heads, int head_dim, int page_size, int write_cache) {
    const int t = blockIdx.x;
    const int row_width = (num_q_heads + 2 * num_kv_heads) * head_dim;
    bf16_t *row = qkv + (size_t)t * row_width;
    const int pos = positions[t];
    const int half = head_dim / 2;
    const float *cs = cos_table + (size_t)pos * half;
    const float *sn = sin_table + (size_t)pos * half;
    int slot = -1;
    if (write_cache) slot = slot_mapping[t];
    const int page = slot >= 0 ? slot / page_size : 0;
    const int off = slot >= 0 ? slot % page_size : 0;
    const int chunks = half / 8;
    const int qk_heads = num_q_heads + num_kv_heads;
    for (int w = threadIdx.x; w < qk_heads * chunks; w += blockDim.x) {
        const int head = w / chunks, p0 = (w % chunks) * 8;
        if (head >= num_q_heads && slot < 0) continue;
        bf16_t *h = row + (size_t)head * head_dim;
        float x1[8], x2[8], c[8], s[8], o1[8], o2[8];
        rk_unpack8(*reinterpret_cast<const uint4 *>(h + p0), x1);
        rk_unpack8(*reinterpret_cast<const uint4 *>(h + half + p0), x2);
        const float4 c0 = *reinterpret_cast<const float4 *>(cs + p0), c1 = *reinterpret_cast<const float4 *>(cs + p0 + 4);
        const float4 s0 = *reinterpret_cast<const float4 *>(sn + p0), s1 = *reinterpret_cast<const float4 *>(sn + p0 + 4);
        c[0] = c0.x; c[1] = c0.y; c[2] = c0.z; c[3] = c0.w; c[4] = c1.x; c[5] = c1.y; c[6] = c1.z; c[7] = c1.w;
        s[0] = s0.x; s[1] = s0.y; s[2] = s0.z; s[3] = s0.w; s[4] = s1.x; s[5] = s1.y; s[6] = s1.z; s[7] = s1.w;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            o1[j] = x1[j] * c[j] - x2[j] * s[j];
            o2[j] = x1[j] * s[j] + x2[j] * c[j];
        }
        if (head >= num_q_heads) {
            // (head_dim is a multiple of 16 here: p0 and half + p0 are whole chunks of 8)
            bf16_t *dst = k_cache + ((size_t)page * num_kv_heads + (head - num_q_heads)) * page_size * head_dim;
            *reinterpret_cast<uint4 *>(dst + kva_k_at(off, p0, page_size, 8)) = rk_pack8(o1);
            *reinterpret_cast<uint4 *>(dst + kva_k_at(off, half + p0, page_size, 8)) = rk_pack8(o2);
        } else {
            *reinterpret_cast<uint4 *>(h + p0) = rk_pack8(o1);
            *reinterpret_cast<uint4 *>(h + half + p0) = rk_pack8(o2);
        }
    }
    if (slot >= 0) {
        const bf16_t *v = row + (size_t)(num_q_heads + num_kv_heads) * head_dim;
        for (int w = threadIdx.x; w < num_kv_heads * head_dim; w += blockDim.x) {
            const int kvh = w / head_dim, j = w % head_dim;
            v_cache[(((size_t)page * num_kv_heads + kvh) * head_dim + j) * page_size + off] = v[w];
        }
    }
}

extern "C" int kva_rope_kv_write(void *qkv, void *k_cache, void *v_cache, const float *cos_table,
                                 const float *sin_table, const int *positions,
                                 const int *slot_mapping, int tokens, int num_q_heads,
                                 int num_kv_heads, int head_dim, int rot_dim, int page_size,
                                 int write_cache, int dtype, hipStream_t stream) {
    KVA_REQUIRE(tokens >= 0 && num_q_heads > 0 && num_kv_heads > 0, "rope_kv_write: bad sizes");
    KVA_REQUIRE(head_dim > 0 && head_dim % 2 == 0, "rope_kv_write: head_dim %d must be even", head_dim);
    KVA_REQUIRE(rot_dim >= 0 && rot_dim <= head_dim && rot_dim % 2 == 0,
                "rope_kv_write: rotary dim %d must be even and at most head_dim %d", rot_dim, head_dim);
    KVA_REQUIRE((cos_table == nullptr) == (sin_table == nullptr), "rope_kv_write: one table missing");
    KVA_REQUIRE(!write_cache || (k_cache && v_cache && slot_mapping && page_size > 0),
                "rope_kv_write: cache write asked for without cache, slots or page size");
    if (tokens == 0) return KVA_OK;
    dim3 grid(tokens), block(256);
    if (dtype == KVA_BF16 && cos_table && rot_dim == head_dim && head_dim % 16 == 0) {
        hipLaunchKernelGGL(rope_kv_write_vec_kernel, grid, block, 0, stream, (bf16_t *)qkv,
                           (bf16_t *)k_cache, (bf16_t *)v_cache, cos_table, sin_table, positions,
                           slot_mapping, num_q_heads, num_kv_heads, head_dim, page_size, write_cache);
        KVA_CHECK_LAUNCH("rope_kv_write");
        return KVA_OK;
    }
    if (dtype == KVA_F32)
        hipLaunchKernelGGL(rope_kv_write_kernel<float>, grid, block, 0, stream, (float *)qkv,
                           (float *)k_cache, (float *)v_cache, cos_table, sin_table, positions,
                           slot_mapping, num_q_heads, num_kv_heads, head_dim, rot_dim, page_size,
                           write_cache);
    else if (dtype == KVA_BF16)
        hipLaunchKernelGGL(rope_kv_write_kernel<bf16_t>, grid, block, 0, stream, (bf16_t *)qkv,
                           (bf16_t *)k_cache, (bf16_t *)v_cache, cos_table, sin_table, positions,
                           slot_mapping, num_q_heads, num_kv_heads, head_dim, rot_dim, page_size,
                           write_cache);
    else KVA_REQUIRE(false, "rope_kv_write: unsupported dtype %d", dtype);
    KVA_CHECK_LAUNCH("rope_kv_write");
    return KVA_OK;
}
