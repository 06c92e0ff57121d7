// Causal grouped-query attention for prompt portions, with the keys and values of a block shared
// by four wavefronts through LDS (bf16, gfx950, pages of 16 keys, head sizes 32/64/96/128).
//
// The one-wavefront kernel (attention_mfma.hip) loads every key and value block once per 32 query
// rows, straight from the page into operand registers; for long prompts that traffic through the
// vector memory path is what it waits for (halving it nearly halves its time).  Here a workgroup
// of four wavefronts takes 128 consecutive query rows of one request and kv head (row =
// token * G + head_in_group, as there), each wavefront 32 of them, and every 32-key block is
// copied from the pages to LDS once for all four: 16 bytes per thread for K and for V^T, in the
// pages' own layout, rows padded so that the operand reads do not collide on the 32 banks (K rows
// 16 bytes longer, V^T rows 72 bytes apart).  The copies of
// block i+1 travel (global -> registers) while block i is computed, are written to the other
// half of LDS afterwards, and one barrier per block separates the two.
//
// The arithmetic per block is the other kernel's: S^T = K Q^T, online softmax in fp32 per query
// row with a lazily re-based reference, O^T += V^T P^T with P taken from the registers S^T came
// out in.  Usually every row's keys lie in one workgroup.  When a step has too few workgroups to
// fill the chip but each walks thousands of keys (a portion late in a long prompt), the keys are
// cut into `splits` ranges of `keys_per_split`, one workgroup each; a split writes un-normalised
// partials (o, m, l) as the one-wavefront kernel does and the same merge kernel combines them.
//
// Reference: the same recurrence as the tiled prefill kernel base/src/kernels.cu:361-466, which
// shares K/V tiles of 32 keys among the 8 query rows of a 256-thread block and cannot read keys
// from the cache.
#include "common.h"
#include "attention_frag.h"
#include "kv_layout.h"
#include <math.h>
#include <type_traits>

template <int D>
struct LdsGeom {
    static constexpr int KROW = D * 2 + 16;          // bytes per key row (D bf16 + pad)
    static constexpr int VROW = 32 * 2 + 8;          // bytes per value-dimension row (32 keys + pad)
    static constexpr int KBYTES = 32 * KROW;
    static constexpr int VBYTES = D * VROW;
    static constexpr int CHUNKS = 4 * D;             // 16-byte chunks of a K tile (and of a V^T tile)
    static constexpr int PER_THREAD = (CHUNKS + 255) / 256;
    static constexpr int SB = 1;                     // 32-key blocks per stage (per barrier); 2 measured slower
    static constexpr int BLOCK_BYTES = KBYTES + VBYTES;
    static constexpr int STAGE_BYTES = SB * BLOCK_BYTES;
};

template <int D>
__device__ __forceinline__ void
attention_lds_item(char *lds, bf16_t *__restrict__ out, float *__restrict__ part_o, float *__restrict__ part_ml,
                   const bf16_t *__restrict__ q, int q_row_stride,
                   const bf16_t *__restrict__ k_cache, const bf16_t *__restrict__ v_cache,
                   const int *__restrict__ block_table, int max_blocks,
                   const int *__restrict__ item_meta, int num_q_heads, int num_kv_heads, float scale,
                   int window, int splits, int keys_per_split, const int item, const int kvh, const int split) {
    using Geo = LdsGeom<D>;
    constexpr int RT = 2, NKS = D / 32, NDT = D / 16;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, g = lane >> 4;
    const int G = num_q_heads / num_kv_heads;

    const int *meta = item_meta + (size_t)__builtin_amdgcn_readfirstlane(item) * 8;
    const int q_start = __builtin_amdgcn_readfirstlane(meta[0]);
    const int q_len = __builtin_amdgcn_readfirstlane(meta[1]);
    const int start_pos = __builtin_amdgcn_readfirstlane(meta[2]);
    const int seat = __builtin_amdgcn_readfirstlane(meta[3]);
    const int row0 = __builtin_amdgcn_readfirstlane(meta[4]);
    const int *bt = block_table + (size_t)seat * max_blocks;
    const int M = q_len * G;

    // ---- this wavefront's 32 rows
    const int wrow0 = row0 + 32 * wave;
    const bool wave_valid = wrow0 < M;
    bool row_valid[RT];
    int tq[RT], head[RT], my_pos[RT], my_lo[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const int row = wrow0 + rt * 16 + r;
        row_valid[rt] = row < M;
        tq[rt] = row_valid[rt] ? row / G : 0;
        head[rt] = kvh * G + (row_valid[rt] ? row % G : 0);
        my_pos[rt] = start_pos + tq[rt];
        my_lo[rt] = (window > 0 && my_pos[rt] - window + 1 > 0) ? my_pos[rt] - window + 1 : 0;
    }
    const int w_last = (wrow0 + 31 < M - 1) ? wrow0 + 31 : M - 1;
    // (uniform over the wavefront: said explicitly, since the division by G is done in the vector
    // ALU and the compiler then takes every test on these for a per-lane one)
    const int w_hi = __builtin_amdgcn_readfirstlane(start_pos + w_last / G);      // last key the wave sees
    const int w_first_pos = __builtin_amdgcn_readfirstlane(start_pos + wrow0 / G);
    const int w_lo = (window > 0 && w_first_pos - window + 1 > 0) ? w_first_pos - window + 1 : 0;
    const bool all_rows = wrow0 + 32 <= M;

    // ---- keys the workgroup visits
    const int g_last = (row0 + 127 < M - 1) ? row0 + 127 : M - 1;
    const int g_hi = __builtin_amdgcn_readfirstlane(start_pos + g_last / G);
    const int g_first_pos = __builtin_amdgcn_readfirstlane(start_pos + row0 / G);
    const int g_lo = (window > 0 && g_first_pos - window + 1 > 0) ? g_first_pos - window + 1 : 0;
    int k_begin = g_lo & ~31;
    int k_end = g_hi + 1;
    if (splits > 1) {               // uniform over the workgroup; an empty range leaves m = -inf, l = 0
        const int s_lo = split * keys_per_split, s_hi = s_lo + keys_per_split;
        if (s_lo > k_begin) k_begin = s_lo;
        if (s_hi < k_end) k_end = s_hi;
    }
    const int lo_tile = g_lo & ~15, hi_tile = g_hi & ~15;

    // ---- Q^T operand: lane (r, g) holds Q[row r][ks * 32 + g * 8 ...]
    Frag8 qf[RT][NKS];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const bf16_t *qrow = q + (size_t)(q_start + tq[rt]) * q_row_stride + (size_t)head[rt] * D;
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks)
            qf[rt][ks].u4 = row_valid[rt] ? *reinterpret_cast<const uint4 *>(qrow + ks * 32 + g * 8)
                                          : make_uint4(0, 0, 0, 0);
    }

    // Running maximum m, accumulator O^T and denominator per query row.  The denominator is one more
    // tile of the second product: against a V^T tile of ones, O^T += V^T P^T adds up the row's P
    // (every element of the tile ends up as the row's sum) - on the matrix cores, which have time
    // to spare here, instead of 16 additions and a 4-lane reduction per block in the vector ALU,
    // which has none.  It also makes the denominator the sum of exactly the rounded P the numerator uses.
    float m[RT];
    f32x4 o[RT][NDT], ol[RT];
    Frag8 ones;
    ones.u4 = make_uint4(0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u);      // 8 x bf16 1.0
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        m[rt] = -INFINITY;
        ol[rt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) o[rt][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    // ---- copies page -> registers -> LDS.  Chunk c of the K tile is 16 bytes of key c % 16 of page c / 2D, dims 8 (c % 2D) / 16 ..;
    // chunk c of the V^T tile is 8 keys of value dimension (c % 2D) / 2 in page c / 2D.  A tile
    // outside the keys the workgroup needs is redirected to the nearest needed one (its page is
    // certainly mapped); its scores are masked away.
    // (named registers, not arrays: as arrays the compiler kept them in scratch memory for head sizes
    // with two chunks per thread, a store and a load of 64 bytes per thread and block)
    static_assert(Geo::SB == 1 && Geo::PER_THREAD <= 2, "the staging registers below are two chunks of one block");
    uint4 stage_k0, stage_k1, stage_v0, stage_v1;
    // which of the block's two pages a thread's chunk lies in is the same for a whole wavefront
    // (said explicitly, so that the page's address stays scalar arithmetic); its place inside the
    // page never changes
    int k_sel[Geo::PER_THREAD], v_sel[Geo::PER_THREAD], k_off[Geo::PER_THREAD], v_off[Geo::PER_THREAD];
#pragma unroll
    for (int i = 0; i < Geo::PER_THREAD; ++i) {
        const int c = tid + i * 256;
        // K pages are [D / 8][16 keys][8] (kv_layout.h): chunk c of the tile is 16 bytes number c % 2D of page c / 2D
        k_sel[i] = __builtin_amdgcn_readfirstlane(c / (2 * D));
        k_off[i] = (c % (2 * D)) * 8;
        const int rem = c % (2 * D);
        v_sel[i] = __builtin_amdgcn_readfirstlane(c / (2 * D));
        v_off[i] = (rem >> 1) * 16 + (rem & 1) * 8;
    }
    auto fetch = [&](int b, int kstart) {
        int pg[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            int tile0 = kstart + t * 16;
            tile0 = tile0 < lo_tile ? lo_tile : (tile0 > hi_tile ? hi_tile : tile0);
            pg[t] = bt[__builtin_amdgcn_readfirstlane(tile0 >> 4)];
        }
        auto chunk = [&](int i, uint4 &k, uint4 &v) {
            const int c = tid + i * 256;
            if (Geo::CHUNKS % 256 == 0 || c < Geo::CHUNKS) {
                const size_t kpage = ((size_t)(k_sel[i] ? pg[1] : pg[0]) * num_kv_heads + kvh) * (size_t)(16 * D);
                k = *reinterpret_cast<const uint4 *>(k_cache + kpage + k_off[i]);
                const size_t vpage = ((size_t)(v_sel[i] ? pg[1] : pg[0]) * num_kv_heads + kvh) * (size_t)(16 * D);
                v = *reinterpret_cast<const uint4 *>(v_cache + vpage + v_off[i]);
            }
        };
        chunk(0, stage_k0, stage_v0);
        if (Geo::PER_THREAD > 1) chunk(1, stage_k1, stage_v1);
    };
    auto stash = [&](int b, char *buf) {
        auto chunk = [&](int i, const uint4 &k, const uint4 &v) {
            const int c = tid + i * 256;
            if (Geo::CHUNKS % 256 == 0 || c < Geo::CHUNKS) {
                const int key = (c / (2 * D)) * 16 + (c & 15), kc = (c % (2 * D)) >> 4;     // the page's chunk order: [dim / 8][key]
                *reinterpret_cast<uint4 *>(buf + key * Geo::KROW + kc * 16) = k;
                const int t = c / (2 * D), rem = c % (2 * D);
                // rows of 72 bytes: 18 banks apart, so that the 16 lanes of an 8-byte operand read (rows r = 0..15
                // of one tile) meet 16 different pairs of the 32 banks; the price is two 8-byte writes here
                char *vp = buf + Geo::KBYTES + (rem >> 1) * Geo::VROW + (t * 16 + (rem & 1) * 8) * 2;
                *reinterpret_cast<uint2 *>(vp) = make_uint2(v.x, v.y);
                *reinterpret_cast<uint2 *>(vp + 8) = make_uint2(v.z, v.w);
            }
        };
        chunk(0, stage_k0, stage_v0);
        if (Geo::PER_THREAD > 1) chunk(1, stage_k1, stage_v1);
    };

    const float scale2 = scale * 1.44269504088896340736f;   // exp(x * scale) = exp2(x * scale * log2 e)
    constexpr float REBASE = 8.f;
    const float rebase_raw = REBASE / scale2;

    auto compute_as = [&](auto masked_tag, const char *buf, int kstart) {
        constexpr bool MASKED = decltype(masked_tag)::value;
        // operands from LDS: K: lane (r, g) holds K[key t*16 + r][ks*32 + g*8 ..]; V^T: lane (r, g)
        // holds V^T[dt*16 + r][keys t*16 + 4g .. +3] for both tiles of the block
        Frag8 kf[2][NKS], vf[NDT];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks)
                kf[t][ks].u4 = *reinterpret_cast<const uint4 *>(buf + (t * 16 + r) * Geo::KROW + (ks * 32 + g * 8) * 2);
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
            for (int t = 0; t < 2; ++t)
                vf[dt].u2[t] = *reinterpret_cast<const uint2 *>(buf + Geo::KBYTES + (dt * 16 + r) * Geo::VROW + (t * 16 + 4 * g) * 2);

        // Behind the workgroup's last key a block holds whatever the page held before (or the nearest
        // needed tile, for a redirected one): P is zero there, and the values are made zero too, so
        // that nothing non-finite left in a page can reach this request.
        if (MASKED && kstart + 31 > g_hi) {
            const int n0 = g_hi + 1 - (kstart + 4 * g), n1 = n0 - 16;
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt) {
                vf[dt].u2[0] = keep_first_keys(vf[dt].u2[0], n0);
                vf[dt].u2[1] = keep_first_keys(vf[dt].u2[1], n1);
            }
        }

        f32x4 s[RT][2];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                s[rt][t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < NKS; ++ks)
                    s[rt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[t][ks].v, qf[rt][ks].v, s[rt][t], 0, 0, 0);
            }
        float sv[RT][8], mloc[RT];
        Frag8 pf[RT];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            float mx = -INFINITY;
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float x = s[rt][t][i];
                    if (MASKED) {
                        const int key = kstart + t * 16 + 4 * g + i;
                        const bool vis = row_valid[rt] && key <= my_pos[rt] && key >= my_lo[rt];
                        x = vis ? x : -INFINITY;
                    }
                    sv[rt][t * 4 + i] = x;
                    mx = fmaxf(mx, x);
                }
            mloc[rt] = mx;            // this lane's part of the row: the whole row's only when the reference moves
        }
        // the reference of the exponentials follows the running maximum lazily (see attention_mfma.hip)
        bool rebase = false;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) rebase = rebase || mloc[rt] > m[rt] + rebase_raw;
        if (__builtin_amdgcn_ballot_w64(rebase) != 0) {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                const float m_new = fmaxf(m[rt], quad_rows_max(mloc[rt]));
                const float c = __builtin_amdgcn_exp2f((m[rt] - ((m_new == -INFINITY) ? 0.f : m_new)) * scale2);
                ol[rt][0] *= c; ol[rt][1] *= c; ol[rt][2] *= c; ol[rt][3] *= c;
#pragma unroll
                for (int dt = 0; dt < NDT; ++dt) {
                    o[rt][dt][0] *= c; o[rt][dt][1] *= c; o[rt][dt][2] *= c; o[rt][dt][3] *= c;
                }
                m[rt] = m_new;
            }
        }
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            const float neg_ref = (MASKED && m[rt] == -INFINITY) ? 0.f : -m[rt] * scale2;
#pragma unroll
            for (int j = 0; j < 8; j += 2) {
                const float p0 = __builtin_amdgcn_exp2f(fmaf(sv[rt][j], scale2, neg_ref));
                const float p1 = __builtin_amdgcn_exp2f(fmaf(sv[rt][j + 1], scale2, neg_ref));
                pf[rt].p2[j / 2] = pack_bf16(p0, p1);
            }
        }
        // Head sizes above 64: the wavefront whose products are ready goes first (head size 128,
        // 8,192-token prompt: 807 -> 772 us; head size 64 loses 1 % by it).  A SIMD issues either a
        // matrix-core product or a vector instruction, from whichever wavefront: timed alone, 8 products
        // and 24 multiply-adds in one wavefront take 126 ns, the products without the multiply-adds 67 and
        // the multiply-adds without the products 56, and given to two wavefronts of one SIMD 109; so a key
        // block costs its products plus its softmax, however the two are interleaved.
        if (D > 64) __builtin_amdgcn_s_setprio(1);
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt)
                o[rt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dt].v, pf[rt].v, o[rt][dt], 0, 0, 0);
            ol[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones.v, pf[rt].v, ol[rt], 0, 0, 0);
        }
        if (D > 64) __builtin_amdgcn_s_setprio(0);
    };

    // ---- the key loop: a stage is SB blocks of 32 keys; one barrier per stage, two LDS buffers.
    // Loads past the end are redirected inside fetch (never out of the mapped pages) and unused.
    auto compute = [&](const char *buf, int kstart) {
        if (wave_valid && kstart < k_end && kstart <= w_hi && kstart + 31 >= w_lo) {
            const bool masked = window > 0 || kstart + 31 > w_first_pos || !all_rows;
            if (masked) compute_as(std::true_type{}, buf, kstart);
            else compute_as(std::false_type{}, buf, kstart);
        }
    };
#pragma unroll
    for (int b = 0; b < Geo::SB; ++b) fetch(b, k_begin + 32 * b);
#pragma unroll
    for (int b = 0; b < Geo::SB; ++b) stash(b, lds + b * Geo::BLOCK_BYTES);
    __syncthreads();
    int which = 0;
    for (int kstart = k_begin; kstart < k_end; kstart += 32 * Geo::SB) {
        const bool more = kstart + 32 * Geo::SB < k_end;       // uniform over the workgroup
        if (more) {
#pragma unroll
            for (int b = 0; b < Geo::SB; ++b) fetch(b, kstart + 32 * (Geo::SB + b));
        }
#pragma unroll
        for (int b = 0; b < Geo::SB; ++b) compute(lds + which * Geo::STAGE_BYTES + b * Geo::BLOCK_BYTES, kstart + 32 * b);
        if (more) {
#pragma unroll
            for (int b = 0; b < Geo::SB; ++b) stash(b, lds + (which ^ 1) * Geo::STAGE_BYTES + b * Geo::BLOCK_BYTES);
        }
        __syncthreads();
        which ^= 1;
    }

    // ---- lane (r, g) holds O[row r][dt * 16 + 4g + i]
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        if (!row_valid[rt]) continue;
        const size_t orow = (size_t)(q_start + tq[rt]) * num_q_heads + head[rt];
        if (splits > 1) {
            float *dst = part_o + (orow * splits + split) * D;
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt)
                *reinterpret_cast<float4 *>(dst + dt * 16 + 4 * g) =
                    make_float4(o[rt][dt][0], o[rt][dt][1], o[rt][dt][2], o[rt][dt][3]);
            if (g == 0) {
                part_ml[(orow * splits + split) * 2] = m[rt] * scale2;   // the merge works in the base-2 domain
                part_ml[(orow * splits + split) * 2 + 1] = ol[rt][0];
            }
            continue;
        }
        const float inv = 1.f / ol[rt][0];
        bf16_t *dst = out + orow * D;
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) {
            union { b16x2 p2[2]; uint2 u2; } w;
            w.p2[0] = pack_bf16(o[rt][dt][0] * inv, o[rt][dt][1] * inv);
            w.p2[1] = pack_bf16(o[rt][dt][2] * inv, o[rt][dt][3] * inv);
            *reinterpret_cast<uint2 *>(dst + dt * 16 + 4 * g) = w.u2;
        }
    }
}

// One workgroup of four wavefronts per (item of 128 query rows or pair of items, kv head); the kv
// head varies fastest so that a die's L2 keeps meeting the same heads.  With `pair` a workgroup
// takes item w and then item n-1-w of the list, which the caller orders by keys visited.
template <int D>
__device__ __forceinline__ void
attention_lds_body(bf16_t *__restrict__ out, float *__restrict__ part_o, float *__restrict__ part_ml,
                   const bf16_t *__restrict__ q, int q_row_stride,
                   const bf16_t *__restrict__ k_cache, const bf16_t *__restrict__ v_cache,
                   const int *__restrict__ block_table, int max_blocks,
                   const int *__restrict__ item_meta, int num_items, int pair, int num_q_heads,
                   int num_kv_heads, float scale, int window, int splits, int keys_per_split) {
    using Geo = LdsGeom<D>;
    __shared__ __align__(16) char lds[2 * Geo::STAGE_BYTES];
    const int kvh = blockIdx.x % num_kv_heads;
    const int w = blockIdx.x / num_kv_heads, split = blockIdx.z;
    attention_lds_item<D>(lds, out, part_o, part_ml, q, q_row_stride, k_cache, v_cache, block_table, max_blocks,
                          item_meta, num_q_heads, num_kv_heads, scale, window, splits, keys_per_split, w, kvh, split);
    const int other = num_items - 1 - w;
    if (pair && other > w)      // the last barrier of the first item has passed: LDS is free again
        attention_lds_item<D>(lds, out, part_o, part_ml, q, q_row_stride, k_cache, v_cache, block_table, max_blocks,
                              item_meta, num_q_heads, num_kv_heads, scale, window, splits, keys_per_split, other, kvh,
                              split);
}

#define LDS_KERNEL_PARAMS                                                                          \
    bf16_t *__restrict__ out, float *__restrict__ part_o, float *__restrict__ part_ml,             \
    const bf16_t *__restrict__ q, int q_row_stride,                                                \
    const bf16_t *__restrict__ k_cache, const bf16_t *__restrict__ v_cache,                        \
    const int *__restrict__ block_table, int max_blocks, const int *__restrict__ item_meta,        \
    int num_items, int pair, int num_q_heads, int num_kv_heads, float scale, int window,           \
    int splits, int keys_per_split
#define LDS_KERNEL_ARGS                                                                            \
    out, part_o, part_ml, q, q_row_stride, k_cache, v_cache, block_table, max_blocks, item_meta,   \
    num_items, pair, num_q_heads, num_kv_heads, scale, window, splits, keys_per_split

template <int D>
__global__ void __launch_bounds__(256) attention_lds_kernel(LDS_KERNEL_PARAMS) {
    attention_lds_body<D>(LDS_KERNEL_ARGS);
}

// Head sizes up to 64 need a few registers more than three wavefronts per SIMD leave each (168):
// held to that, the compiler spills a handful of values, and three wavefronts instead of two are
// worth far more than those cost (the kernel is bound by vector work the wavefronts overlap).
template <int D>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3)))
attention_lds_kernel_3(LDS_KERNEL_PARAMS) {
    attention_lds_body<D>(LDS_KERNEL_ARGS);
}

// Head sizes 96 and 128: left alone the compiler takes over 300 registers, which leaves one wavefront
// per SIMD and nothing to overlap matrix-core, vector and LDS work with.
template <int D>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2)))
attention_lds_kernel_2(LDS_KERNEL_PARAMS) {
    attention_lds_body<D>(LDS_KERNEL_ARGS);
}

extern "C" int kva_attention_lds_supported(int head_dim, int page_size) {
    return (page_size == 16 && (head_dim == 32 || head_dim == 64 || head_dim == 96 || head_dim == 128)) ? 1 : 0;
}

// item_meta: [num_items, 8] int32 = (q_start, q_len, start_pos, seat, row0, 0, 0, 0) per item of
// 128 query rows (row0 a multiple of 128).  q: bf16 rows `q_row_stride` elements apart; out
// [tokens, num_q_heads * head_dim] bf16.
// With splits > 1: part_o [tokens * num_q_heads, splits, head_dim] and part_ml [.., splits, 2] fp32
// take the partials, keys_per_split is a multiple of 32, and the merge runs after the kernel: over
// every row of out (`all_rows`: the items cover them all) or over the items' rows alone.
extern "C" int kva_attention_lds(void *out, float *part_o, float *part_ml, const void *q, int q_row_stride,
                                 const void *k_cache, const void *v_cache, const int *block_table, int max_blocks,
                                 const int *item_meta, int num_items, int pair, int num_q_heads,
                                 int num_kv_heads, int head_dim, int page_size, float scale, int window,
                                 int splits, int keys_per_split, int total_rows, int all_rows,
                                 hipStream_t stream) {
    KVA_REQUIRE(splits >= 1 && splits <= MERGE_MAX_SPLITS && num_kv_heads <= 65535,
                "attention_lds: 1..%d splits and at most 65535 kv heads", MERGE_MAX_SPLITS);
    KVA_REQUIRE(splits == 1 || (keys_per_split > 0 && keys_per_split % 32 == 0 && part_o && part_ml),
                "attention_lds: splits need a key count that is a multiple of 32 and a workspace");
    KVA_REQUIRE(num_items >= 0 && num_q_heads > 0 && num_kv_heads > 0 && max_blocks > 0, "attention_lds: bad sizes");
    KVA_REQUIRE(num_q_heads % num_kv_heads == 0, "attention_lds: %d query heads is not a multiple of %d kv heads",
                num_q_heads, num_kv_heads);
    KVA_REQUIRE(kva_attention_lds_supported(head_dim, page_size),
                "attention_lds: head_dim %d with pages of %d keys is not supported (32/64/96/128, 16)", head_dim, page_size);
    KVA_REQUIRE(q_row_stride % 8 == 0 && q_row_stride >= num_q_heads * head_dim, "attention_lds: q row stride %d", q_row_stride);
    KVA_REQUIRE(window >= 0 && scale > 0.f, "attention_lds: window must not be negative and the scale positive");
    KVA_REQUIRE(item_meta != nullptr || num_items == 0, "attention_lds: item records are needed");
    if (num_items == 0) return KVA_OK;
    const int groups = pair ? (num_items + 1) / 2 : num_items;
    KVA_REQUIRE((long)groups * num_kv_heads < (1L << 31), "attention_lds: too many work items");
    dim3 grid(groups * num_kv_heads, 1, splits), block(256);
#define LAUNCH(KERNEL, DD)                                                                          \
    hipLaunchKernelGGL((KERNEL<DD>), grid, block, 0, stream, (bf16_t *)out, part_o, part_ml,        \
                       (const bf16_t *)q, q_row_stride, (const bf16_t *)k_cache,                    \
                       (const bf16_t *)v_cache, block_table, max_blocks, item_meta, num_items, pair, \
                       num_q_heads, num_kv_heads, scale, window, splits, keys_per_split)
    switch (head_dim) {
    case 32: LAUNCH(attention_lds_kernel_3, 32); break;
    case 64: LAUNCH(attention_lds_kernel_3, 64); break;
    case 96: LAUNCH(attention_lds_kernel_2, 96); break;
    default: LAUNCH(attention_lds_kernel_2, 128); break;
    }
#undef LAUNCH
    KVA_CHECK_LAUNCH("attention_lds");
    if (splits > 1)
        return kva_attention_merge_launch(out, part_o, part_ml, head_dim, splits, item_meta, nullptr, nullptr, nullptr,
                                          num_items, 128, total_rows, num_q_heads, num_kv_heads, all_rows, stream);
    return KVA_OK;
}
