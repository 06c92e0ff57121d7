// Causal grouped-query attention over the paged cache on the matrix cores (bf16, gfx950).
//
// One kernel serves prompt portions and decoded tokens.  Work is cut into ITEMS: an item is
// 16 * RT consecutive "query rows" of one request and one kv head, where
// row = token_in_step * G + g enumerates (token, query head of the kv head's group) pairs,
// G = num_q_heads / num_kv_heads.  A decoded token of a model with G <= 16 is one item of one
// row tile (RT = 1); prompt portions may use RT = 2 so that every key and value a wavefront
// loads serves 32 query rows.  One 64-lane wavefront runs one
// (item, kv head, key split); up to four wavefronts of one workgroup may take neighbouring key
// splits of the same item and add their results up in LDS (one barrier, at the end), which leaves
// the merge kernel fewer partial results, or none and no launch.
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
// ([kv_head, head_dim / 8, page_size, 8], kv_layout.h) in operand layout too, so there is no LDS and no barrier.
// Operand registers are double-buffered: the loads of block i+1 are issued before block i is
// computed.  With pages of 16 keys or a multiple, a 16-key tile lies in one page and the
// block-table lookup is uniform over the wavefront.
//
// Softmax is online in fp32 per query row (running max m, denominator l), scores scaled after
// the product and kept in the base-2 domain (exp(x) = exp2(x log2 e), one instruction); P is
// rounded to bf16 for the second product, the accumulator stays fp32.  Keys
// are visited in blocks of 32 aligned to absolute positions.  With `splits` > 1 each split
// writes an un-normalised partial (o, m, l) and attention_merge combines them (flash-decoding);
// with one split the normalised result is written directly.  The merge runs over every row of the
// output when the launch covered them all (`all_rows`), else over the rows the items name.
//
// Reference: same recurrence as paged_attention/src/kernels.cu:150-219 and the tiled prefill
// kernel base/src/kernels.cu:361-466, which work one key at a time on CUDA cores.
#include "common.h"
#include "attention_frag.h"
#include "kv_layout.h"
#include <type_traits>
#include <math.h>

// STREAM: keys and values are loaded with the non-temporal hint (see load_block).
// a wavefront's key range from which a third block of keys is kept in flight (decoded tokens)
#define LONG_RANGE_KEYS 1536
// wavefronts of one workgroup that may share an item (decoded tokens, head sizes up to 128)
#define KVA_ATTN_MAX_WAVES 4

// ROPE: the item is one decoded token whose Q, K and V lie in `q` as the joined projection left them
// ([.., q heads | k heads | v heads] per row, not yet rotated, nothing cached).  The wavefront
// rotates Q as it loads it, rotates the token's new K, puts K and V into the block of keys that
// holds the token's position (in registers: the page is not read back) and - one wavefront per
// (token, kv head) - stores them to the token's cache slot.  What the reference does in three
// launches before its attention kernel (ropePackedKernel twice, scatterKVPackedKernel;
// base/src/kernels.cu:289-319, paged_attention/src/kernels.cu:335-363) costs a decode step of
// many requests one launch per layer less.  Head sizes that are multiples of 64 (a lane holds both
// elements of a rotate-half pair), pages of 16.
struct RopeArgs {
    const float *cos_t, *sin_t;     // [positions, D / 2] fp32; both null: no rotation
    const int *slots;               // [tokens] cache slot of each token (negative: no write); null: nothing is cached
};

__device__ __forceinline__ void unpack8(const Frag8 &f, float (&x)[8]) {
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = bf16_bits_to_float(f.h[i]);
}

// (a, b) <- (a c - b s, a s + b c) element by element, rounded to bf16 as the rotation kernel rounds
__device__ __forceinline__ void rotate_pair(Frag8 &fa, Frag8 &fb, const float (&c)[8], const float (&s)[8]) {
    float a[8], b[8];
    unpack8(fa, a);
    unpack8(fb, b);
#pragma unroll
    for (int i = 0; i < 8; i += 2) {
        fa.p2[i / 2] = pack_bf16(a[i] * c[i] - b[i] * s[i], a[i + 1] * c[i + 1] - b[i + 1] * s[i + 1]);
        fb.p2[i / 2] = pack_bf16(a[i] * s[i] + b[i] * c[i], a[i + 1] * s[i + 1] + b[i + 1] * c[i + 1]);
    }
}

template <int D, int RT, bool FAST, bool STREAM, bool ROPE = false>
__device__ __forceinline__ void
attention_item(bf16_t *__restrict__ out, float *__restrict__ part_o, float *__restrict__ part_ml,
                      const bf16_t *__restrict__ q, int q_row_stride,
                      const bf16_t *__restrict__ k_cache, const bf16_t *__restrict__ v_cache,
                      const int *__restrict__ block_table, int max_blocks,
                      const int *__restrict__ item_meta,
                      const int *__restrict__ item_entry, const int *__restrict__ item_row0,
                      const int *__restrict__ entry_seat, const int *__restrict__ entry_q_start,
                      const int *__restrict__ entry_start_pos, int num_q_heads, int num_kv_heads,
                      int page_size, float scale, int window, int splits, int keys_per_split, const int item, const int kvh, const int split,
                      const RopeArgs rope = RopeArgs{nullptr, nullptr, nullptr}, const int ws = 1, const int wv = 0) {
    constexpr int KSTEP = (D % 32 == 0) ? 32 : 16;   // head-dim slice per S^T product
    static_assert(!ROPE || (RT == 1 && FAST && D % 64 == 0), "rotation inside the kernel: one row tile, pages of 16, head sizes that are multiples of 64");
    constexpr int NKS = D / KSTEP;
    constexpr int NDT = D / 16;                      // 16-wide tiles of the value dimension

    const int lane = threadIdx.x & (KVA_WAVE - 1), r = lane & 15, g = lane >> 4;   // (a workgroup may hold several wavefronts)
    const int G = num_q_heads / num_kv_heads;

    // Everything about the item is uniform over the wavefront: keep it in scalar registers.  Every
    // dependent load at the start of a short kernel costs a trip to memory, so the caller may
    // hand over all of it in one record per item (item_meta: q_start, q_len, start_pos, seat,
    // row0, 3 unused) instead of the chain item -> entry -> entry's arrays.
    int row0, q_start, q_len, start_pos, seat;
    if (item_meta != nullptr) {
        const int *meta = item_meta + (size_t)__builtin_amdgcn_readfirstlane(item) * 8;
        q_start = __builtin_amdgcn_readfirstlane(meta[0]);
        q_len = __builtin_amdgcn_readfirstlane(meta[1]);
        start_pos = __builtin_amdgcn_readfirstlane(meta[2]);
        seat = __builtin_amdgcn_readfirstlane(meta[3]);
        row0 = __builtin_amdgcn_readfirstlane(meta[4]);
    } else {
        const int e = __builtin_amdgcn_readfirstlane(item_entry[item]);
        row0 = __builtin_amdgcn_readfirstlane(item_row0[item]);
        q_start = __builtin_amdgcn_readfirstlane(entry_q_start[e]);
        q_len = __builtin_amdgcn_readfirstlane(entry_q_start[e + 1]) - q_start;
        start_pos = __builtin_amdgcn_readfirstlane(entry_start_pos[e]);
        seat = __builtin_amdgcn_readfirstlane(entry_seat[e]);
    }
    const int *bt = block_table + (size_t)seat * max_blocks;
    const int M = q_len * G;

    // per row tile: this lane's query row
    bool row_valid[RT];
    int tq[RT], head[RT], my_pos[RT], my_lo[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const int row = row0 + rt * 16 + r;
        row_valid[rt] = row < M;
        tq[rt] = row_valid[rt] ? row / G : 0;
        head[rt] = kvh * G + (row_valid[rt] ? row % G : 0);
        my_pos[rt] = start_pos + tq[rt];
        my_lo[rt] = (window > 0 && my_pos[rt] - window + 1 > 0) ? my_pos[rt] - window + 1 : 0;
    }

    // keys any row of this item may see
    const int last_row = (row0 + 16 * RT - 1 < M - 1) ? row0 + 16 * RT - 1 : M - 1;
    // (uniform over the wavefront like everything above: said explicitly, because the division by G
    // is done in the vector ALU and the compiler then takes every test on these for a per-lane one)
    const int item_hi = __builtin_amdgcn_readfirstlane(start_pos + last_row / G);                       // inclusive
    const int item_pos_lo = __builtin_amdgcn_readfirstlane(start_pos + row0 / G);
    const int item_lo = (window > 0 && item_pos_lo - window + 1 > 0) ? item_pos_lo - window + 1 : 0;
    int k_begin = item_lo & ~31;
    int k_end = item_hi + 1;                                            // exclusive
    if (splits > 1) {
        const int s_lo = split * keys_per_split, s_hi = s_lo + keys_per_split;
        if (s_lo > k_begin) k_begin = s_lo;
        if (s_hi < k_end) k_end = s_hi;
    }

    // Q^T operand: lane (r, g) holds Q[row r][ks * KSTEP + g * KSTEP/4 ...]
    Frag8 qf8[RT][NKS];
    Frag4 qf4[RT][NKS];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const bf16_t *qrow = q + (size_t)(q_start + tq[rt]) * q_row_stride + (size_t)head[rt] * D;
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
            // rows past the item's last read the entry's first row (tq and head are clamped): no
            // select on the loaded value, which would wait for it here, long before its first
            // use; every score of such a row is masked below and nothing of it is stored
            if (KSTEP == 32) qf8[rt][ks].u4 = *reinterpret_cast<const uint4 *>(qrow + ks * 32 + g * 8);
            else qf4[rt][ks].u2 = *reinterpret_cast<const uint2 *>(qrow + ks * 16 + g * 4);
        }
    }

    // ---- ROPE: rotate Q; make the token's K (rotated) and V ready for the cache and for the
    // block of keys that holds its position
    constexpr int HK = NKS / 2;                       // a rotate-half pair lies HK slices apart
    Frag8 k_new[ROPE ? NKS : 1];
    uint16_t v_new[ROPE ? NDT : 1];
    const bool caches = ROPE && rope.slots != nullptr;
    int rope_slot = -1;
    float cs[ROPE ? HK : 1][8], sn[ROPE ? HK : 1][8];
    if constexpr (ROPE) {
#pragma unroll
        for (int h = 0; h < HK; ++h)
#pragma unroll
            for (int i = 0; i < 8; ++i) { cs[h][i] = 1.f; sn[h][i] = 0.f; }
        if (caches) rope_slot = rope.slots[q_start];
        if (rope.cos_t != nullptr) {
            const size_t at = (size_t)start_pos * (D / 2) + g * 8;
#pragma unroll
            for (int h = 0; h < HK; ++h) {
                const float4 c0 = *reinterpret_cast<const float4 *>(rope.cos_t + at + h * 32);
                const float4 c1 = *reinterpret_cast<const float4 *>(rope.cos_t + at + h * 32 + 4);
                const float4 s0 = *reinterpret_cast<const float4 *>(rope.sin_t + at + h * 32);
                const float4 s1 = *reinterpret_cast<const float4 *>(rope.sin_t + at + h * 32 + 4);
                cs[h][0] = c0.x; cs[h][1] = c0.y; cs[h][2] = c0.z; cs[h][3] = c0.w;
                cs[h][4] = c1.x; cs[h][5] = c1.y; cs[h][6] = c1.z; cs[h][7] = c1.w;
                sn[h][0] = s0.x; sn[h][1] = s0.y; sn[h][2] = s0.z; sn[h][3] = s0.w;
                sn[h][4] = s1.x; sn[h][5] = s1.y; sn[h][6] = s1.z; sn[h][7] = s1.w;
            }
        }
        const bf16_t *tok_row = q + (size_t)q_start * q_row_stride;
        if (caches) {
            // every lane takes the slice of its lane group g (the same for all 16 rows r) and its
            // row's value dimensions: no branch around loads
            const bf16_t *krow = tok_row + (size_t)(num_q_heads + kvh) * D;
            const bf16_t *vrow = tok_row + (size_t)(num_q_heads + num_kv_heads + kvh) * D;
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) k_new[ks].u4 = *reinterpret_cast<const uint4 *>(krow + ks * 32 + g * 8);
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt) v_new[dt] = vrow[dt * 16 + r].bits;
        }
    }
    // The arithmetic on what was asked for above waits for it, so it runs after the first blocks of
    // keys have been asked for as well (one trip to memory for all of it, not two).
    auto rotate_and_store = [&]() {
        if constexpr (ROPE) {
            if (rope.cos_t != nullptr) {
    #pragma unroll
                for (int h = 0; h < HK; ++h) {
                    rotate_pair(qf8[0][h], qf8[0][h + HK], cs[h], sn[h]);
                    if (caches) rotate_pair(k_new[h], k_new[h + HK], cs[h], sn[h]);
                }
            }
            // one wavefront per (token, kv head) stores them: the one whose key range holds the position
            const int off = start_pos & 15;
            const bool owner = caches && row0 == 0 && (splits == 1 || split == start_pos / keys_per_split);
            const int slot = rope_slot;
            if (owner && slot >= 0) {
                const size_t page_elems = ((size_t)(slot >> 4) * num_kv_heads + kvh) * (size_t)(16 * D);
                if (r == off) {
    #pragma unroll
                    for (int ks = 0; ks < NKS; ++ks)
                        *reinterpret_cast<uint4 *>(const_cast<bf16_t *>(k_cache) + page_elems + kva_k_at(slot & 15, ks * 32 + g * 8, 16, 8)) = k_new[ks].u4;
                }
                if (g == 0) {
    #pragma unroll
                    for (int dt = 0; dt < NDT; ++dt)
                        const_cast<bf16_t *>(v_cache)[page_elems + (size_t)(dt * 16 + r) * 16 + (slot & 15)].bits = v_new[dt];
                }
            }
        }
    };

    float m[RT], l[RT];
    f32x4 o[RT][NDT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        m[rt] = -INFINITY;
        l[rt] = 0.f;
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) o[rt][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    // Operands of one 32-key block.  K: lane (r, g) holds K[key kstart + t*16 + r][ks*KSTEP +
    // g*KSTEP/4 ..].  V^T: lane (r, g) holds V^T[dt*16 + r][keys kstart + t*16 + 4g .. +3].
    // Two sets, so that the loads of block i+1 are in flight while block i is computed.
    struct BlockFrags {
        Frag8 k8[2][NKS];
        Frag4 k4[2][NKS];
        Frag8 v[NDT];
    };
    // FAST: pages of exactly 16 keys (the default).  A 16-key tile is one page, so the block-table lookup and
    // all address arithmetic up to a per-lane constant are scalar, and every load is
    // unconditional: a tile outside the keys the item needs is redirected to the nearest needed
    // tile (whose page is certainly mapped) and its scores are masked away.
    const int lo_tile = item_lo & ~15, hi_tile = item_hi & ~15;
    // K pages are [D / 8][16 keys][8] (kv_layout.h): a lane's 16 bytes (8 with head-dim slices of 16)
    // of key r are chunk (dim / 8) of that key, and a wavefront's load is one run of neighbouring bytes
    const uint32_t k_lane = KSTEP == 32 ? (uint32_t)(g * 16 + r) * 16u
                                        : (uint32_t)((g >> 1) * 16 + r) * 16u + (uint32_t)(g & 1) * 8u;   // bytes
    constexpr uint32_t k_slice = KSTEP == 32 ? 4u * 256u : 2u * 256u;          // bytes from one head-dim slice to the next
    const uint32_t v_lane = (uint32_t)(r * 16 + 4 * g) * 2u;                   // bytes
    constexpr uint32_t v_tile_stride = 16u * 16u * 2u;                         // 16 value dims
    // STREAM: keys and values go past the caches (non-temporal loads).  Right for decoded tokens
    // whose keys and values are read once per step and are too many to still be in the
    // memory-side cache at the next step; prompt items share theirs with the other row tiles of
    // the request through L2, and the keys of a few short requests (a few tens of megabytes over
    // all layers) survive a step in the memory-side cache if they are allowed in.
    auto load_block = [&](BlockFrags &f, int kstart) {
        if constexpr (FAST) {
            // the index is uniform: said so explicitly, the lookups are scalar loads (both issued
            // before either is waited for) and do not stand in the queue of the vector loads
            int pg[2];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                int tile0 = kstart + t * 16;
                tile0 = tile0 < lo_tile ? lo_tile : (tile0 > hi_tile ? hi_tile : tile0);
                pg[t] = bt[__builtin_amdgcn_readfirstlane(tile0 >> 4)];
            }
            __builtin_amdgcn_sched_barrier(0);                  // both lookups are out before either is used
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const size_t page_bytes = ((size_t)pg[t] * num_kv_heads + kvh) * (size_t)(16 * D * 2);
                const char *kb = reinterpret_cast<const char *>(k_cache) + page_bytes;
                const char *vb = reinterpret_cast<const char *>(v_cache) + page_bytes;
#pragma unroll
                for (int ks = 0; ks < NKS; ++ks) {
                    if (KSTEP == 32)
                        f.k8[t][ks].u4 = STREAM ? load_streamed_u4(kb + k_lane + ks * k_slice)
                                                : *reinterpret_cast<const uint4 *>(kb + k_lane + ks * k_slice);
                    else
                        f.k4[t][ks].u2 = STREAM ? load_streamed_u2(kb + k_lane + ks * k_slice)
                                                : *reinterpret_cast<const uint2 *>(kb + k_lane + ks * k_slice);
                }
#pragma unroll
                for (int dt = 0; dt < NDT; ++dt)
                    f.v[dt].u2[t] = STREAM ? load_streamed_u2(vb + v_lane + dt * v_tile_stride)
                                           : *reinterpret_cast<const uint2 *>(vb + v_lane + dt * v_tile_stride);
            }
            return;
        }
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int tile0 = kstart + t * 16;
            const bf16_t *krow = k_cache;
            size_t vbase = 0;
            const int key = tile0 + r, key0 = tile0 + 4 * g;
            const bool kvalid = key <= item_hi && key >= item_lo;       // pages outside may be unmapped
            const bool vvalid = key0 <= item_hi && key0 + 3 >= item_lo;
            int krow_in_page = 0;
            if (kvalid) {
                krow += ((size_t)bt[key / page_size] * num_kv_heads + kvh) * page_size * D;     // the page of this kv head
                krow_in_page = key % page_size;
            }
            if (vvalid)
                vbase = ((size_t)bt[key0 / page_size] * num_kv_heads + kvh) * D * page_size +
                        key0 % page_size;
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) {
                if (KSTEP == 32)
                    f.k8[t][ks].u4 = kvalid ? *reinterpret_cast<const uint4 *>(krow + kva_k_at(krow_in_page, ks * 32 + g * 8, page_size, 8))
                                            : make_uint4(0, 0, 0, 0);
                else
                    f.k4[t][ks].u2 = kvalid ? *reinterpret_cast<const uint2 *>(krow + kva_k_at(krow_in_page, ks * 16 + g * 4, page_size, 8))
                                            : make_uint2(0, 0);
            }
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt)
                f.v[dt].u2[t] = vvalid ? *reinterpret_cast<const uint2 *>(
                                             v_cache + vbase + (size_t)(dt * 16 + r) * page_size)
                                       : make_uint2(0, 0);
        }
    };

    // exponentials are taken in base 2: exp(x * scale) = exp2(x * scale * log2(e))
    const float scale2 = scale * 1.44269504088896340736f;
    const int first_pos = item_pos_lo;                   // smallest position among the item's rows
    const bool all_rows = row0 + 16 * RT <= M;

    // One 32-key block for all row tiles of the item, as straight-line code: first every S^T
    // product, then the softmax updates, then every P V product, so that the independent chains
    // of the row tiles overlap (matrix-core latency behind vector work and the other way round).
    // MASKED is decided per block (wave-uniform): blocks wholly visible to every row need no mask.
    auto compute_block_as = [&](auto masked_tag, const BlockFrags &f, int kstart) {
        constexpr bool MASKED = decltype(masked_tag)::value;
        f32x4 s[RT][2];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                s[rt][t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < NKS; ++ks) {
                    if (KSTEP == 32)
                        s[rt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.k8[t][ks].v, qf8[rt][ks].v, s[rt][t], 0, 0, 0);
                    else
                        s[rt][t] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(f.k4[t][ks].v, qf4[rt][ks].v, s[rt][t], 0, 0, 0);
                }
            }
        // ---- mask, online softmax for query row r (its keys are spread over 4 lane groups).
        // m and the maxima are kept in the domain of the raw products q.k; the scale (times
        // log2 e, for exp2) goes into the one fused multiply-add in front of every exponential.
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
        // m[rt] is the reference the row's exponentials are taken against.  It follows the
        // running maximum lazily: only when a row's maximum has outgrown it by more than
        // 2^REBASE (after scaling) does the wave re-base (multiply l and O by
        // exp2((old - new) * scale2)), which costs as much as the rest of the block.  In between,
        // p = exp2((s - m) * scale2) may reach 2^REBASE, which fp32 sums and bf16 products hold
        // without loss; o / l does not depend on the reference.
        constexpr float REBASE = 8.f;
        const float rebase_raw = REBASE / scale2;
        bool rebase = false;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) rebase = rebase || mloc[rt] > m[rt] + rebase_raw;
        if (__builtin_amdgcn_ballot_w64(rebase) != 0) {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                const float m_new = fmaxf(m[rt], quad_rows_max(mloc[rt]));
                // a row that has seen no key yet keeps m = -inf (exp2(-inf) = 0 clears nothing that counts)
                const float c = __builtin_amdgcn_exp2f((m[rt] - ((m_new == -INFINITY) ? 0.f : m_new)) * scale2);
                l[rt] *= c;
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
            float lsum = 0.f;
#pragma unroll
            for (int j = 0; j < 8; j += 2) {
                const float p0 = __builtin_amdgcn_exp2f(fmaf(sv[rt][j], scale2, neg_ref));   // exp2(-inf) = 0
                const float p1 = __builtin_amdgcn_exp2f(fmaf(sv[rt][j + 1], scale2, neg_ref));
                lsum += p0 + p1;
                pf[rt].p2[j / 2] = pack_bf16(p0, p1);
            }
            l[rt] += quad_rows_sum(lsum);
        }
        // ---- O^T += V^T * P^T
        // Behind the item's last key a block holds whatever the page held before (or the nearest
        // needed tile, for a redirected one): P is zero there, and the values are made zero too, so
        // that nothing non-finite left in a page can reach this request.  Straight-line code for
        // every masked block (the masks are all ones where the block ends before the item's last key).
        uint2 keep[2];
        if (MASKED) {
            const int n0 = item_hi + 1 - (kstart + 4 * g);
            keep[0] = keep_first_keys(make_uint2(~0u, ~0u), n0);
            keep[1] = keep_first_keys(make_uint2(~0u, ~0u), n0 - 16);
        }
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt) {
                Frag8 vv = f.v[dt];
                if (MASKED) {
                    vv.u2[0].x &= keep[0].x; vv.u2[0].y &= keep[0].y;
                    vv.u2[1].x &= keep[1].x; vv.u2[1].y &= keep[1].y;
                }
                o[rt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vv.v, pf[rt].v, o[rt][dt], 0, 0, 0);
            }
    };
    auto compute_block = [&](BlockFrags &f, int kstart) {
        if constexpr (ROPE) {
            // the block that holds the token's own position gets its key and value from registers
            if (caches && kstart <= start_pos && start_pos < kstart + 32) {
                // (selects between values: a store through a pointer chosen at run time, or under a
                // branch per tile, makes the compiler keep the fragments in memory)
                const int off = start_pos & 15, i = start_pos & 3;
                const bool second = start_pos - kstart >= 16;           // uniform
                const bool k0 = r == off && !second, k1 = r == off && second;
#pragma unroll
                for (int ks = 0; ks < NKS; ++ks) {
                    const uint4 n = k_new[ks].u4, a = f.k8[0][ks].u4, b = f.k8[1][ks].u4;
                    f.k8[0][ks].u4 = make_uint4(k0 ? n.x : a.x, k0 ? n.y : a.y, k0 ? n.z : a.z, k0 ? n.w : a.w);
                    f.k8[1][ks].u4 = make_uint4(k1 ? n.x : b.x, k1 ? n.y : b.y, k1 ? n.z : b.z, k1 ? n.w : b.w);
                }
                const bool mine = g == (off >> 2);
                const uint32_t sh = (i & 1) * 16, keep = ~(0xffffu << sh);
                const bool x0 = mine && !second && i < 2, y0 = mine && !second && i >= 2;
                const bool x1 = mine && second && i < 2, y1 = mine && second && i >= 2;
#pragma unroll
                for (int dt = 0; dt < NDT; ++dt) {
                    const uint32_t put = (uint32_t)v_new[dt] << sh;
                    const uint2 a = f.v[dt].u2[0], b = f.v[dt].u2[1];
                    f.v[dt].u2[0] = make_uint2(x0 ? (a.x & keep) | put : a.x, y0 ? (a.y & keep) | put : a.y);
                    f.v[dt].u2[1] = make_uint2(x1 ? (b.x & keep) | put : b.x, y1 ? (b.y & keep) | put : b.y);
                }
            }
        }
        // incl. redirected tiles and items whose last row tile is cut short
        const bool masked = window > 0 || kstart + 31 > first_pos || !all_rows;
        if (masked) compute_block_as(std::true_type{}, f, kstart);
        else compute_block_as(std::false_type{}, f, kstart);
    };

    // Two blocks in flight; three for a decoded token's wavefront that walks all of a long context
    // alone (few wavefronts, each a long stream: decode steps of 48 requests at 8,192 keys 3.78 ->
    // 3.56 ms, 64 requests 4.02 -> 3.88, 48 at 2,048 keys 1.86 -> 1.81; short ranges lose 1 % by it,
    // wavefronts that share a context in splits 3 % - there are a thousand of them and the third set of
    // registers costs them their place - and prompt items wait for the softmax's vector work, not
    // for memory).  The
    // loads are issued unconditionally (a block past the end is
    // redirected or predicated off inside load_block and its values are never used): a load
    // under a branch would make the wait before the next product a wait for everything.
    BlockFrags fa, fb;
    load_block(fa, k_begin);
    if (RT == 1 && STREAM && D <= 128 && splits == 1 && k_end - k_begin >= LONG_RANGE_KEYS) {   // (a third set of registers spills from 224 on)
        BlockFrags fc;
        load_block(fb, k_begin + 32);
        rotate_and_store();
        for (int kstart = k_begin; kstart < k_end; kstart += 96) {
            load_block(fc, kstart + 64);
            compute_block(fa, kstart);
            load_block(fa, kstart + 96);
            if (kstart + 32 < k_end) compute_block(fb, kstart + 32);
            load_block(fb, kstart + 128);
            if (kstart + 64 < k_end) compute_block(fc, kstart + 64);
        }
    } else {
        if constexpr (ROPE) {
            // the first turn written out, so that the second block is asked for before the rotation waits
            load_block(fb, k_begin + 32);
            rotate_and_store();
            if (k_begin < k_end) {
                compute_block(fa, k_begin);
                load_block(fa, k_begin + 64);
                if (k_begin + 32 < k_end) compute_block(fb, k_begin + 32);
            }
            k_begin += 64;
        }
        for (int kstart = k_begin; kstart < k_end; kstart += 64) {
            load_block(fb, kstart + 32);
            compute_block(fa, kstart);
            load_block(fa, kstart + 64);
            if (kstart + 32 < k_end) compute_block(fb, kstart + 32);
        }
    }

    // ---- Several wavefronts of a workgroup on one item (ws > 1): each has walked a range of its
    // own; all but the first leave (o, m, l) in LDS, lane by lane, and the first adds them to its
    // own as the merge kernel would - one launch less where the workgroup's ranges are all there
    // are, fewer partial results for the merge kernel otherwise.  Every wavefront reaches the barrier.
    int out_splits = splits, out_split = split;
    if (ws > 1) {
        extern __shared__ float xch[];
        constexpr int PER = RT * (NDT * 4 + 2);                 // floats per lane
        if (wv > 0) {
            float *mine = xch + ((size_t)(wv - 1) * PER) * KVA_WAVE + lane;
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
                for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) mine[(size_t)((rt * NDT + dt) * 4 + i) * KVA_WAVE] = o[rt][dt][i];
                mine[(size_t)(RT * NDT * 4 + 2 * rt) * KVA_WAVE] = m[rt];
                mine[(size_t)(RT * NDT * 4 + 2 * rt + 1) * KVA_WAVE] = l[rt];
            }
        }
        __syncthreads();
        if (wv > 0) return;
        for (int w = 1; w < ws; ++w) {
            const float *theirs = xch + ((size_t)(w - 1) * PER) * KVA_WAVE + lane;
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                const float m_w = theirs[(size_t)(RT * NDT * 4 + 2 * rt) * KVA_WAVE];
                const float l_w = theirs[(size_t)(RT * NDT * 4 + 2 * rt + 1) * KVA_WAVE];
                const float m_new = fmaxf(m[rt], m_w);
                // a range without a visible key has m = -inf and weighs nothing
                const float c_me = (m[rt] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f((m[rt] - m_new) * scale2);
                const float c_w = (m_w == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f((m_w - m_new) * scale2);
                l[rt] = l[rt] * c_me + l_w * c_w;
#pragma unroll
                for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        o[rt][dt][i] = o[rt][dt][i] * c_me + theirs[(size_t)((rt * NDT + dt) * 4 + i) * KVA_WAVE] * c_w;
                m[rt] = m_new;
            }
        }
        out_splits = splits / ws;
        out_split = split / ws;
    }

    // lane (r, g) holds O[row r][dt * 16 + 4g + i]
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        if (!row_valid[rt]) continue;
        const size_t orow = (size_t)(q_start + tq[rt]) * num_q_heads + head[rt];
        if (out_splits == 1) {
            const float inv = 1.f / l[rt];
            bf16_t *dst = out + orow * D;
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt) {
                union { b16x2 p2[2]; uint2 u2; } w;
                w.p2[0] = pack_bf16(o[rt][dt][0] * inv, o[rt][dt][1] * inv);
                w.p2[1] = pack_bf16(o[rt][dt][2] * inv, o[rt][dt][3] * inv);
                *reinterpret_cast<uint2 *>(dst + dt * 16 + 4 * g) = w.u2;
            }
        } else {
            float *dst = part_o + (orow * out_splits + out_split) * D;
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt)
                *reinterpret_cast<float4 *>(dst + dt * 16 + 4 * g) =
                    make_float4(o[rt][dt][0], o[rt][dt][1], o[rt][dt][2], o[rt][dt][3]);
            if (g == 0) {
                part_ml[(orow * out_splits + out_split) * 2] = m[rt] * scale2;   // the merge works in the base-2 domain
                part_ml[(orow * out_splits + out_split) * 2 + 1] = l[rt];
            }
        }
    }
}

// One wavefront per (item or pair of items, kv head, key split).  Workgroups are handed to the 8
// dies in turn, each die with its own L2: the kv head varies fastest, so a die keeps meeting the
// same heads' keys and values.  With `pair`, a wavefront takes item w and then item n-1-w of the
// list: the caller orders the list by the number of keys an item visits (most first), so every
// wavefront gets about the same work - rows late in a prompt visit many keys, early rows few.
template <int D, int RT, bool FAST, bool STREAM>
__global__ void __launch_bounds__(KVA_WAVE * KVA_ATTN_MAX_WAVES)
attention_mfma_kernel(bf16_t *__restrict__ out, float *__restrict__ part_o, float *__restrict__ part_ml,
                      const bf16_t *__restrict__ q, int q_row_stride,
                      const bf16_t *__restrict__ k_cache, const bf16_t *__restrict__ v_cache,
                      const int *__restrict__ block_table, int max_blocks,
                      const int *__restrict__ item_meta,
                      const int *__restrict__ item_entry, const int *__restrict__ item_row0,
                      const int *__restrict__ entry_seat, const int *__restrict__ entry_q_start,
                      const int *__restrict__ entry_start_pos, int num_q_heads, int num_kv_heads,
                      int page_size, float scale, int window, int splits, int keys_per_split, int num_items, int pair) {
    // (blockDim.x / 64 wavefronts of a workgroup take neighbouring key ranges of one item; `splits` counts all ranges)
    const int ws = blockDim.x / KVA_WAVE, wv = threadIdx.x / KVA_WAVE;
    const int kvh = blockIdx.x % num_kv_heads, split = blockIdx.z * ws + wv;
    const int w = blockIdx.x / num_kv_heads;
    attention_item<D, RT, FAST, STREAM>(out, part_o, part_ml, q, q_row_stride, k_cache, v_cache, block_table, max_blocks,
                                item_meta, item_entry, item_row0, entry_seat, entry_q_start, entry_start_pos, num_q_heads,
                                num_kv_heads, page_size, scale, window, splits, keys_per_split, w, kvh, split,
                                RopeArgs{nullptr, nullptr, nullptr}, ws, wv);
    const int other = num_items - 1 - w;
    if (pair && other > w)
        attention_item<D, RT, FAST, STREAM>(out, part_o, part_ml, q, q_row_stride, k_cache, v_cache, block_table, max_blocks,
                                    item_meta, item_entry, item_row0, entry_seat, entry_q_start, entry_start_pos, num_q_heads,
                                    num_kv_heads, page_size, scale, window, splits, keys_per_split, other, kvh, split);
}

// One wavefront per (decoded token, kv head, key split), with rotation and cache write inside.
template <int D, bool STREAM>
__global__ void __launch_bounds__(KVA_WAVE * KVA_ATTN_MAX_WAVES)
attention_mfma_rope_kernel(bf16_t *__restrict__ out, float *__restrict__ part_o, float *__restrict__ part_ml,
                           const bf16_t *__restrict__ qkv, int row_stride,
                           bf16_t *k_cache, bf16_t *v_cache,
                           const int *__restrict__ block_table, int max_blocks,
                           const int *__restrict__ item_meta, int num_q_heads, int num_kv_heads,
                           float scale, int window, int splits, int keys_per_split, const RopeArgs rope) {
    const int ws = blockDim.x / KVA_WAVE, wv = threadIdx.x / KVA_WAVE;
    const int kvh = blockIdx.x % num_kv_heads, split = blockIdx.z * ws + wv;
    const int w = blockIdx.x / num_kv_heads;
    attention_item<D, 1, true, STREAM, true>(out, part_o, part_ml, qkv, row_stride, k_cache, v_cache, block_table, max_blocks,
                                             item_meta, nullptr, nullptr, nullptr, nullptr, nullptr, num_q_heads,
                                             num_kv_heads, 16, scale, window, splits, keys_per_split, w, kvh, split, rope, ws, wv);
}

// out[row, :] = sum_s o_s * exp(m_s - M) / sum_s l_s * exp(m_s - M),  M = max_s m_s.
// One wavefront per row: lanes first own splits (max and denominator by wave reduction, the
// weights go to LDS), then own value dimensions and add the weighted partials.  The partials of
// the first MERGE_EARLY splits are loaded before the weights are known, so that the kernel makes
// one trip to memory, not two.
#define MERGE_EARLY 32
__global__ void __launch_bounds__(KVA_WAVE)
attention_merge_kernel(bf16_t *__restrict__ out, const float *__restrict__ part_o,
                       const float *__restrict__ part_ml, int head_dim, int splits,
                       const int *__restrict__ item_meta, const int *__restrict__ item_entry,
                       const int *__restrict__ item_row0, const int *__restrict__ entry_q_start,
                       int num_q_heads, int num_kv_heads) {
    __shared__ float w_s[MERGE_MAX_SPLITS];
    // Either one workgroup per row of `out` (the launch covered every row: item arrays null), or
    // one per (item, kv head, row of the item): then only the rows the items name are touched.
    size_t row = blockIdx.x;
    if (item_entry != nullptr || item_meta != nullptr) {
        const int kvh = blockIdx.x % num_kv_heads, item = blockIdx.x / num_kv_heads;
        int row0, q_start, q_len;
        if (item_meta != nullptr) {
            const int *meta = item_meta + (size_t)item * 8;
            q_start = meta[0]; q_len = meta[1]; row0 = meta[4];
        } else {
            const int e = item_entry[item];
            row0 = item_row0[item];
            q_start = entry_q_start[e];
            q_len = entry_q_start[e + 1] - q_start;
        }
        const int G = num_q_heads / num_kv_heads;
        const int r = row0 + (int)blockIdx.y;
        if (r >= q_len * G) return;
        row = (size_t)(q_start + r / G) * num_q_heads + kvh * G + r % G;
    }
    const int lane = threadIdx.x;
    const float2 *ml = reinterpret_cast<const float2 *>(part_ml) + row * splits;
    const float *po = part_o + row * splits * head_dim;
    // Every load whose address is known goes out before anything is waited for: this lane's
    // (max, sum) pairs and the first partial outputs of its first dimension.
    float2 first = make_float2(-INFINITY, 0.f);
    if (lane < splits) first = ml[lane];
    float early[MERGE_EARLY];
    const bool j0_ok = lane < head_dim;
#pragma unroll
    for (int s = 0; s < MERGE_EARLY; ++s)
        early[s] = (j0_ok && s < splits) ? po[(size_t)s * head_dim + lane] : 0.f;
    float M = first.x;
    for (int s = lane + KVA_WAVE; s < splits; s += KVA_WAVE) M = fmaxf(M, ml[s].x);
    M = wave_max(M);
    float denom = 0.f;
    auto weigh = [&](int s, float2 v) {
        const float w = (v.x == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(v.x - M);   // m is kept in the base-2 domain
        w_s[s] = w;
        denom += v.y * w;
    };
    if (lane < splits) weigh(lane, first);
    for (int s = lane + KVA_WAVE; s < splits; s += KVA_WAVE) weigh(s, ml[s]);
    denom = wave_sum(denom);
    __syncthreads();
    const float inv = 1.f / denom;
    for (int j = lane; j < head_dim; j += KVA_WAVE) {
        float acc = 0.f;
        int s0 = 0;
        if (j == lane) {                                   // this lane's first dimension: loaded already
            const int n = splits < MERGE_EARLY ? splits : MERGE_EARLY;
#pragma unroll
            for (int s = 0; s < MERGE_EARLY; ++s)
                if (s < n) acc += early[s] * w_s[s];
            s0 = n;
        }
#pragma unroll 8
        for (int s = s0; s < splits; ++s) acc += po[(size_t)s * head_dim + j] * w_s[s];
        out[row * head_dim + j].bits = float_to_bf16_bits(acc * inv);
    }
}

// Merges the partials of `splits` key splits into `out`: over every row of `out` (`all_rows`), or
// over the rows of the items alone, `rows_per_item` rows each, named by item_meta or by
// (item_entry, item_row0, entry_q_start).  Shared by the two matrix-core attention kernels.
int kva_attention_merge_launch(void *out, const float *part_o, const float *part_ml, int head_dim, int splits,
                               const int *item_meta, const int *item_entry, const int *item_row0,
                               const int *entry_q_start, int num_items, int rows_per_item, int total_rows,
                               int num_q_heads, int num_kv_heads, int all_rows, hipStream_t stream) {
    KVA_REQUIRE(splits >= 2 && splits <= MERGE_MAX_SPLITS && part_o && part_ml,
                "attention_merge: 2..%d splits and their partial results are needed", MERGE_MAX_SPLITS);
    if (all_rows)
        hipLaunchKernelGGL(attention_merge_kernel, dim3(total_rows), dim3(64), 0, stream, (bf16_t *)out,
                           part_o, part_ml, head_dim, splits, nullptr, nullptr, nullptr, nullptr,
                           num_q_heads, num_kv_heads);
    else
        hipLaunchKernelGGL(attention_merge_kernel, dim3(num_items * num_kv_heads, rows_per_item), dim3(64),
                           0, stream, (bf16_t *)out, part_o, part_ml, head_dim, splits, item_meta,
                           item_entry, item_row0, entry_q_start, num_q_heads, num_kv_heads);
    KVA_CHECK_LAUNCH("attention_merge");
    return KVA_OK;
}

extern "C" int kva_attention_max_splits() { return MERGE_MAX_SPLITS; }

extern "C" int kva_attention_mfma_supported(int head_dim, int page_size) {
    switch (head_dim) {
    case 16: case 32: case 48: case 64: case 80: case 96: case 112: case 128: case 160: case 192:
    case 224: case 256:
        return page_size % 4 == 0 ? 1 : 0;
    default:
        return 0;
    }
}

// Row tiles per item the kernel is built with for a head size when `wide` items are asked for.
extern "C" int kva_attention_mfma_row_tiles(int head_dim, int wide) {
    if (!wide) return 1;
    if (head_dim <= 128) return 2;
    return 1;
}

// Wavefronts of one workgroup that share an item (each a key range of its own, added up in LDS):
// 1, 2 or 4; more than one for items of one row tile, not in pairs, head sizes up to 128, and a
// number of key ranges they divide.
static bool kva_attention_mfma_waves_ok(int waves, int splits, int head_dim, int row_tiles, int pair) {
    if (waves == 1) return true;
    return (waves == 2 || waves == KVA_ATTN_MAX_WAVES) && row_tiles == 1 && !pair && head_dim <= 128 &&
           splits >= waves && splits % waves == 0;
}

// LDS in which all but the first of them leave their (o, m, l): head_dim + 2 floats per lane each.
static size_t kva_attention_mfma_exchange_bytes(int waves, int head_dim) {
    return waves > 1 ? (size_t)(waves - 1) * (head_dim / 16 * 4 + 2) * KVA_WAVE * sizeof(float) : 0;
}

// `out` null (more than one partial result a row left, splits / waves > 1): no merge launch; the
// partial results in part_o / part_ml are the call's result (kva_gemv_merged adds them up).
extern "C" int kva_attention_mfma(void *out, float *part_o, float *part_ml, const void *q,
                                  int q_row_stride, const void *k_cache, const void *v_cache,
                                  const int *block_table, int max_blocks, const int *item_meta,
                                  const int *item_entry, const int *item_row0, int num_items, int row_tiles,
                                  const int *entry_seat, const int *entry_q_start,
                                  const int *entry_start_pos, int total_rows, int num_q_heads,
                                  int num_kv_heads, int head_dim, int page_size, float scale, int window,
                                  int splits, int keys_per_split, int pair, int all_rows,
                                  int keep_cached, int waves, hipStream_t stream) {
    KVA_REQUIRE(num_items >= 0 && num_q_heads > 0 && num_kv_heads > 0 && max_blocks > 0,
                "attention_mfma: bad sizes");
    KVA_REQUIRE(kva_attention_mfma_waves_ok(waves, splits, head_dim, row_tiles, pair),
                "attention_mfma: %d wavefronts per item need one row tile, no pairs, a head size up to 128 and a "
                "number of key ranges (%d) they divide", waves, splits);
    KVA_REQUIRE(num_q_heads % num_kv_heads == 0, "attention_mfma: %d query heads is not a multiple of %d kv heads",
                num_q_heads, num_kv_heads);
    KVA_REQUIRE(kva_attention_mfma_supported(head_dim, page_size),
                "attention_mfma: head_dim %d / page_size %d not supported (head_dim a multiple of 16 up "
                "to 128 or 160/192/224/256, page_size a multiple of 4)", head_dim, page_size);
    KVA_REQUIRE(q_row_stride % 8 == 0, "attention_mfma: query row stride %d must be a multiple of 8", q_row_stride);
    KVA_REQUIRE(splits >= 1 && splits <= MERGE_MAX_SPLITS && num_kv_heads <= 65535,
                "attention_mfma: at most %d splits and 65535 kv heads", MERGE_MAX_SPLITS);
    KVA_REQUIRE(splits == 1 || (keys_per_split > 0 && keys_per_split % 32 == 0),
                "attention_mfma: splits need a key count that is a multiple of 32");
    KVA_REQUIRE(splits == waves || (part_o && part_ml), "attention_mfma: key ranges of several workgroups need a workspace");
    // without `out` the partial results (splits / waves a row) are left to the caller: no merge launch
    KVA_REQUIRE(out != nullptr || splits / waves > 1, "attention_mfma: no output");
    KVA_REQUIRE(window >= 0, "attention_mfma: negative window");
    KVA_REQUIRE(scale > 0.f, "attention_mfma: the score scale must be positive");
    KVA_REQUIRE(row_tiles == 1 || row_tiles == kva_attention_mfma_row_tiles(head_dim, 1),
                "attention_mfma: %d row tiles per item is not what head_dim %d is built with", row_tiles, head_dim);
    if (num_items == 0) return KVA_OK;
    KVA_REQUIRE((long)num_items * num_kv_heads < (1L << 31), "attention_mfma: too many work items");
    const int waves_x = pair ? (num_items + 1) / 2 : num_items;
    dim3 grid(waves_x * num_kv_heads, 1, splits / waves), block(KVA_WAVE * waves);
    const size_t lds = kva_attention_mfma_exchange_bytes(waves, head_dim);
    const bool fast = page_size == 16;
#define LAUNCH(DD, RR, FF, SS)                                                                  \
    hipLaunchKernelGGL((attention_mfma_kernel<DD, RR, FF, SS>), grid, block, lds, stream, (bf16_t *)out, \
                       part_o, part_ml, (const bf16_t *)q, q_row_stride, (const bf16_t *)k_cache, \
                       (const bf16_t *)v_cache, block_table, max_blocks, item_meta, item_entry,  \
                       item_row0,                                                               \
                       entry_seat, entry_q_start, entry_start_pos, num_q_heads, num_kv_heads,    \
                       page_size, scale, window, splits, keys_per_split, num_items, pair)
#define CASE(DD, WIDE)                                                                          \
    case DD:                                                                                    \
        if (row_tiles == 1) {                                                                   \
            if (fast && keep_cached) LAUNCH(DD, 1, true, false);                                \
            else if (fast) LAUNCH(DD, 1, true, true);                                           \
            else LAUNCH(DD, 1, false, false);                                                   \
        } else {                                                                                \
            if (fast) LAUNCH(DD, WIDE, true, false); else LAUNCH(DD, WIDE, false, false);       \
        }                                                                                       \
        break
    switch (head_dim) {
    CASE(16, 2); CASE(32, 2); CASE(48, 2); CASE(64, 2);
    CASE(80, 2); CASE(96, 2); CASE(112, 2); CASE(128, 2);
    CASE(160, 1); CASE(192, 1); CASE(224, 1); CASE(256, 1);
    default: KVA_REQUIRE(false, "attention_mfma: head_dim %d", head_dim);
    }
#undef CASE
#undef LAUNCH
    KVA_CHECK_LAUNCH("attention_mfma");
    if (splits / waves > 1 && out != nullptr)
        return kva_attention_merge_launch(out, part_o, part_ml, head_dim, splits / waves, item_meta, item_entry, item_row0,
                                          entry_q_start, num_items, 16 * row_tiles, total_rows, num_q_heads,
                                          num_kv_heads, all_rows, stream);
    return KVA_OK;
}

extern "C" int kva_attention_mfma_rope_supported(int head_dim, int page_size, int group) {
    return ((head_dim == 64 || head_dim == 128) && page_size == 16 && group >= 1 && group <= 16) ? 1 : 0;
}

// Attention of decoded tokens (one token per item: item_meta [items, 8] = (token row, 1, position,
// seat, 0, 0, 0, 0)) straight from the joined Q/K/V projection `qkv` [tokens, (nq + 2 nkv) d] bf16,
// not yet rotated: the kernel rotates Q and K by the token's position (cos_t / sin_t [positions, d / 2]
// fp32, both null: no rotation), stores the rotated K and the V at the token's cache slot
// (slots [tokens], a negative slot or slots == null: nothing is stored and the token's key is taken
// from the cache like every other) and attends.  At most 16 query heads per kv head.
extern "C" int kva_attention_mfma_rope(void *out, float *part_o, float *part_ml, const void *qkv, int row_stride,
                                       void *k_cache, void *v_cache, const int *block_table, int max_blocks,
                                       const int *item_meta, int num_items, int total_rows, int num_q_heads,
                                       int num_kv_heads, int head_dim, int page_size, float scale, int window,
                                       int splits, int keys_per_split, int keep_cached, const float *cos_t,
                                       const float *sin_t, const int *slots, int waves, hipStream_t stream) {
    KVA_REQUIRE(kva_attention_mfma_waves_ok(waves, splits, head_dim, 1, 0),
                "attention_mfma_rope: %d wavefronts per item must be 1, 2 or 4 and divide the %d key ranges", waves, splits);
    KVA_REQUIRE(num_items >= 0 && num_q_heads > 0 && num_kv_heads > 0 && max_blocks > 0 && item_meta != nullptr,
                "attention_mfma_rope: bad sizes");
    KVA_REQUIRE(num_q_heads % num_kv_heads == 0, "attention_mfma_rope: %d query heads is not a multiple of %d kv heads",
                num_q_heads, num_kv_heads);
    KVA_REQUIRE(kva_attention_mfma_rope_supported(head_dim, page_size, num_q_heads / num_kv_heads),
                "attention_mfma_rope: head_dim %d / page_size %d / %d heads per kv head not supported (64 or 128, 16, "
                "at most 16)", head_dim, page_size, num_q_heads / num_kv_heads);
    KVA_REQUIRE(row_stride % 8 == 0 && row_stride >= (num_q_heads + 2 * num_kv_heads) * head_dim,
                "attention_mfma_rope: row stride %d does not hold the joined projection", row_stride);
    KVA_REQUIRE(splits >= 1 && splits <= MERGE_MAX_SPLITS && num_kv_heads <= 65535,
                "attention_mfma_rope: at most %d splits and 65535 kv heads", MERGE_MAX_SPLITS);
    KVA_REQUIRE(splits == 1 || (keys_per_split > 0 && keys_per_split % 32 == 0),
                "attention_mfma_rope: splits need a key count that is a multiple of 32");
    KVA_REQUIRE(splits == waves || (part_o && part_ml), "attention_mfma_rope: key ranges of several workgroups need a workspace");
    KVA_REQUIRE(window >= 0 && scale > 0.f, "attention_mfma_rope: window must not be negative and the scale positive");
    KVA_REQUIRE((cos_t == nullptr) == (sin_t == nullptr), "attention_mfma_rope: one table missing");
    if (num_items == 0) return KVA_OK;
    KVA_REQUIRE((long)num_items * num_kv_heads < (1L << 31), "attention_mfma_rope: too many work items");
    dim3 grid(num_items * num_kv_heads, 1, splits / waves), block(KVA_WAVE * waves);
    const size_t lds = kva_attention_mfma_exchange_bytes(waves, head_dim);
    const RopeArgs rope{cos_t, sin_t, slots};
#define LAUNCH(DD, SS)                                                                               \
    hipLaunchKernelGGL((attention_mfma_rope_kernel<DD, SS>), grid, block, lds, stream, (bf16_t *)out, part_o, \
                       part_ml, (const bf16_t *)qkv, row_stride, (bf16_t *)k_cache, (bf16_t *)v_cache,     \
                       block_table, max_blocks, item_meta, num_q_heads, num_kv_heads, scale, window,  \
                       splits, keys_per_split, rope)
    if (head_dim == 64) { if (keep_cached) LAUNCH(64, false); else LAUNCH(64, true); }
    else { if (keep_cached) LAUNCH(128, false); else LAUNCH(128, true); }
#undef LAUNCH
    KVA_CHECK_LAUNCH("attention_mfma_rope");
    if (splits / waves > 1)
        return kva_attention_merge_launch(out, part_o, part_ml, head_dim, splits / waves, item_meta, nullptr, nullptr,
                                          nullptr, num_items, 16, total_rows, num_q_heads, num_kv_heads, 1, stream);
    return KVA_OK;
}

// ---------------------------------------------------------------------------------------------
// The same attention for callers that cannot allocate (declared in attention_static.h).
//
// kva_attention_mfma takes the partial results of its key splits in two buffers that the caller
// allocates per call.  Here they live in one file-scope device array instead: each GPU the
// library runs on holds its own copy, at its own address, until the process ends.  The array's
// name is only a host-side handle; the address kernels can use is asked for once per device
// (hipGetSymbolAddress, with that device current) and kept.
#include "attention_static.h"
#include <mutex>

static __device__ __align__(256) unsigned char scratch[KVA_ATTENTION_STATIC_SCRATCH_BYTES];

namespace {
constexpr int STATIC_MAX_DEVICES = 64;
std::mutex static_scratch_lock;
unsigned char *static_scratch_of_device[STATIC_MAX_DEVICES] = {};
}  // namespace

// The device address of `scratch` on the current device, looked up at the first call there.
static int static_scratch_address(unsigned char **out) {
    int device = -1;
    hipError_t e = hipGetDevice(&device);
    KVA_REQUIRE(e == hipSuccess && device >= 0 && device < STATIC_MAX_DEVICES,
                "attention_mfma_static: no current device (%s)", hipGetErrorString(e));
    std::lock_guard<std::mutex> hold(static_scratch_lock);
    if (static_scratch_of_device[device] == nullptr) {
        unsigned char *ptr = nullptr;
        e = hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch));
        KVA_REQUIRE(e == hipSuccess && ptr != nullptr,
                    "attention_mfma_static: the scratch array has no address on device %d (%s)", device,
                    hipGetErrorString(e));
        static_scratch_of_device[device] = ptr;
    }
    *out = static_scratch_of_device[device];
    return KVA_OK;
}

extern "C" long long kva_attention_mfma_static_scratch_bytes(int total_rows, int head_dim, int splits) {
    if (splits <= 1) return 0;
    // partial outputs [rows, splits, head_dim] fp32, then (max, sum) pairs [rows, splits, 2] fp32
    const long long outputs = ((long long)total_rows * splits * head_dim * 4 + 255) / 256 * 256;
    return outputs + (long long)total_rows * splits * 2 * 4;
}

extern "C" int kva_attention_mfma_static(void *out, const void *q, int q_row_stride, const void *k_cache,
                                         const void *v_cache, const int *block_table, int max_blocks,
                                         const int *item_meta, const int *item_entry, const int *item_row0,
                                         int num_items, int row_tiles, const int *entry_seat,
                                         const int *entry_q_start, const int *entry_start_pos, int total_rows,
                                         int num_q_heads, int num_kv_heads, int head_dim, int page_size,
                                         float scale, int window, int splits, int keys_per_split, int pair,
                                         int all_rows, hipStream_t stream) {
    KVA_REQUIRE(total_rows >= 0 && head_dim > 0 && splits >= 1, "attention_mfma_static: bad sizes");
    float *part_o = nullptr, *part_ml = nullptr;
    if (splits > 1) {
        const long long need = kva_attention_mfma_static_scratch_bytes(total_rows, head_dim, splits);
        KVA_REQUIRE(need <= (long long)KVA_ATTENTION_STATIC_SCRATCH_BYTES,
                    "attention_mfma_static: %d rows x %d splits x head size %d need %lld bytes of scratch, the "
                    "static array holds %lld; use fewer splits or kva_attention_mfma with buffers of your own",
                    total_rows, splits, head_dim, need, (long long)KVA_ATTENTION_STATIC_SCRATCH_BYTES);
        unsigned char *base = nullptr;
        const int rc = static_scratch_address(&base);
        if (rc != KVA_OK) return rc;
        part_o = reinterpret_cast<float *>(base);
        part_ml = reinterpret_cast<float *>(base + ((long long)total_rows * splits * head_dim * 4 + 255) / 256 * 256);
        // Nothing in the array has to start at zero: every (row, split) partial that the merge reads
        // is written by the attention launch before it, ranges without keys included.
    }
    return kva_attention_mfma(out, part_o, part_ml, q, q_row_stride, k_cache, v_cache, block_table, max_blocks,
                              item_meta, item_entry, item_row0, num_items, row_tiles, entry_seat, entry_q_start,
                              entry_start_pos, total_rows, num_q_heads, num_kv_heads, head_dim, page_size, scale,
                              window, splits, keys_per_split, pair, all_rows, /*keep_cached=*/0, /*waves=*/1, stream);
}
