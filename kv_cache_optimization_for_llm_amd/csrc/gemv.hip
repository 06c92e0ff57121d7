// y = x W^T for one or two tokens: matrix-vector products that stream the row-major weight once.
// Stands where the reference's decode step calls cublasGemmEx with one column per active row
// (base/src/engine.cu:1040-1117, 1141-1159, 1166-1253) followed by its norm, rotation, activation
// and residual kernels (base/src/kernels.cu:10-52, 227-275).
//
// For one or two tokens the matrix cores have nothing to reuse, and what bounds the product is how
// soon a wavefront has asked for all of its bytes and how short the chain is from the last byte's
// arrival to the stores.  Measured inside a graph at the 1B sizes with the model's epilogues, one
// token, microseconds (the few-rows kernel of gemm_skinny.hip -> this one): Q/K/V with rotation
// 7.3 -> 5.5, output 5.8 -> 4.2, gate/up 13.5 -> 12.6, down 13.1 -> 8.6.
//
// A wavefront takes whole rows of W, RB at a time.  Lane l keeps columns (64 c + l) * 8 .. + 8 of
// the token(s) in registers for the whole kernel, asks for its 16 bytes of every KiB of its RB
// rows before it uses any of them (non-temporal loads: the weights of a decode step are read once),
// multiplies pairs of bf16 into fp32 sums (v_dot2c_f32_bf16) and adds the 64 lanes' sums inside
// the vector ALU.  The epilogues are the
// few-rows kernel's, value for value: an optional per-token scale that finishes the input's
// RMSNorm; plain (bf16 or fp32); SwiGLU over a joined [gate; up] matrix (a wavefront takes row i of
// both halves); residual add + preparation of the next norm; rotate-half rotation + cache write for
// the joined Q/K/V matrix (a wavefront takes rows j and j + d/2 of a head).
#include "common.h"
#include "kv_layout.h"

#include <algorithm>

namespace {

enum { GV_PLAIN = 0, GV_SWIGLU = 1, GV_RESID = 2, GV_ROPE = 3 };

struct GemvArgs {
    const bf16_t *X;
    const bf16_t *W;
    int M, N, K, ldx;
    const float *sumsq;          // [M, sumsq_parts] or null
    int sumsq_parts, norm_width;
    float eps;
    // GV_PLAIN / GV_SWIGLU
    void *Y;
    int ldy, out_f32, inter;
    // GV_RESID
    bf16_t *hidden;
    const void *next_w;
    int next_w_f32;
    bf16_t *scaled_out;
    float *sumsq_out;            // [M, one part per workgroup and round]
    int parts_out;
    // GV_RESID with X given as the partial results of an attention kernel's key ranges (X null):
    // part_o [M * heads, parts, part_head_dim], part_ml [M * heads, parts] (maximum in the base-2
    // domain, sum), heads = K / part_head_dim
    const float *part_o, *part_ml;
    int parts, part_head_dim;
    // GV_ROPE (Y is the Q output, row stride ldy)
    const float *cos_t, *sin_t;
    const int *positions, *slots;
    bf16_t *k_cache, *v_cache;
    int nq, nkv, head_dim, page_size;
};

// c + a.lo * b.lo + a.hi * b.hi for two packed pairs of bf16, in one instruction
typedef __bf16 gv_bf16x2 __attribute__((ext_vector_type(2)));
__device__ inline float gv_dot2(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(gv_bf16x2, a), __builtin_bit_cast(gv_bf16x2, b), c, false);
}

__device__ inline float gv_round_bf16(float v) { return bf16_bits_to_float(float_to_bf16_bits(v)); }

// acc[r][m] of the pair (r, m) that this lane finishes: a chain of selects, no indexed registers
template <int RB, int M>
__device__ inline float gv_pick(const float (&acc)[RB][M], int r, int m) {
    float v = 0.f;
#pragma unroll
    for (int rr = 0; rr < RB; ++rr)
#pragma unroll
        for (int mm = 0; mm < M; ++mm)
            if (rr == r && mm == m) v = acc[rr][mm];
    return v;
}

constexpr int GV_WAVES = 4;          // wavefronts per workgroup
// Partial sums of squares a lane asks for per token before anything else: 512 in all, which is what
// the down projection of a 2,048-wide model leaves (a part per four rows).  Beyond them a loop of
// load, wait, add takes over, and that wait is for every load in flight, the rows of W included:
// 0.8 us of the Q/K/V product's 5.5 when four were asked for here.
constexpr int GV_NORM_LOADS = 8;
// Partial results of key ranges per row that the merged form adds up (a lane holds 10 floats of
// each): up to 4 in one instance, up to 8 in another that exists for one token only - the registers
// of eight cost the steps that need four 1.5-2 % (one / two requests at 768 keys 0.660 / 0.741 ->
// 0.670 / 0.757 ms), and one request at 2,049-4,096 keys gains 3 % from them (0.720 -> 0.698 at 3,000).
constexpr int GV_MERGE_PARTS = 4;
constexpr int GV_MERGE_MAX_PARTS = 8;

// KV: 16-byte vectors per lane and row (K = 512 KV); M: tokens; RB: rows a wavefront has in flight.
// Row r of unit u: plain / residual: u RB + r.  SwiGLU (RB even): pair t = r / 2 of the unit is
// column u RB/2 + t; r even is its gate row, r odd its up row (inter further on).  Rotation (RB
// even): unit u = (head, block of RB/2 features below d/2); r even is feature f, r odd f + d/2.
//
// Everything a wavefront reads is asked for before it waits for any of it: the tokens, the rows of
// W, the partial sums that finish the input's norm, and what its epilogue needs (the residual
// stream and the next norm's weight, or the rotation's cosines and sines).  After the wavefront
// reductions every lane has every sum, and lane l finishes pair (row l % RB, token l / RB).
//
// MERGED (residual epilogue, K up to 4,096): the token(s) are not read but made - the output
// projection of an attention layer takes the partial results that the attention kernel left per
// key range (at most PARTS a row) and adds them up itself, as the merge kernel would
// (weights 2^(m_s - max m), the sum divided by the weighted sum of the l_s, rounded to bf16), so
// that one or two decoded tokens need no merge launch.  The wavefronts of a workgroup share the
// work: wavefront w makes the columns of vectors c = w, w + GV_WAVES, ... and leaves them in LDS.
template <int KV, int M, int RB, int EPI, int PARTS = 0>
__global__ void __launch_bounds__(64 * GV_WAVES) gemv_kernel(const GemvArgs a) {
    constexpr bool MERGED = PARTS > 0;
    constexpr int MAXP = MERGED ? PARTS : 1;       // partial results a row that a lane has room for
    const int lane = threadIdx.x & 63, wave_in_block = threadIdx.x >> 6;
    const int K = a.K;
    constexpr int PAIRS = RB / 2;
    constexpr int OUTS = (EPI == GV_SWIGLU || EPI == GV_ROPE) ? PAIRS : RB;   // results per token and unit
    __shared__ float block_ss[2][GV_WAVES][M];
    int units;
    if (EPI == GV_SWIGLU) units = (a.inter + PAIRS - 1) / PAIRS;
    else if (EPI == GV_ROPE) units = (a.nq + 2 * a.nkv) * (a.head_dim / 2 / PAIRS);
    else units = (a.N + RB - 1) / RB;
    int base = blockIdx.x * GV_WAVES;
    if (base >= units) return;
    // this lane's part of the epilogue
    const int my = lane % OUTS, my_m = lane / OUTS;
    const bool finishing = lane < OUTS * M;

    // position and cache slot of this lane's token: the same addresses for every lane, read first
    // so that the rotation's table rows can be asked for while W is on its way
    int pos = 0, slot = -1;
    if (EPI == GV_ROPE) {
#pragma unroll
        for (int m = 0; m < M; ++m) {
            const int p = a.cos_t != nullptr ? a.positions[m] : 0;
            const int sl = a.slots != nullptr ? a.slots[m] : -1;
            if (m == my_m) pos = p, slot = sl;
        }
    }

    // The partial sums of squares of the input's norm are the first thing asked for: they come
    // from L2 and are added up, and the scale taken, while W is on its way.
    float norm_part[M][GV_NORM_LOADS];
    if (a.sumsq != nullptr) {
#pragma unroll
        for (int m = 0; m < M; ++m)
#pragma unroll
            for (int i = 0; i < GV_NORM_LOADS; ++i) {
                const int p = min(lane + 64 * i, a.sumsq_parts - 1);       // masked where they are added
                norm_part[m][i] = a.sumsq[(size_t)m * a.sumsq_parts + p];
            }
    }

    // the token(s), kept packed: lane l owns columns (64 c + l) * 8 .. + 8
    uint4 xp[M][KV];
    constexpr int MINE = MERGED ? (KV + GV_WAVES - 1) / GV_WAVES : 1;     // vectors this wavefront makes per token
    float2 pml[MINE][M][MAXP];
    float4 pov[MINE][M][MAXP][2];
    if constexpr (MERGED) {
        const int heads = K / a.part_head_dim;
#pragma unroll
        for (int i = 0; i < MINE; ++i) {
            const int c = min(wave_in_block + i * GV_WAVES, KV - 1);
            const int col = (c * 64 + lane) * 8;
            const int head = col / a.part_head_dim, j0 = col - head * a.part_head_dim;
#pragma unroll
            for (int m = 0; m < M; ++m) {
                const size_t row = (size_t)m * heads + head;
#pragma unroll
                for (int sp = 0; sp < MAXP; ++sp) {
                    const int ss = min(sp, a.parts - 1);                      // masked where they are added
                    pml[i][m][sp] = reinterpret_cast<const float2 *>(a.part_ml)[row * a.parts + ss];
                    const float4 *po = reinterpret_cast<const float4 *>(a.part_o + (row * a.parts + ss) * a.part_head_dim + j0);
                    pov[i][m][sp][0] = po[0];
                    pov[i][m][sp][1] = po[1];
                }
            }
        }
    } else {
#pragma unroll
        for (int m = 0; m < M; ++m)
#pragma unroll
            for (int c = 0; c < KV; ++c)
                xp[m][c] = *reinterpret_cast<const uint4 *>(a.X + (size_t)m * a.ldx + (c * 64 + lane) * 8);
    }
    uint4 w[RB][KV];
    // asks for the rows of W of unit u (an index past the end takes the last unit's rows again)
    auto ask_for_rows = [&](int u) {
#pragma unroll
        for (int r = 0; r < RB; ++r) {
            int n;
            if (EPI == GV_SWIGLU) {
                int col = u * PAIRS + r / 2;
                if (col >= a.inter) col = a.inter - 1;
                n = (r & 1) ? a.inter + col : col;
            } else if (EPI == GV_ROPE) {
                const int per_head = a.head_dim / 2 / PAIRS;
                const int head = u / per_head, f = (u - head * per_head) * PAIRS + r / 2;
                n = head * a.head_dim + f + ((r & 1) ? a.head_dim / 2 : 0);
            } else {
                n = u * RB + r;
                if (n >= a.N) n = a.N - 1;
            }
#pragma unroll
            for (int c = 0; c < KV; ++c)
                w[r][c] = load_streamed_u4(a.W + (size_t)n * K + (c * 64 + lane) * 8);
        }
    };
    bool active = base + wave_in_block < units;
    int u = active ? base + wave_in_block : units - 1;
    ask_for_rows(u);

    const float inv_width = a.sumsq != nullptr ? 1.f / (float)a.norm_width : 1.f;
    // everything is asked for before anything is waited for
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (MERGED) {
        __shared__ uint4 merged_x[M][KV * 64];
#pragma unroll
        for (int i = 0; i < MINE; ++i) {
            const int c = wave_in_block + i * GV_WAVES;
#pragma unroll
            for (int m = 0; m < M; ++m) {
                float mx = -INFINITY;
#pragma unroll
                for (int sp = 0; sp < MAXP; ++sp)
                    if (sp < a.parts) mx = fmaxf(mx, pml[i][m][sp].x);
                float denom = 0.f, acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int sp = 0; sp < MAXP; ++sp) {
                    if (sp < a.parts) {
                        const float wgt = pml[i][m][sp].x == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(pml[i][m][sp].x - mx);
                        denom += pml[i][m][sp].y * wgt;
                        const float4 lo = pov[i][m][sp][0], hi = pov[i][m][sp][1];
                        acc[0] += lo.x * wgt; acc[1] += lo.y * wgt; acc[2] += lo.z * wgt; acc[3] += lo.w * wgt;
                        acc[4] += hi.x * wgt; acc[5] += hi.y * wgt; acc[6] += hi.z * wgt; acc[7] += hi.w * wgt;
                    }
                }
                const float inv = 1.f / denom;
                uint32_t pk[4];
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    pk[j] = (uint32_t)float_to_bf16_bits(acc[2 * j] * inv) |
                            ((uint32_t)float_to_bf16_bits(acc[2 * j + 1] * inv) << 16);
                if (c < KV) merged_x[m][c * 64 + lane] = make_uint4(pk[0], pk[1], pk[2], pk[3]);
            }
        }
        __syncthreads();
#pragma unroll
        for (int m = 0; m < M; ++m)
#pragma unroll
            for (int c = 0; c < KV; ++c) xp[m][c] = merged_x[m][c * 64 + lane];
    }
    float rinv[M];
#pragma unroll
    for (int m = 0; m < M; ++m) {
        rinv[m] = 1.f;
        if (a.sumsq != nullptr) {
            float sp = 0.f;
#pragma unroll
            for (int i = 0; i < GV_NORM_LOADS; ++i) sp += lane + 64 * i < a.sumsq_parts ? norm_part[m][i] : 0.f;
            for (int p = lane + 64 * GV_NORM_LOADS; p < a.sumsq_parts; p += 64)
                sp += a.sumsq[(size_t)m * a.sumsq_parts + p];
            // (v_rsq_f32, one ulp: the precise square root and division of the few-rows kernel sit
            // on the path from the sums' arrival to the scale and cost 0.1-0.3 us of a 5 us kernel)
            rinv[m] = rsqrtf(wave_sum_valu(sp) * inv_width + a.eps);
        }
    }
    int parity = 0;

    // every wavefront of a workgroup goes round as often as the others: the residual epilogue
    // adds their sums of squares through LDS
    for (;;) {
        // what the epilogue reads
        float e0 = 0.f, e1 = 1.f;        // residual: stream value, next norm's weight; rotation: cos, sin
        int my_n = 0;
        if (EPI == GV_RESID) {
            my_n = u * RB + my;
            if (finishing && my_n < a.N) {
                e0 = to_float(a.hidden[(size_t)my_m * a.N + my_n]);
                if (a.next_w != nullptr)
                    e1 = a.next_w_f32 ? reinterpret_cast<const float *>(a.next_w)[my_n]
                                      : to_float(reinterpret_cast<const bf16_t *>(a.next_w)[my_n]);
            }
        } else if (EPI == GV_ROPE) {
            const int per_head = a.head_dim / 2 / PAIRS;
            const int head = u / per_head;
            my_n = (u - head * per_head) * PAIRS + my;                       // the feature below d/2
            e0 = 1.f, e1 = 0.f;
            if (finishing && a.cos_t != nullptr && head < a.nq + a.nkv) {
                e0 = a.cos_t[(size_t)pos * (a.head_dim / 2) + my_n];
                e1 = a.sin_t[(size_t)pos * (a.head_dim / 2) + my_n];
            }
        }

        // two chains of sums per (row, token): a dot product of two bf16 pairs per instruction
        float part[RB][M][2];
#pragma unroll
        for (int r = 0; r < RB; ++r)
#pragma unroll
            for (int m = 0; m < M; ++m) part[r][m][0] = part[r][m][1] = 0.f;
#pragma unroll
        for (int c = 0; c < KV; ++c)
#pragma unroll
            for (int r = 0; r < RB; ++r) {
                const uint32_t wv[4] = {w[r][c].x, w[r][c].y, w[r][c].z, w[r][c].w};
#pragma unroll
                for (int m = 0; m < M; ++m) {
                    const uint32_t xv[4] = {xp[m][c].x, xp[m][c].y, xp[m][c].z, xp[m][c].w};
#pragma unroll
                    for (int j = 0; j < 4; ++j) part[r][m][j & 1] = gv_dot2(wv[j], xv[j], part[r][m][j & 1]);
                }
            }
        float acc[RB][M];
#pragma unroll
        for (int r = 0; r < RB; ++r)
#pragma unroll
            for (int m = 0; m < M; ++m) acc[r][m] = part[r][m][0] + part[r][m][1];
#pragma unroll
        for (int r = 0; r < RB; ++r)
#pragma unroll
            for (int m = 0; m < M; ++m) acc[r][m] = wave_sum_valu(acc[r][m]) * rinv[m];

        // the next round's rows are on their way while this one is finished
        const int cur_u = u, cur_base = base;
        const bool cur_active = active;
        base += gridDim.x * GV_WAVES;
        const bool more = base < units;
        if (more) {
            active = base + wave_in_block < units;
            u = active ? base + wave_in_block : units - 1;
            ask_for_rows(u);
        }

        // ---- epilogue: lane l finishes result l % OUTS of token l / OUTS
        if (EPI == GV_PLAIN) {
            const int n = cur_u * RB + my;
            if (cur_active && finishing && n < a.N) {
                const float v = gv_pick<RB, M>(acc, my, my_m);
                if (a.out_f32) reinterpret_cast<float *>(a.Y)[(size_t)my_m * a.ldy + n] = v;
                else reinterpret_cast<bf16_t *>(a.Y)[(size_t)my_m * a.ldy + n].bits = float_to_bf16_bits(v);
            }
        } else if (EPI == GV_SWIGLU) {
            const int col = cur_u * PAIRS + my;
            if (cur_active && finishing && col < a.inter) {
                const float g = gv_pick<RB, M>(acc, 2 * my, my_m), up = gv_pick<RB, M>(acc, 2 * my + 1, my_m);
                reinterpret_cast<bf16_t *>(a.Y)[(size_t)my_m * a.ldy + col].bits =
                    float_to_bf16_bits(g * (1.f / (1.f + expf(-g))) * up);
            }
        } else if (EPI == GV_RESID) {
            float sq = 0.f;
            if (cur_active && finishing && my_n < a.N) {
                const uint16_t sb = float_to_bf16_bits(e0 + gv_pick<RB, M>(acc, my, my_m));
                a.hidden[(size_t)my_m * a.N + my_n].bits = sb;
                const float sv = bf16_bits_to_float(sb);
                sq = sv * sv;
                a.scaled_out[(size_t)my_m * a.N + my_n].bits = float_to_bf16_bits(sv * e1);
            }
            // the unit's rows of a token sit in RB neighbouring lanes
#pragma unroll
            for (int off = 1; off < RB; off <<= 1) sq += __shfl_xor(sq, off, KVA_WAVE);
            if (finishing && my == 0) block_ss[parity][wave_in_block][my_m] = sq;
            __syncthreads();
            if (threadIdx.x < M) {
                float ss = 0.f;
#pragma unroll
                for (int wv = 0; wv < GV_WAVES; ++wv) ss += block_ss[parity][wv][threadIdx.x];
                a.sumsq_out[(size_t)threadIdx.x * a.parts_out + cur_base / GV_WAVES] = ss;
            }
            parity ^= 1;
        } else {   // GV_ROPE
            const int D = a.head_dim, per_head = D / 2 / PAIRS;
            const int head = cur_u / per_head, f = my_n;
            const bool rotated = head < a.nq + a.nkv;
            if (cur_active && finishing && (head < a.nq || slot >= 0)) {
                const int page = slot >= 0 ? slot / a.page_size : 0;
                const int off = slot >= 0 ? slot - page * a.page_size : 0;
                // the product is rounded to the storage type before it is rotated, as a product
                // followed by a rotation kernel would have it
                const float va = gv_round_bf16(gv_pick<RB, M>(acc, 2 * my, my_m));
                const float vb = gv_round_bf16(gv_pick<RB, M>(acc, 2 * my + 1, my_m));
                if (rotated) {
                    float o1 = va, o2 = vb;
                    if (a.cos_t != nullptr) {
                        o1 = va * e0 - vb * e1;
                        o2 = va * e1 + vb * e0;
                    }
                    if (head < a.nq) {
                        bf16_t *dst = reinterpret_cast<bf16_t *>(a.Y) + (size_t)my_m * a.ldy + (size_t)head * D + f;
                        dst[0].bits = float_to_bf16_bits(o1);
                        dst[D / 2].bits = float_to_bf16_bits(o2);
                    } else {
                        bf16_t *pg = a.k_cache + ((size_t)page * a.nkv + (head - a.nq)) * a.page_size * D;
                        const int kc = kva_k_chunk(D);
                        pg[kva_k_at(off, f, a.page_size, kc)].bits = float_to_bf16_bits(o1);
                        pg[kva_k_at(off, f + D / 2, a.page_size, kc)].bits = float_to_bf16_bits(o2);
                    }
                } else {
                    bf16_t *dst = a.v_cache + (((size_t)page * a.nkv + (head - a.nq - a.nkv)) * D + f) * a.page_size + off;
                    dst[0].bits = float_to_bf16_bits(va);
                    dst[(size_t)(D / 2) * a.page_size].bits = float_to_bf16_bits(vb);
                }
            }
        }
        if (!more) break;
    }
}

// Rows a wavefront has in flight, by the vectors a lane loads per row (K / 512) and the epilogue.
// At K of 1,536 and 2,048 two rows (8 KiB) are enough and give twice the wavefronts, which the
// narrow matrices need to reach every compute unit (output 4.2 -> 3.9 us, gate/up 12.6 -> 12.4);
// the rotation epilogue is no faster for it and keeps four.
int rows_in_flight(int kv, int epi) {
    if (kv <= 2) return 8;
    if (kv <= 4) return epi == GV_ROPE ? 4 : 2;
    if (kv <= 8) return 2;
    return (epi == GV_SWIGLU || epi == GV_ROPE) ? 2 : 1;
}

template <int EPI>
int launch(const GemvArgs &a, hipStream_t stream) {
    const int kv = a.K / 512;
    constexpr bool paired = EPI == GV_SWIGLU || EPI == GV_ROPE;
    // a wavefront per unit of rows, up to 8,192 wavefronts: beyond that a wavefront takes several
    // units and loads its token registers once for all of them
    const int rb = rows_in_flight(kv, EPI);
    long units;
    if (EPI == GV_SWIGLU) units = (a.inter + rb / 2 - 1) / (rb / 2);
    else if (EPI == GV_ROPE) units = (long)(a.nq + 2 * a.nkv) * (a.head_dim / 2 / (rb / 2));
    else units = (a.N + rb - 1) / rb;
    const dim3 grid((unsigned)std::min<long>(2048, (units + GV_WAVES - 1) / GV_WAVES)), block(64 * GV_WAVES);
    if constexpr (EPI == GV_RESID) {
        if (a.part_o != nullptr) {
#define GVP(KVV, RBB)                                                                                          \
    if (a.M == 1 && a.parts > GV_MERGE_PARTS)                                                                  \
        hipLaunchKernelGGL((gemv_kernel<KVV, 1, RBB, GV_RESID, GV_MERGE_MAX_PARTS>), grid, block, 0, stream, a); \
    else if (a.M == 1)                                                                                         \
        hipLaunchKernelGGL((gemv_kernel<KVV, 1, RBB, GV_RESID, GV_MERGE_PARTS>), grid, block, 0, stream, a);   \
    else hipLaunchKernelGGL((gemv_kernel<KVV, 2, RBB, GV_RESID, GV_MERGE_PARTS>), grid, block, 0, stream, a)
            switch (kv) {
            case 1: GVP(1, 8); break;
            case 2: GVP(2, 8); break;
            case 3: GVP(3, 2); break;
            case 4: GVP(4, 2); break;
            case 5: GVP(5, 2); break;
            case 6: GVP(6, 2); break;
            case 7: GVP(7, 2); break;
            case 8: GVP(8, 2); break;
            default:
                kva_set_error("gemv: K=%d has no instance that adds up partial results", a.K);
                return KVA_ERR_ARG;
            }
#undef GVP
            KVA_CHECK_LAUNCH("gemv");
            return KVA_OK;
        }
    }
#define GV(KVV, MM, RBB) hipLaunchKernelGGL((gemv_kernel<KVV, MM, RBB, EPI>), grid, block, 0, stream, a)
#define GVM(KVV, RBB)                                                                          \
    if (a.M == 1) GV(KVV, 1, RBB); else GV(KVV, 2, RBB)
    switch (kv) {
    case 1: GVM(1, 8); break;
    case 2: GVM(2, 8); break;
    case 3: if constexpr (EPI == GV_ROPE) { GVM(3, 4); } else { GVM(3, 2); } break;
    case 4: if constexpr (EPI == GV_ROPE) { GVM(4, 4); } else { GVM(4, 2); } break;
    case 5: GVM(5, 2); break;
    case 6: GVM(6, 2); break;
    case 7: GVM(7, 2); break;
    case 8: GVM(8, 2); break;
    case 10: if constexpr (paired) { GVM(10, 2); } else { GVM(10, 1); } break;
    case 12: if constexpr (paired) { GVM(12, 2); } else { GVM(12, 1); } break;
    case 14: if constexpr (paired) { GVM(14, 2); } else { GVM(14, 1); } break;
    case 16: if constexpr (paired) { GVM(16, 2); } else { GVM(16, 1); } break;
    default:
        kva_set_error("gemv: K=%d has no instance", a.K);
        return KVA_ERR_ARG;
    }
#undef GVM
#undef GV
    KVA_CHECK_LAUNCH("gemv");
    return KVA_OK;
}

bool k_has_instance(int K) {
    if (K < 512 || K % 512 != 0) return false;
    const int kv = K / 512;
    return kv <= 8 || kv == 10 || kv == 12 || kv == 14 || kv == 16;
}

} // namespace

// One or two tokens, K a multiple of 512 with an instance (512 .. 4096 in steps of 512, 5120,
// 6144, 7168, 8192).
extern "C" int kva_gemv_supported(int M, int N, int K) {
    return (M >= 1 && M <= 2 && N >= 1 && k_has_instance(K)) ? 1 : 0;
}

// Partial sums of squares per token that a residual-epilogue product with N columns and K inputs writes.
extern "C" int kva_gemv_sumsq_parts(int N, int K) {
    if (!k_has_instance(K)) return 0;
    const int rb = rows_in_flight(K / 512, GV_RESID);
    const int units = (N + rb - 1) / rb;
    return (units + GV_WAVES - 1) / GV_WAVES;
}

// The rotation epilogue takes heads whose half is a multiple of the pairs a wavefront works on.
extern "C" int kva_gemv_qkv_rope_supported(int M, int K, int head_dim) {
    if (!kva_gemv_supported(M, 1, K) || head_dim < 2 || head_dim % 2 != 0) return 0;
    const int pairs = rows_in_flight(K / 512, GV_ROPE) / 2;
    return (head_dim / 2) % pairs == 0 ? 1 : 0;
}

static int fill_common(GemvArgs &a, const void *X, const void *W, int M, int N, int K, int ldx, const float *sumsq,
                       int sumsq_parts, int norm_width, float eps) {
    KVA_REQUIRE(kva_gemv_supported(M, N, K), "gemv: M=%d N=%d K=%d not supported (1-2 rows, K a multiple of 512 "
                "with an instance)", M, N, K);
    KVA_REQUIRE(ldx >= K && ldx % 8 == 0, "gemv: X row stride %d must be a multiple of 8 and >= K", ldx);
    KVA_REQUIRE(sumsq == nullptr || (sumsq_parts >= 1 && norm_width >= 1),
                "gemv: row scaling needs a part count and the norm's width");
    a.X = (const bf16_t *)X; a.W = (const bf16_t *)W; a.M = M; a.N = N; a.K = K; a.ldx = ldx;
    a.sumsq = sumsq; a.sumsq_parts = sumsq_parts; a.norm_width = norm_width; a.eps = eps;
    return KVA_OK;
}

// W: the plain row-major [N, K] weight.  mode 0: Y bf16 [M, N]; mode 1: Y fp32 [M, N]; mode 2: W is
// [2 inter, K] = [gate; up], Y bf16 [M, inter] = silu(X gate^T) * (X up^T); mode 3: hidden[M, N] +=
// X W^T in place, scaled_out[M, N] = round(hidden * next_w), sumsq_out[M, kva_gemv_sumsq_parts(N, K)].
extern "C" int kva_gemv(void *Y, const void *X, const void *W, int M, int N, int K, int ldx, int ldy, int mode,
                        const float *sumsq, int sumsq_parts, int norm_width, float eps, void *hidden,
                        const void *next_w, int next_w_f32, void *scaled_out, float *sumsq_out,
                        hipStream_t stream) {
    GemvArgs a = {};
    const int rc = fill_common(a, X, W, M, N, K, ldx, sumsq, sumsq_parts, norm_width, eps);
    if (rc != KVA_OK) return rc;
    KVA_REQUIRE(mode >= 0 && mode <= 3, "gemv: unknown mode %d", mode);
    if (mode == 3) {
        KVA_REQUIRE(hidden && scaled_out && sumsq_out, "gemv: the residual epilogue needs hidden, scaled_out and sumsq_out");
        a.hidden = (bf16_t *)hidden; a.next_w = next_w; a.next_w_f32 = next_w_f32;
        a.scaled_out = (bf16_t *)scaled_out; a.sumsq_out = sumsq_out;
        a.parts_out = kva_gemv_sumsq_parts(N, K);
        return launch<GV_RESID>(a, stream);
    }
    KVA_REQUIRE(Y != nullptr, "gemv: no output");
    a.Y = Y; a.ldy = ldy; a.out_f32 = mode == 1 ? 1 : 0;
    if (mode == 2) {
        KVA_REQUIRE(N % 2 == 0 && ldy >= N / 2, "gemv: a joined [gate; up] matrix needs an even row count and room for its half");
        a.inter = N / 2;
        return launch<GV_SWIGLU>(a, stream);
    }
    KVA_REQUIRE(ldy >= N, "gemv: Y row stride %d is smaller than its %d columns", ldy, N);
    return launch<GV_PLAIN>(a, stream);
}

// Whether kva_gemv_merged takes these sizes: one or two tokens, K up to 4,096 with an instance,
// heads of a multiple of 8 features that divide K, 2 to kva_gemv_merge_max_parts(M) partial results a row.
extern "C" int kva_gemv_merge_max_parts(int M) { return M == 1 ? GV_MERGE_MAX_PARTS : GV_MERGE_PARTS; }
extern "C" int kva_gemv_merged_supported(int M, int N, int K, int head_dim, int parts) {
    return (kva_gemv_supported(M, N, K) && K <= 4096 && head_dim >= 8 && head_dim % 8 == 0 && K % head_dim == 0 &&
            parts >= 2 && parts <= kva_gemv_merge_max_parts(M)) ? 1 : 0;
}

// kva_gemv's mode 3 (hidden[M, N] += X W^T, the next norm prepared) with X = the attention output
// of M decoded tokens given as what the attention kernel left per key range: part_o
// [M * (K / head_dim), parts, head_dim] fp32, part_ml [M * (K / head_dim), parts, 2] fp32
// (maximum in the base-2 domain, sum).  Stands for the merge kernel followed by kva_gemv.
extern "C" int kva_gemv_merged(const float *part_o, const float *part_ml, int parts, int head_dim, const void *W,
                               int M, int N, int K, void *hidden, const void *next_w, int next_w_f32,
                               void *scaled_out, float *sumsq_out, hipStream_t stream) {
    KVA_REQUIRE(kva_gemv_merged_supported(M, N, K, head_dim, parts),
                "gemv_merged: M=%d N=%d K=%d head_dim=%d parts=%d not supported", M, N, K, head_dim, parts);
    KVA_REQUIRE(part_o && part_ml && ((uintptr_t)part_o % 16) == 0 && ((uintptr_t)part_ml % 8) == 0,
                "gemv_merged: aligned partial results are needed");
    KVA_REQUIRE(hidden && scaled_out && sumsq_out && W, "gemv_merged: hidden, scaled_out, sumsq_out and W are needed");
    GemvArgs a = {};
    a.W = (const bf16_t *)W; a.M = M; a.N = N; a.K = K; a.ldx = K;
    a.part_o = part_o; a.part_ml = part_ml; a.parts = parts; a.part_head_dim = head_dim;
    a.hidden = (bf16_t *)hidden; a.next_w = next_w; a.next_w_f32 = next_w_f32;
    a.scaled_out = (bf16_t *)scaled_out; a.sumsq_out = sumsq_out;
    a.parts_out = kva_gemv_sumsq_parts(N, K);
    return launch<GV_RESID>(a, stream);
}

// The joined Q/K/V projection of one or two tokens with rotation and cache write: as
// kva_gemm_skinny_qkv_rope, over the plain row-major weight.
extern "C" int kva_gemv_qkv_rope(void *q_out, int ldq, const void *X, const void *W, int M, int K, int ldx, int nq,
                                 int nkv, int head_dim, const float *sumsq, int sumsq_parts, int norm_width,
                                 float eps, const float *cos_t, const float *sin_t, const int *positions,
                                 const int *slots, void *k_cache, void *v_cache, int page_size,
                                 hipStream_t stream) {
    KVA_REQUIRE(nq >= 1 && nkv >= 1, "gemv_qkv_rope: bad head counts %d, %d", nq, nkv);
    KVA_REQUIRE(kva_gemv_qkv_rope_supported(M, K, head_dim), "gemv_qkv_rope: M=%d K=%d head_dim=%d not supported", M, K,
                head_dim);
    GemvArgs a = {};
    const int rc = fill_common(a, X, W, M, (nq + 2 * nkv) * head_dim, K, ldx, sumsq, sumsq_parts, norm_width, eps);
    if (rc != KVA_OK) return rc;
    KVA_REQUIRE(ldq >= nq * head_dim, "gemv_qkv_rope: Q row stride %d does not fit", ldq);
    KVA_REQUIRE((cos_t == nullptr) == (sin_t == nullptr), "gemv_qkv_rope: one table missing");
    KVA_REQUIRE(cos_t == nullptr || positions != nullptr, "gemv_qkv_rope: rotation needs positions");
    KVA_REQUIRE(slots == nullptr || (k_cache && v_cache && page_size > 0),
                "gemv_qkv_rope: cache write asked for without cache or page size");
    a.Y = q_out; a.ldy = ldq;
    a.cos_t = cos_t; a.sin_t = sin_t; a.positions = positions; a.slots = slots;
    a.k_cache = (bf16_t *)k_cache; a.v_cache = (bf16_t *)v_cache;
    a.nq = nq; a.nkv = nkv; a.head_dim = head_dim; a.page_size = page_size;
    return launch<GV_ROPE>(a, stream);
}
