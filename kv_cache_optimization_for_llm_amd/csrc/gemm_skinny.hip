// Y[M,N] = X[M,K] * W[N,K]^T for few rows (M <= 64): the decode-time matrix products, on the
// matrix cores, bound by streaming W from HBM exactly once.
//
// Stands where the reference calls cublasGemmEx with n = active rows
// (base/src/engine.cu:1040-1117, 1141-1159, 1166-1253).  bf16 operands, fp32 accumulation.
//
// Mapping (64-lane wavefronts, mfma_f32_16x16x32_bf16):
//   A = 16 rows of W (an "n-tile") x 32 of K      lane (r, g) loads W[n0 + r][k + 8g .. 8g+7]
//   B = X^T, 32 of K x 16 tokens                   lane (r, g) loads X[m0 + r][k + 8g .. 8g+7]
//   D[n0 + 4g + i][m0 + r]                         -> 4 consecutive outputs of token m0 + r
// W comes pre-tiled ([n-tile][K/32][g 4][r 16][8], made once at load time): a wave's 1 KiB per step is
// contiguous.  Both operands are read from memory directly in operand layout (16 bytes per lane).  A wave
// keeps one accumulator per 16-token tile (MT = ceil(M / 16) <= 4) and per n-tile it owns
// (NTW = 1, 2 or 4: wide matrices give a wave several n-tiles so that a loaded X fragment is
// used several times), so W is read once whatever M is.  K is split over `k_waves` wavefronts of
// a workgroup (partials summed through LDS in a fixed order) so that narrow matrices still put
// about 2048 waves on the 256 compute units.  A wave keeps up to 8 steps of its K range in flight.
//
// A column of the result depends only on its own token's row of X, and with at most 16 rows the
// order of its sum does not depend on M: bitwise the same result in any batch that small.
//
// Two more shapes of the same loop.  Above 16 rows (gated and vocabulary-sized products) the waves
// of a workgroup that work on the same K range stage X through LDS, once for all of them, instead
// of each loading MT fragments of X per fragment of W.  Matrices with at most half as many tile
// groups as the chip has compute units are cut into half tiles: two workgroups share a tile, each
// taking 8 of its 16 rows, because the chip's 6 TB/s are 24 GB/s from each of 256 compute units and
// a matrix that leaves half of them without a workgroup gets half of it.
//
// Row scaling.  With `sumsq` the rows of X are un-normalised norm inputs: X = round(h * w_norm)
// and sumsq[m, 0..parts) are partial sums of h[m,:]^2; the product is multiplied by
// rsqrt(sum / norm_width + eps) per token at the end (RMSNorm finished inside the product; the
// reference runs rmsNormKernel, base/src/kernels.cu:10-36, before the GEMM).
//
// Epilogues.
//   EPI_PLAIN   bf16 or fp32 output.
//   EPI_SWIGLU  W is a joined [gate; up] matrix; output silu(gate) * up (reference siluKernel,
//               base/src/kernels.cu:45-52): the 2*I-wide intermediate never goes to memory.
//   EPI_RESID   the residual stream takes the product in place, hidden = round(hidden + y)
//               (reference residualKernel, base/src/kernels.cu:38-43), and the sum is prepared for
//               the next norm: scaled = round(hidden * w_next) and one partial sum of squares per
//               (token, n-tile).
//   EPI_ROPE    W is the joined [q; k; v] projection.  A wave owns two tiles of one head: for a
//               Q or K head the tiles with features f and f + d/2 (the rotate-half pair,
//               reference ropePackedKernel, base/src/kernels.cu:289-319), for a V head two
//               neighbouring tiles.  The product is rounded to bf16 as a separate GEMM would
//               leave it, rotated by the token's position with the fp32 cos/sin tables, and goes
//               to its place: Q to a [M, nq*d] buffer, K and V to the token's slot of the paged
//               cache (reference scatterKVPackedKernel, paged_attention/src/kernels.cu:335-363).
#include "common.h"
#include "kv_layout.h"
#include <math.h>
#include <type_traits>

typedef __bf16 gb16x8 __attribute__((ext_vector_type(8)));
typedef float gf32x4 __attribute__((ext_vector_type(4)));

union GFrag8 {
    gb16x8 v;
    uint4 u4;
};

enum { EPI_PLAIN = 0, EPI_SWIGLU = 1, EPI_RESID = 2, EPI_ROPE = 3 };

struct SkinnyArgs {
    const bf16_t *X;
    const bf16_t *W;
    void *Y;                 // EPI_PLAIN / EPI_SWIGLU output
    int M, N, K, ldx, ldy;
    int k_waves, out_f32, inter;
    // row scaling of the input (optional)
    const float *sumsq;
    int sumsq_parts, norm_width;
    float eps;
    // EPI_RESID
    bf16_t *hidden;          // [M, N] in/out
    const void *next_w;      // [N] weight of the next norm (bf16 or fp32), may be null
    int next_w_f32;
    bf16_t *scaled_out;      // [M, N]
    float *sumsq_out;        // [M, n_tiles]
    // EPI_ROPE (Y is the Q output [M, nq * head_dim] with row stride ldy)
    const float *cos_t, *sin_t;   // [positions, head_dim / 2], both null: no rotation
    const int *positions;         // [M]
    const int *slots;             // [M] cache slot per token (negative: no write), null: no cache write
    bf16_t *k_cache, *v_cache;    // [pages, nkv, d / 8, page, 8] (kv_layout.h) and [pages, nkv, d, page]
    int nq, nkv, head_dim, page_size;
    // half tiles: a tile group takes 8 of its tiles' 16 rows (see choose_half_tiles)
    int half;
    // X (x_tiled) or the bf16 result (y_tiled) laid out [columns / 8][tile_rows][8], the order in
    // which the lanes of the consuming product read it (neighbouring lanes take the same 8 columns
    // of neighbouring rows: contiguous bytes; row-major they take pieces a row apart).  tile_rows
    // is M rounded up to 16, or 8 for up to 8 rows: lanes 8..15 of a lane group then read rows
    // 0..7 again (the same addresses, no traffic) instead of 8 rows of padding.  A private layout
    // between two products of one part.
    int x_tiled, y_tiled, tile_rows;
    // K cut into k_slices ranges, one per blockIdx.y, each leaving its own fp32 partial product
    // [M, N] in Y (slice s at Y + s * M * ldy): for matrices with too few tiles to fill the chip
    // with whole-K workgroups when the rows go through LDS (see kva_gemm_skinny_partials)
    int k_slices;
};

// XL: the waves of a workgroup that work on the same K range (one per tile group) share X through
// LDS instead of each loading it (see the main loop).
template <int MT, int NTW, int EPI, bool XL = false>
__global__ void __launch_bounds__(XL ? 512 : 1024) gemm_skinny_kernel(const SkinnyArgs a) {
    extern __shared__ __align__(16) float red[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int waves = blockDim.x >> 6;
    const int k_waves = a.k_waves;
    const int groups_per_wg = waves / k_waves;                 // tile groups (NTW tiles) per workgroup
    const int kpart = wave % k_waves;
    const int r = lane & 15, g = lane >> 4;
    // With half tiles two waves (of different workgroups) share a tile group: each takes 8 of the
    // 16 rows of its tiles.  The upper 8 lanes-rows of the matrix-core operand repeat the lower
    // ones, so lane groups 2 and 3 end up with copies of the results and store nothing.
    const int unit = blockIdx.x * groups_per_wg + wave / k_waves;
    const int group = a.half ? unit >> 1 : unit;
    const int hrow = a.half ? (unit & 1) * 8 : 0;
    const int wrow = a.half ? hrow + (r & 7) : r;               // row of a tile that lane (r, g) loads
    const int orow = a.half ? hrow + 4 * (g & 1) : 4 * g;       // first of the 4 rows whose results it holds
    const bool lane_on = !a.half || g < 2;
    const int rows = EPI == EPI_SWIGLU ? a.inter : a.N;        // output columns
    const int n_tiles = (rows + 15) / 16;
    // EPI_SWIGLU: a wave's two tiles are the gate tile and the up tile of the same columns
    const int out_tiles = (EPI == EPI_SWIGLU || EPI == EPI_ROPE) ? 1 : NTW;
    const int tile0 = group * out_tiles;
    // EPI_ROPE: group = (head, j) with j in [0, d/32); N is a multiple of 32
    const bool group_ok = EPI == EPI_ROPE ? group < n_tiles / 2 : tile0 < n_tiles;
    int rope_head = 0, rope_j = 0;
    bool rope_rotated = false;
    if (EPI == EPI_ROPE) {
        const int hp = a.head_dim / 32;
        rope_head = group / hp;
        rope_j = group - rope_head * hp;
        rope_rotated = rope_head < a.nq + a.nkv;
    }
    const int K = a.K;
    const int kslice = K / a.k_slices;
    const int kper = kslice / k_waves;
    const int kbeg = (int)blockIdx.y * kslice + kpart * kper, kend = kbeg + kper;

    // W is stored tiled: [n-tile][K / 32][g][r][8 of K], so the 1 KiB a wave needs per step is
    // contiguous, in the order of its lanes (lane r + 16 g takes bytes 16 (r + 16 g) ..), and a
    // wave walks its n-tile as one sequential stream.  For EPI_SWIGLU the up tiles follow the
    // gate tiles.
    const bf16_t *wp[NTW];
#pragma unroll
    for (int t = 0; t < NTW; ++t) {
        int tile = EPI == EPI_SWIGLU ? tile0 + t * n_tiles : tile0 + t;
        if (EPI == EPI_ROPE) {
            const int first = rope_head * (a.head_dim / 16);
            tile = rope_rotated ? first + rope_j + t * (a.head_dim / 32) : first + 2 * rope_j + t;
        }
        const int last = (EPI == EPI_SWIGLU ? 2 * n_tiles : n_tiles) - 1;
        if (tile > last) tile = last;
        wp[t] = a.W + (size_t)tile * (size_t)(K / 32) * 512 + (16 * g + wrow) * 8;
    }
    const bf16_t *xr[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = mt * 16 + r;
        xr[mt] = a.x_tiled ? a.X + ((size_t)g * a.tile_rows + (a.tile_rows == 8 ? (m & 7) : m)) * 8
                           : a.X + (size_t)(m < a.M ? m : 0) * a.ldx + 8 * g;
    }

    gf32x4 acc[NTW][MT];
#pragma unroll
    for (int t = 0; t < NTW; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[t][mt] = gf32x4{0.f, 0.f, 0.f, 0.f};

    // The first wave of a tile group also needs, per token, the sum of squares that finishes the
    // input norm: lane group g adds a contiguous quarter of the partial sums.  The loads are
    // issued here, ahead of the main loop, and (for up to 32 tokens) their values are only added
    // after it, so this wave starts streaming W as early as the others; with more token tiles
    // there are no registers to hold them and they are added at once.
    constexpr int DV = (MT == 1 && NTW <= 2) ? 8 : ((MT == 1 || (MT == 2 && NTW <= 2)) ? 4 : 0);   // vectors of 4 sums held per token tile
    float4 dv[MT][DV > 0 ? DV : 1];
    int dv_end[MT];
    float ssum[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) { ssum[mt] = 0.f; dv_end[mt] = 0; }
    if (a.sumsq != nullptr && kpart == 0 && group_ok) {
        const int parts = a.sumsq_parts;
        const int q = (parts + 3) / 4;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = mt * 16 + r;
            if (m >= a.M) continue;
            const float *sp = a.sumsq + (size_t)m * parts;
            int lo = g * q;
            const int hi = (lo + q < parts) ? lo + q : parts;
            float s = 0.f;
            if ((parts & 15) == 0) {
                if (DV > 0) {
                    dv_end[mt] = hi - lo;
#pragma unroll
                    for (int j = 0; j < DV; ++j) {
                        const int p = lo + 4 * j;
                        dv[mt][j] = *reinterpret_cast<const float4 *>(sp + (p < hi ? p : hi - 4));
                    }
                    lo += 4 * DV;
                }
                // 8 vectors of 4 at a time, all loaded before any is added (a load past the
                // lane's quarter repeats its last vector and is not counted)
                for (int base = lo; base < hi; base += 32) {
                    float4 v[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const int p = base + 4 * j;
                        v[j] = *reinterpret_cast<const float4 *>(sp + (p < hi ? p : hi - 4));
                    }
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        s += (base + 4 * j < hi) ? (v[j].x + v[j].y) + (v[j].z + v[j].w) : 0.f;
                }
            } else {
                for (int p = lo; p < hi; ++p) s += sp[p];
            }
            ssum[mt] = s;
        }
    }

    // Operands of the epilogue that do not depend on the product are loaded here as well (the
    // token's position, its cache slot and its cos/sin entries; the residual stream and the next
    // norm's weight), so that no memory latency is left after the main loop.
    int pre_slot[MT];
    float4 pre_cos[MT], pre_sin[MT];
    uint2 pre_hidden[MT];
    // the next norm's weight as loaded (converted in the epilogue: a conversion here would wait for the load)
    float4 pre_wn_f = make_float4(1.f, 1.f, 1.f, 1.f);
    uint2 pre_wn_b = make_uint2(0x3f803f80u, 0x3f803f80u);
    constexpr bool kPreRope = EPI == EPI_ROPE && MT <= 2;
    constexpr bool kPreResid = EPI == EPI_RESID && NTW == 1 && MT <= 2;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        pre_slot[mt] = -1;
        pre_cos[mt] = make_float4(1.f, 1.f, 1.f, 1.f);
        pre_sin[mt] = make_float4(0.f, 0.f, 0.f, 0.f);
        pre_hidden[mt] = make_uint2(0u, 0u);
    }
    int pre_pos[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) pre_pos[mt] = 0;
    if (kPreRope && kpart == 0 && group_ok) {
        // slot and position now; the cos/sin entries, whose address needs the position, after the
        // main loop (a wait here would hold back this wave's stream of W)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = mt * 16 + r;
            if (m >= a.M) continue;
            if (a.slots != nullptr && rope_head >= a.nq) pre_slot[mt] = a.slots[m];
            if (rope_rotated && a.cos_t != nullptr) pre_pos[mt] = a.positions[m];
        }
    }
    const bool resid_vec = kPreResid && (a.N % 4 == 0) && tile0 * 16 + orow + 3 < rows;
    if (kPreResid && kpart == 0 && group_ok && resid_vec) {
        const int n = tile0 * 16 + orow;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = mt * 16 + r;
            if (m < a.M) pre_hidden[mt] = *reinterpret_cast<const uint2 *>(a.hidden + (size_t)m * a.N + n);
        }
        // both forms are loaded, one of them from a place that is always there (X), so that no
        // branch joins here with a load in flight
        const bool wf = a.next_w != nullptr && a.next_w_f32, wb = a.next_w != nullptr && !a.next_w_f32;
        pre_wn_f = *(wf ? reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(a.next_w) + n)
                        : reinterpret_cast<const float4 *>(a.X));
        pre_wn_b = *(wb ? reinterpret_cast<const uint2 *>(reinterpret_cast<const bf16_t *>(a.next_w) + n)
                        : reinterpret_cast<const uint2 *>(a.X));
    }

    // ---- the main loop.  Rows of X past M are read from row 0 instead (their columns of the
    // result are never stored), so the loop body has no branch.
    if constexpr (XL) {
        // More than 16 tokens: every wave needs MT fragments of X per fragment of W, and loading
        // them per wave makes X (from L2, in half-used cache lines) the larger stream.  Here the
        // waves of the workgroup that share a K range stage X through LDS: chunks of 64 of K,
        // each loaded once per workgroup in full 128-byte lines, double-buffered, one barrier per
        // chunk.  A token's row of a chunk is 128 bytes; tokens r and r + 8 of a tile lie next to
        // each other and the 16-byte units of a row are XOR-swizzled with the token, so that the
        // operand reads (16 tokens x 16 bytes at the same K) touch every bank once.  W is
        // fetched two chunks ahead into two register buffers.  All waves run the loop (barriers);
        // a wave past the last tile group computes a copy of the last one and stores nothing.
        constexpr int KC = 64, ROWS = MT * 16, UNITS = ROWS * (KC / 8);
        const int J = groups_per_wg;
        const int sj = wave / k_waves;                          // place among the waves of this K range
        char *xbase = reinterpret_cast<char *>(red) + (size_t)kpart * 2 * ROWS * 128;
        const int n_chunks = (kper + KC - 1) / KC;
        // X and W of a chunk are requested NB chunks ahead (one chunk ahead left every turn of the
        // loop waiting for L2; three and four ahead, 201 and 230 registers, were measured no
        // faster: gate/up at 64 rows 19.6 / 20.0 / 19.8 us).  The staging registers are indexed by
        // constants only (every loop over them is unrolled), or they would end up in scratch memory.
        constexpr int NB = 2;
        // Every workgroup reads the same rows of X, and workgroups that walk K in the same order ask
        // L2 for the same lines at the same time.  Each workgroup of a die starts at a chunk of its
        // own and wraps around (the sum over K has the same terms in another order).  Decode steps of
        // 64 requests at the 1B sizes 1.379 -> 1.355 ms, the LM head at 64 rows 96 -> 91 us, gate/up
        // 18.9 -> 18.8; starting at blockIdx % chunks instead (the same start within a die, another
        // on every die) gave gate/up 17.9 but the LM head 99.8 and the step 1.398.  For the kernel
        // below, whose waves read X themselves, the same rotation changed nothing.
        const int rot = __builtin_amdgcn_readfirstlane((int)((blockIdx.x >> 3) % (unsigned)n_chunks));   // workgroups b, b + 8, .. share a die's L2
        auto place = [&](int c) -> int { const int pc = c + rot; return pc >= n_chunks ? pc - n_chunks : pc; };
        struct XRegs { uint4 v0, v1, v2, v3; };
        XRegs xs[NB];
#pragma unroll
        for (int i = 0; i < NB; ++i)
            xs[i] = XRegs{make_uint4(0, 0, 0, 0), make_uint4(0, 0, 0, 0), make_uint4(0, 0, 0, 0), make_uint4(0, 0, 0, 0)};
        auto load_unit = [&](int i, int c) -> uint4 {
            int u = (i * J + sj) * 64 + lane;
            if (u >= UNITS) u = 0;
            const int q = u >> 3, c16 = u & 7;
            const int row = (q & ~15) | ((q >> 1) & 7) | ((q & 1) << 3);
            int k = kbeg + place(c) * KC + c16 * 8;
            if (k >= kend) k = kbeg;
            return *reinterpret_cast<const uint4 *>(a.X + (size_t)(row < a.M ? row : 0) * a.ldx + k);
        };
        auto store_unit = [&](int i, int c, const uint4 &v) {
            const int u = (i * J + sj) * 64 + lane;
            const int q = u >> 3, c16 = u & 7;
            const int row = (q & ~15) | ((q >> 1) & 7) | ((q & 1) << 3);
            if (u < UNITS)
                *reinterpret_cast<uint4 *>(xbase + (c & 1) * ROWS * 128 + q * 128 + ((c16 ^ (row & 7)) << 4)) = v;
        };
        auto load_x = [&](XRegs &x, int c) {
            x.v0 = load_unit(0, c);
            if constexpr (MT > 1) x.v1 = load_unit(1, c);
            if constexpr (MT > 2) x.v2 = load_unit(2, c);
            if constexpr (MT > 3) x.v3 = load_unit(3, c);
        };
        auto store_x = [&](const XRegs &x, int c) {
            store_unit(0, c, x.v0);
            if constexpr (MT > 1) store_unit(1, c, x.v1);
            if constexpr (MT > 2) store_unit(2, c, x.v2);
            if constexpr (MT > 3) store_unit(3, c, x.v3);
        };
        GFrag8 wbuf[NB][2][NTW];
        auto load_w = [&](GFrag8 (&w)[2][NTW], int c) {
#pragma unroll
            for (int st = 0; st < 2; ++st) {
                int k = kbeg + place(c) * KC + st * 32;
                if (k >= kend) k = kbeg;                        // half a chunk at the end: loaded from a valid place, not used
#pragma unroll
                for (int t = 0; t < NTW; ++t) w[st][t].u4 = load_streamed_u4(wp[t] + (size_t)k * 16);
            }
        };
        auto compute = [&](GFrag8 (&w)[2][NTW], int c) {
            const char *buf = xbase + (c & 1) * ROWS * 128 + (((r & 7) << 1) + (r >> 3)) * 128;
#pragma unroll
            for (int st = 0; st < 2; ++st) {
                if (kbeg + place(c) * KC + st * 32 < kend) {
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt) {
                        GFrag8 x;
                        x.u4 = *reinterpret_cast<const uint4 *>(buf + mt * 16 * 128 + (((st * 4 + g) ^ (r & 7)) << 4));
#pragma unroll
                        for (int t = 0; t < NTW; ++t)
                            acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[st][t].v, x.v, acc[t][mt], 0, 0, 0);
                    }
                }
            }
        };
#pragma unroll
        for (int i = 0; i < NB; ++i)
            if (i == 0 || i < n_chunks) load_x(xs[i], i);
#pragma unroll
        for (int i = 0; i < NB; ++i)
            if (i == 0 || i < n_chunks) load_w(wbuf[i], i);
        // NB chunks per turn while every load of the turn exists: no branch in the body, so the
        // waits count exactly and the loads issued last stay in flight across them.
        int c = 0;
        for (; c + 2 * NB - 1 < n_chunks; c += NB) {
#pragma unroll
            for (int i = 0; i < NB; ++i) {
                store_x(xs[i], c + i);
                __syncthreads();
                load_x(xs[i], c + i + NB);
                compute(wbuf[i], c + i);
                load_w(wbuf[i], c + i + NB);
            }
        }
        // the last one to 2 NB - 1 chunks: chunk c + i is in set i % NB
#pragma unroll
        for (int i = 0; i < 2 * NB - 1; ++i) {
            if (c + i < n_chunks) {
                store_x(xs[i % NB], c + i);
                __syncthreads();
                if (i < NB - 1 && c + i + NB < n_chunks) load_x(xs[i % NB], c + i + NB);
                compute(wbuf[i % NB], c + i);
                if (i < NB - 1 && c + i + NB < n_chunks) load_w(wbuf[i % NB], c + i + NB);
            }
        }
        __syncthreads();                                        // the sums below reuse the buffer
    } else if (group_ok) {
        // S steps are in flight at any time: all of a chunk's loads are asked for before its first
        // product, and as soon as a step's product has used its registers they are asked for
        // again, for the same step of the next chunk.  (A plain loop of load, wait, product - what
        // the compiler makes of `for k` here, its trip count being a vector register's - costs one
        // trip to memory per step, 0.43 us each.)  What is left after the whole chunks goes in
        // chunks of S/2, S/4, .. 1 steps, each with its loads up front.
        constexpr int S = NTW + MT <= 2 ? 8 : ((MT == 1 && NTW == 2) ? 4 : (NTW * MT >= 12 ? 1 : 2));   // by registers
        const size_t xstep = a.x_tiled ? a.tile_rows : 1;      // a step of 32 columns is 4 chunks of tile_rows rows x 8
        const int kb = __builtin_amdgcn_readfirstlane(kbeg), ke = __builtin_amdgcn_readfirstlane(kend);
        const int steps = (ke - kb) / 32, full = steps / S;
        GFrag8 w[S][NTW], x[S][MT];
        auto ask = [&](int st, int k) {
#pragma unroll
            for (int t = 0; t < NTW; ++t) w[st][t].u4 = load_streamed_u4(wp[t] + (size_t)k * 16);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) x[st][mt].u4 = *reinterpret_cast<const uint4 *>(xr[mt] + (size_t)k * xstep);
        };
        auto multiply = [&](int st) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int t = 0; t < NTW; ++t)
                    acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[st][t].v, x[st][mt].v, acc[t][mt], 0, 0, 0);
        };
        int k = kb;
        if (full > 0) {
#pragma unroll
            for (int st = 0; st < S; ++st) ask(st, k + 32 * st);
            for (int c = 1; c < full; ++c) {
                k += 32 * S;
#pragma unroll
                for (int st = 0; st < S; ++st) {
                    multiply(st);
                    ask(st, k + 32 * st);
                    __builtin_amdgcn_sched_barrier(0);        // in this order: S - 1 steps stay in flight
                }
            }
#pragma unroll
            for (int st = 0; st < S; ++st) multiply(st);
            k += 32 * S;
        }
        const int left = steps - full * S;
#pragma unroll
        for (int part = S / 2; part >= 1; part /= 2) {
            if (left & part) {
#pragma unroll
                for (int st = 0; st < (S > 1 ? S / 2 : 1); ++st)
                    if (st < part) ask(st, k + 32 * st);
#pragma unroll
                for (int st = 0; st < (S > 1 ? S / 2 : 1); ++st)
                    if (st < part) multiply(st);
                k += 32 * part;
            }
        }
    }

    if (kPreRope && kpart == 0 && group_ok && rope_rotated && a.cos_t != nullptr) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            if (mt * 16 + r >= a.M) continue;
            const size_t at = (size_t)pre_pos[mt] * (a.head_dim / 2) + rope_j * 16 + orow;
            pre_cos[mt] = *reinterpret_cast<const float4 *>(a.cos_t + at);
            pre_sin[mt] = *reinterpret_cast<const float4 *>(a.sin_t + at);
        }
    }
    if (DV > 0) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            float s = ssum[mt];
#pragma unroll
            for (int j = 0; j < DV; ++j)
                s += (4 * j < dv_end[mt]) ? (dv[mt][j].x + dv[mt][j].y) + (dv[mt][j].z + dv[mt][j].w) : 0.f;
            ssum[mt] = s;
        }
    }

    if (k_waves > 1) {
        // partial sums of the K slices, added by the first wave of each tile group in slice
        // order; one token tile at a time, so the buffer does not grow with M
        float *mine = red + (size_t)wave * (NTW * 64 * 4);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            if (mt > 0) __syncthreads();
            if (kpart != 0) {
#pragma unroll
                for (int t = 0; t < NTW; ++t)
                    *reinterpret_cast<float4 *>(mine + (t * 64 + lane) * 4) =
                        make_float4(acc[t][mt][0], acc[t][mt][1], acc[t][mt][2], acc[t][mt][3]);
            }
            __syncthreads();
            if (kpart == 0) {
                // three slices are read at a time and then added in slice order (one read per
                // turn leaves this wave waiting for LDS fifteen times in a row)
                constexpr int RB = NTW * MT <= 2 ? 3 : 1;       // (where registers allow)
                int p = 1;
                for (; RB > 1 && p + RB - 1 < k_waves; p += RB) {
                    float4 v[RB][NTW];
#pragma unroll
                    for (int j = 0; j < RB; ++j)
#pragma unroll
                        for (int t = 0; t < NTW; ++t)
                            v[j][t] = *reinterpret_cast<const float4 *>(red + (size_t)(wave + p + j) * (NTW * 64 * 4) +
                                                                        (t * 64 + lane) * 4);
#pragma unroll
                    for (int j = 0; j < RB; ++j)
#pragma unroll
                        for (int t = 0; t < NTW; ++t) {
                            acc[t][mt][0] += v[j][t].x; acc[t][mt][1] += v[j][t].y;
                            acc[t][mt][2] += v[j][t].z; acc[t][mt][3] += v[j][t].w;
                        }
                }
                for (; p < k_waves; ++p) {
                    const float *other = red + (size_t)(wave + p) * (NTW * 64 * 4);
#pragma unroll
                    for (int t = 0; t < NTW; ++t) {
                        const float4 v = *reinterpret_cast<const float4 *>(other + (t * 64 + lane) * 4);
                        acc[t][mt][0] += v.x; acc[t][mt][1] += v.y; acc[t][mt][2] += v.z; acc[t][mt][3] += v.w;
                    }
                }
            }
        }
    }
    if (kpart != 0 || !group_ok) return;

    // ---- per-token scale that finishes the input's RMSNorm (the sums were loaded before the loop)
    float rinv[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        rinv[mt] = 1.f;
        if (a.sumsq != nullptr) {
            float s = ssum[mt];
            s = quad_rows_sum(s);
            rinv[mt] = 1.f / sqrtf(s / (float)a.norm_width + a.eps);
        }
    }

    if (EPI == EPI_ROPE) {
        const int D = a.head_dim;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = mt * 16 + r;
            if (m >= a.M || !lane_on) continue;
            float va[4], vb[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                va[i] = bf16_bits_to_float(float_to_bf16_bits(acc[0][mt][i] * rinv[mt]));
                vb[i] = bf16_bits_to_float(float_to_bf16_bits(acc[NTW - 1][mt][i] * rinv[mt]));
            }
            int slot = -1;
            if (kPreRope) slot = pre_slot[mt];
            else if (a.slots != nullptr && rope_head >= a.nq) slot = a.slots[m];
            const int page = slot >= 0 ? slot / a.page_size : 0;
            const int off = slot >= 0 ? slot - page * a.page_size : 0;
            if (rope_rotated) {
                const int f = rope_j * 16 + orow;              // feature in [0, d/2); partner f + d/2
                float o1[4], o2[4];
                if (a.cos_t != nullptr) {
                    float4 c4 = pre_cos[mt], s4 = pre_sin[mt];
                    if (!kPreRope) {
                        const int pos = a.positions[m];
                        c4 = *reinterpret_cast<const float4 *>(a.cos_t + (size_t)pos * (D / 2) + f);
                        s4 = *reinterpret_cast<const float4 *>(a.sin_t + (size_t)pos * (D / 2) + f);
                    }
                    const float c[4] = {c4.x, c4.y, c4.z, c4.w}, s[4] = {s4.x, s4.y, s4.z, s4.w};
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        o1[i] = va[i] * c[i] - vb[i] * s[i];
                        o2[i] = va[i] * s[i] + vb[i] * c[i];
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < 4; ++i) { o1[i] = va[i]; o2[i] = vb[i]; }
                }
                bf16_t *dst, *dst2;
                if (rope_head < a.nq) {
                    dst = reinterpret_cast<bf16_t *>(a.Y) + (size_t)m * a.ldy + (size_t)rope_head * D + f;
                    dst2 = dst + D / 2;
                } else {
                    if (slot < 0) continue;
                    // (f is a multiple of 4 and D of 32: four neighbouring features lie inside one chunk of 8)
                    bf16_t *pg = a.k_cache + ((size_t)page * a.nkv + (rope_head - a.nq)) * a.page_size * D;
                    dst = pg + kva_k_at(off, f, a.page_size, 8);
                    dst2 = pg + kva_k_at(off, f + D / 2, a.page_size, 8);
                }
                *reinterpret_cast<uint2 *>(dst) =
                    make_uint2((uint32_t)float_to_bf16_bits(o1[0]) | ((uint32_t)float_to_bf16_bits(o1[1]) << 16),
                               (uint32_t)float_to_bf16_bits(o1[2]) | ((uint32_t)float_to_bf16_bits(o1[3]) << 16));
                *reinterpret_cast<uint2 *>(dst2) =
                    make_uint2((uint32_t)float_to_bf16_bits(o2[0]) | ((uint32_t)float_to_bf16_bits(o2[1]) << 16),
                               (uint32_t)float_to_bf16_bits(o2[2]) | ((uint32_t)float_to_bf16_bits(o2[3]) << 16));
            } else {
                if (slot < 0) continue;
                const int f = rope_j * 32 + orow;              // value features f..f+3 and f+16..f+19
                bf16_t *dst = a.v_cache + (((size_t)page * a.nkv + (rope_head - a.nq - a.nkv)) * D + f) * a.page_size + off;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    dst[(size_t)i * a.page_size].bits = float_to_bf16_bits(va[i]);
                    dst[(size_t)(16 + i) * a.page_size].bits = float_to_bf16_bits(vb[i]);
                }
            }
        }
        return;
    }

#pragma unroll
    for (int t = 0; t < out_tiles; ++t) {
        const int tile = tile0 + t;
        if (tile >= n_tiles) break;
        const int n = tile * 16 + orow;                    // first of this lane's 4 outputs
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = mt * 16 + r;
            const bool m_ok = m < a.M;
            float v[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (EPI == EPI_SWIGLU) {
                    const float gt = acc[0][mt][i] * rinv[mt];
                    v[i] = gt * (1.f / (1.f + expf(-gt))) * (acc[1][mt][i] * rinv[mt]);
                } else {
                    v[i] = acc[t][mt][i] * rinv[mt];
                }
            }
            if (EPI == EPI_RESID) {
                float ss = 0.f;
                if (m_ok && lane_on) {
                    bf16_t *hp = a.hidden + (size_t)m * a.N + n;
                    bf16_t *sp = a.scaled_out + (size_t)m * a.N + n;
                    if (n + 3 < rows && (a.N % 4 == 0)) {
                        const uint2 hv = kPreResid ? pre_hidden[mt] : *reinterpret_cast<const uint2 *>(hp);
                        const float h0[4] = {bf16_bits_to_float((uint16_t)(hv.x & 0xffffu)),
                                             bf16_bits_to_float((uint16_t)(hv.x >> 16)),
                                             bf16_bits_to_float((uint16_t)(hv.y & 0xffffu)),
                                             bf16_bits_to_float((uint16_t)(hv.y >> 16))};
                        float wn[4] = {pre_wn_f.x, pre_wn_f.y, pre_wn_f.z, pre_wn_f.w};
                        if (a.next_w == nullptr) {
                            wn[0] = wn[1] = wn[2] = wn[3] = 1.f;
                        } else if (kPreResid && !a.next_w_f32) {
                            wn[0] = bf16_bits_to_float((uint16_t)(pre_wn_b.x & 0xffffu));
                            wn[1] = bf16_bits_to_float((uint16_t)(pre_wn_b.x >> 16));
                            wn[2] = bf16_bits_to_float((uint16_t)(pre_wn_b.y & 0xffffu));
                            wn[3] = bf16_bits_to_float((uint16_t)(pre_wn_b.y >> 16));
                        }
                        if (!kPreResid && a.next_w != nullptr) {
                            if (a.next_w_f32) {
                                const float4 wv = *reinterpret_cast<const float4 *>(
                                    reinterpret_cast<const float *>(a.next_w) + n);
                                wn[0] = wv.x; wn[1] = wv.y; wn[2] = wv.z; wn[3] = wv.w;
                            } else {
                                const uint2 wv = *reinterpret_cast<const uint2 *>(
                                    reinterpret_cast<const bf16_t *>(a.next_w) + n);
                                wn[0] = bf16_bits_to_float((uint16_t)(wv.x & 0xffffu));
                                wn[1] = bf16_bits_to_float((uint16_t)(wv.x >> 16));
                                wn[2] = bf16_bits_to_float((uint16_t)(wv.y & 0xffffu));
                                wn[3] = bf16_bits_to_float((uint16_t)(wv.y >> 16));
                            }
                        }
                        uint16_t sb[4], xb[4];
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            sb[i] = float_to_bf16_bits(h0[i] + v[i]);
                            const float sv = bf16_bits_to_float(sb[i]);
                            ss += sv * sv;
                            xb[i] = float_to_bf16_bits(sv * wn[i]);
                        }
                        *reinterpret_cast<uint2 *>(hp) =
                            make_uint2((uint32_t)sb[0] | ((uint32_t)sb[1] << 16), (uint32_t)sb[2] | ((uint32_t)sb[3] << 16));
                        *reinterpret_cast<uint2 *>(sp) =
                            make_uint2((uint32_t)xb[0] | ((uint32_t)xb[1] << 16), (uint32_t)xb[2] | ((uint32_t)xb[3] << 16));
                    } else {
                        for (int i = 0; i < 4; ++i) {
                            if (n + i >= rows) break;
                            const uint16_t sb = float_to_bf16_bits(to_float(hp[i]) + v[i]);
                            hp[i].bits = sb;
                            const float sv = bf16_bits_to_float(sb);
                            ss += sv * sv;
                            float wn = 1.f;
                            if (a.next_w != nullptr)
                                wn = a.next_w_f32 ? reinterpret_cast<const float *>(a.next_w)[n + i]
                                                  : to_float(reinterpret_cast<const bf16_t *>(a.next_w)[n + i]);
                            sp[i].bits = float_to_bf16_bits(sv * wn);
                        }
                    }
                }
                ss = quad_rows_sum(ss);
                if (m_ok && g == 0) {
                    if (a.half) a.sumsq_out[(size_t)m * (2 * n_tiles) + 2 * tile + (hrow >> 3)] = ss;
                    else a.sumsq_out[(size_t)m * n_tiles + tile] = ss;
                }
                continue;
            }
            if (!m_ok || !lane_on) continue;
            if (a.out_f32) {
                float *dst = reinterpret_cast<float *>(a.Y) + ((size_t)blockIdx.y * a.M + m) * a.ldy + n;
                if (n + 3 < rows && (a.ldy % 4 == 0)) {
                    *reinterpret_cast<float4 *>(dst) = make_float4(v[0], v[1], v[2], v[3]);
                } else {
                    for (int i = 0; i < 4; ++i)
                        if (n + i < rows) dst[i] = v[i];
                }
            } else {
                bf16_t *dst = reinterpret_cast<bf16_t *>(a.Y) + (size_t)m * a.ldy + n;
                if (a.y_tiled) dst = reinterpret_cast<bf16_t *>(a.Y) + ((size_t)(n >> 3) * a.tile_rows + m) * 8 + (n & 7);
                if (n + 3 < rows && (a.y_tiled || a.ldy % 4 == 0)) {
                    uint2 w;
                    w.x = (uint32_t)float_to_bf16_bits(v[0]) | ((uint32_t)float_to_bf16_bits(v[1]) << 16);
                    w.y = (uint32_t)float_to_bf16_bits(v[2]) | ((uint32_t)float_to_bf16_bits(v[3]) << 16);
                    *reinterpret_cast<uint2 *>(dst) = w;
                } else {
                    for (int i = 0; i < 4; ++i)
                        if (n + i < rows) dst[i].bits = float_to_bf16_bits(v[i]);
                }
            }
        }
    }
}

// k_waves: how many wavefronts share one tile group's K range.  Depends on N and K only, never
// on M, so a token's result does not depend on the batch it is in (the launcher cuts it to 4 where
// the waves share X through LDS, above 16 rows: that changes the order of the sum, not more).  These products are bound by
// memory latency until the waves together keep tens of megabytes in flight, so K is cut as deep
// as a workgroup allows (16 waves) while a wave keeps at least 4 steps of 32, the chip is not
// oversubscribed (4096 waves) and the waves do not already cover the bandwidth-delay product.
static int choose_k_waves(int groups, int K, int ntw) {
    int kw = 1;
    while (kw < 16) {
        const int next = kw * 2;
        if (K % (32 * next) != 0 || K / next < 128) break;
        if ((long)groups * next > 4096) break;
        const long in_flight = (long)groups * kw * ntw * 8192;     // 8 steps of 1 KiB per tile and wave
        if (in_flight >= (48L << 20)) break;
        kw = next;
    }
    return kw;
}

// Every compute unit has its share of the chip's bandwidth to give (24 GB/s each), so a matrix with
// at most half as many tile groups as the chip has compute units is spread over twice as many workgroups:
// each takes half (8) of the rows of its tiles.  Depends on the matrix only, never on M.
static int compute_units() {
    static int cus = 0;
    if (cus == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            n = 256;
        cus = n;
    }
    return cus;
}
static int choose_half_tiles(int groups) { return groups * 2 <= compute_units() ? 1 : 0; }

extern "C" int kva_gemm_skinny_supported(int M, int N, int K) {
    return (M >= 1 && M <= 64 && N >= 1 && K >= 32 && K % 32 == 0) ? 1 : 0;
}

// Number of partial sums of squares per token that an EPI_RESID product with N columns writes.
extern "C" int kva_gemm_skinny_sumsq_parts(int N) {
    const int n_tiles = (N + 15) / 16;
    return choose_half_tiles(n_tiles) ? 2 * n_tiles : n_tiles;
}

// Rows of the [columns / 8][rows][8] layout that holds M rows (TiledRows of the Python side).  8
// rows for up to 8: with 16 the down projection of 8 requests read as many bytes of padding as
// of activations, in every workgroup (decode steps of 8 requests at 8,192 / 768 keys 1.194 / 0.877
// -> 1.173 / 0.858 ms, of 4 at 768 keys 0.856 -> 0.836).
extern "C" int kva_tiled_rows(int M) { return M <= 8 ? 8 : (M + 15) / 16 * 16; }

template <int NTW, int EPI>
static void launch_xl(const SkinnyArgs &a, dim3 grid, dim3 block, size_t lds, hipStream_t stream) {
    switch ((a.M + 15) / 16) {
    case 2: hipLaunchKernelGGL((gemm_skinny_kernel<2, NTW, EPI, true>), grid, block, lds, stream, a); break;
    case 3: hipLaunchKernelGGL((gemm_skinny_kernel<3, NTW, EPI, true>), grid, block, lds, stream, a); break;
    default: hipLaunchKernelGGL((gemm_skinny_kernel<4, NTW, EPI, true>), grid, block, lds, stream, a); break;
    }
}

template <int NTW, int EPI>
static void launch_mt(const SkinnyArgs &a, dim3 grid, dim3 block, size_t lds, hipStream_t stream) {
    switch ((a.M + 15) / 16) {
    case 1: hipLaunchKernelGGL((gemm_skinny_kernel<1, NTW, EPI>), grid, block, lds, stream, a); break;
    case 2: hipLaunchKernelGGL((gemm_skinny_kernel<2, NTW, EPI>), grid, block, lds, stream, a); break;
    case 3: hipLaunchKernelGGL((gemm_skinny_kernel<3, NTW, EPI>), grid, block, lds, stream, a); break;
    default: hipLaunchKernelGGL((gemm_skinny_kernel<4, NTW, EPI>), grid, block, lds, stream, a); break;
    }
}

// W: the tiled copy of the [N, K] weight (rows padded to a multiple of 16 with zeros; for mode 2
// the gate half and the up half are tiled separately, gate tiles first).
// mode 0: Y bf16 [M, N]; mode 1: Y fp32 [M, N]; mode 2: W is [2*inter, K] = [gate; up], Y bf16
// [M, inter] = silu(X gate^T) * (X up^T); mode 3: hidden[M, N] += X W^T in place, plus
// scaled_out[M, N] = round(hidden * next_w) and sumsq_out[M, ceil(N/16)].
// sumsq (optional, any mode): partial sums of squares of the un-normalised input rows.
extern "C" int kva_gemm_skinny(void *Y, const void *X, const void *W, int M, int N, int K, int ldx,
                               int ldy, int mode, const float *sumsq, int sumsq_parts, int norm_width,
                               float eps, void *hidden, const void *next_w, int next_w_f32,
                               void *scaled_out, float *sumsq_out, int x_tiled, int y_tiled,
                               hipStream_t stream) {
    KVA_REQUIRE(kva_gemm_skinny_supported(M, N, K), "gemm_skinny: M=%d N=%d K=%d not supported "
                "(1 <= M <= 64, K a multiple of 32)", M, N, K);
    KVA_REQUIRE(mode >= 0 && mode <= 3, "gemm_skinny: unknown mode %d", mode);
    KVA_REQUIRE(ldx >= K && ldx % 8 == 0, "gemm_skinny: X row stride %d must be a multiple of 8 and >= K", ldx);
    KVA_REQUIRE(mode != 2 || N % 2 == 0, "gemm_skinny: a joined [gate; up] matrix needs an even row count");
    KVA_REQUIRE(sumsq == nullptr || (sumsq_parts >= 1 && norm_width >= 1),
                "gemm_skinny: row scaling needs a part count and the norm's width");
    KVA_REQUIRE(mode != 3 || (hidden && scaled_out && sumsq_out),
                "gemm_skinny: the residual epilogue needs hidden, scaled_out and sumsq_out");
    SkinnyArgs a = {};
    a.X = (const bf16_t *)X; a.W = (const bf16_t *)W; a.Y = Y;
    a.M = M; a.N = N; a.K = K; a.ldx = ldx; a.ldy = ldy; a.k_slices = 1;
    a.inter = mode == 2 ? N / 2 : 0;
    a.out_f32 = mode == 1 ? 1 : 0;
    a.sumsq = sumsq; a.sumsq_parts = sumsq_parts; a.norm_width = norm_width; a.eps = eps;
    a.hidden = (bf16_t *)hidden; a.next_w = next_w; a.next_w_f32 = next_w_f32;
    a.scaled_out = (bf16_t *)scaled_out; a.sumsq_out = sumsq_out;
    // (tiled X or Y: [columns / 8][rows rounded up to 16][8])
    KVA_REQUIRE(!y_tiled || (mode == 2 && (N / 2) % 8 == 0), "gemm_skinny: a tiled result is for the gated product with a multiple of 8 columns");
    KVA_REQUIRE(!x_tiled || K % 8 == 0, "gemm_skinny: tiled X");
    a.x_tiled = x_tiled ? 1 : 0; a.y_tiled = y_tiled ? 1 : 0;
    a.tile_rows = kva_tiled_rows(M);
    const int rows = mode == 2 ? a.inter : N;
    KVA_REQUIRE(mode == 3 || ldy >= rows, "gemm_skinny: Y row stride %d is smaller than its %d columns", ldy, rows);
    const int n_tiles = (rows + 15) / 16;
    // tiles per wave: wide matrices reuse each loaded X fragment for several n-tiles
    int ntw = 1;
    if (mode == 2) ntw = 2;
    else if (mode == 3) ntw = 1;
    else if (n_tiles >= 4096) ntw = 4;
    else if (n_tiles >= 2048) ntw = 2;
    const int out_tiles = mode == 2 ? 1 : ntw;
    int groups = (n_tiles + out_tiles - 1) / out_tiles;
    a.half = mode == 3 ? choose_half_tiles(groups) : 0;
    if (a.half) groups *= 2;
    int kw = choose_k_waves(groups, K, ntw);
    int groups_per_wg = kw >= 4 ? 1 : 4 / kw;
    // The gated product has two tile groups or more per compute unit.  Two of them in a workgroup,
    // K over two wavefronts each, leave a unit one workgroup's reads of X where two workgroups of
    // K over 8 wavefronts made two: decode steps of 12 / 16 requests at the 1B sizes 0.920 /
    // 0.978 -> 0.908 / 0.954 ms (the product alone at 16 rows 13.8 -> 12.75 us), at 8 requests
    // the same, at 3 / 4 requests 0.831 / 0.836 -> 0.837 / 0.844; 16 requests at the 3B / 8B sizes
    // 1-6 % faster.  For every row count up to 16 alike, so that a token's result does not
    // depend on how many share its step.
    if (mode == 2 && M <= 16 && kw > 2 && groups % 2 == 0 && groups >= 2 * compute_units()) { kw = 2; groups_per_wg = 2; }
    // The products into the residual stream: K over at most 8 wavefronts (16 left each of them 4
    // steps of the output projection; 1B sizes, 8 / 16 rows: output 5.40 / 6.24 -> 5.14 / 5.85 us,
    // down 10.6 / 13.7 -> 10.3 / 13.2; decode steps of 4-16 requests 1 % faster, 8B sizes the same).
    if (mode == 3 && M <= 16 && kw > 8) kw = 8;
    // Vocabulary-sized matrices (four tiles a wavefront, all of K each): eight wavefronts a workgroup
    // rather than four, 251 workgroups (LM head of the 1B sizes at 8 / 16 rows 89.4 / 90.5 -> 84.1 / 85.4 us).
    if (ntw == 4 && M <= 16 && kw == 1) groups_per_wg = 8;
    // More than 16 tokens and several tiles per wave: workgroups of several tile groups that
    // share X through LDS (at most 4 K ranges of 2 x 64 tokens x 128 bytes: 64 KiB).
    const bool xl = M > 16 && ntw >= 2 && groups >= 2 && !x_tiled;      // tiled rows are read in whole cache lines as they are
    if (xl) {
        kw = kw < 4 ? kw : 4;
        groups_per_wg = kw == 4 ? 2 : 4;
        // A workgroup re-reads all of X for its tile groups: with two groups of a joined [gate; up]
        // matrix that is as many bytes as its share of W.  Where four groups per workgroup still leave
        // nearly a workgroup per compute unit, K goes over two ranges of waves instead of four and a
        // workgroup takes four groups (8B sizes, 896 groups: decode steps of 48 / 64 requests
        // 5.05 / 5.48 -> 4.96 / 5.30 ms; with 512 groups, 128 workgroups, 5 % slower).
        if (kw == 4 && groups / 4 >= compute_units() * 7 / 8) { kw = 2; groups_per_wg = 4; }
        if (kw == 1) groups_per_wg = 8;                          // (LM head at 32 / 64 rows 85.6 / 91.9 -> 84.1 / 90.3 us)
        // Three or four row tiles: K over two ranges, four wavefronts a workgroup (fewer, longer
        // streams and half the barriers' company; the gated product of the 1B sizes at 48 / 64 rows
        // 17.0 / 19.2 -> 16.2 / 17.7 us, decode steps of 64 requests 1.404 -> 1.382 ms; at 17-32 rows
        // the same either way).
        if (kw == 4 && groups_per_wg == 2 && M > 32) kw = 2;
    }
    // the waves of a K range bring X to LDS together, 64 of a chunk's 128 units per row tile each
    KVA_REQUIRE(!xl || groups_per_wg >= 2, "gemm_skinny: the shared-X form needs two tile groups per workgroup");
    a.k_waves = kw;
    const int waves = kw * groups_per_wg;
    size_t lds = kw > 1 ? (size_t)waves * ntw * 64 * 4 * sizeof(float) : 0;
    if (xl) {
        const size_t stage = (size_t)kw * 2 * ((M + 15) / 16 * 16) * 128;
        lds = lds > stage ? lds : stage;
    }
    KVA_REQUIRE(lds <= 64 * 1024, "gemm_skinny: LDS buffer of %zu bytes does not fit", lds);
    dim3 grid((groups + groups_per_wg - 1) / groups_per_wg), block(64 * waves);
    if (xl) {
        if (mode == 2) launch_xl<2, EPI_SWIGLU>(a, grid, block, lds, stream);
        else if (ntw == 4) launch_xl<4, EPI_PLAIN>(a, grid, block, lds, stream);
        else launch_xl<2, EPI_PLAIN>(a, grid, block, lds, stream);
    }
    else if (mode == 2) launch_mt<2, EPI_SWIGLU>(a, grid, block, lds, stream);
    else if (mode == 3) launch_mt<1, EPI_RESID>(a, grid, block, lds, stream);
    else if (ntw == 4) launch_mt<4, EPI_PLAIN>(a, grid, block, lds, stream);
    else if (ntw == 2) launch_mt<2, EPI_PLAIN>(a, grid, block, lds, stream);
    else launch_mt<1, EPI_PLAIN>(a, grid, block, lds, stream);
    KVA_CHECK_LAUNCH("gemm_skinny");
    return KVA_OK;
}

// The joined Q/K/V projection with rotary encoding and the cache write in its epilogue.
// W: tiled copy of the [(nq + 2 nkv) * d, K] weight; q_out bf16 [M, nq * d] (row stride ldq).
// cos/sin [positions, d / 2] fp32 or both null (no rotation); slots null: nothing is cached.
// head_dim must be a multiple of 32 (a wave takes the tile pair f, f + d/2).
extern "C" int kva_gemm_skinny_qkv_rope_supported(int M, int K, int head_dim) {
    return (M >= 1 && M <= 64 && K >= 32 && K % 32 == 0 && head_dim >= 32 && head_dim % 32 == 0) ? 1 : 0;
}

extern "C" int kva_gemm_skinny_qkv_rope(void *q_out, int ldq, const void *X, const void *W, int M, int K,
                                        int ldx, int nq, int nkv, int head_dim, const float *sumsq,
                                        int sumsq_parts, int norm_width, float eps, const float *cos_t,
                                        const float *sin_t, const int *positions, const int *slots,
                                        void *k_cache, void *v_cache, int page_size, hipStream_t stream) {
    KVA_REQUIRE(nq >= 1 && nkv >= 1, "gemm_skinny_qkv_rope: bad head counts %d, %d", nq, nkv);
    KVA_REQUIRE(kva_gemm_skinny_qkv_rope_supported(M, K, head_dim),
                "gemm_skinny_qkv_rope: M=%d K=%d head_dim=%d not supported (1 <= M <= 64, K and "
                "head_dim multiples of 32)", M, K, head_dim);
    KVA_REQUIRE(ldx >= K && ldx % 8 == 0, "gemm_skinny_qkv_rope: X row stride %d must be a multiple of 8 and >= K", ldx);
    KVA_REQUIRE(ldq >= nq * head_dim && ldq % 4 == 0, "gemm_skinny_qkv_rope: Q row stride %d does not fit", ldq);
    KVA_REQUIRE((cos_t == nullptr) == (sin_t == nullptr), "gemm_skinny_qkv_rope: one table missing");
    KVA_REQUIRE(cos_t == nullptr || positions != nullptr, "gemm_skinny_qkv_rope: rotation needs positions");
    KVA_REQUIRE(slots == nullptr || (k_cache && v_cache && page_size > 0),
                "gemm_skinny_qkv_rope: cache write asked for without cache or page size");
    KVA_REQUIRE(sumsq == nullptr || (sumsq_parts >= 1 && norm_width >= 1),
                "gemm_skinny_qkv_rope: row scaling needs a part count and the norm's width");
    SkinnyArgs a = {};
    a.X = (const bf16_t *)X; a.W = (const bf16_t *)W; a.Y = q_out;
    a.M = M; a.N = (nq + 2 * nkv) * head_dim; a.K = K; a.ldx = ldx; a.ldy = ldq; a.k_slices = 1;
    a.sumsq = sumsq; a.sumsq_parts = sumsq_parts; a.norm_width = norm_width; a.eps = eps;
    a.cos_t = cos_t; a.sin_t = sin_t; a.positions = positions; a.slots = slots;
    a.k_cache = (bf16_t *)k_cache; a.v_cache = (bf16_t *)v_cache;
    a.nq = nq; a.nkv = nkv; a.head_dim = head_dim; a.page_size = page_size;
    int groups = a.N / 32;
    // More than 16 tokens: workgroups of several tile groups share X through LDS, as in
    // kva_gemm_skinny (17 / 32 / 48 / 64 tokens of the 1B shape: 12.3 / 12.8 / 16.2 / 20.1 us -> 11.5 /
    // 11.8 / 14.2 / 16.3 us), without half tiles.
    const bool xl = M > 16 && groups >= 2;
    a.half = xl ? 0 : choose_half_tiles(groups);
    if (a.half) groups *= 2;
    int kw = choose_k_waves(groups, K, 2);
    if (!xl && kw > 8) kw = 8;                                  // as for the products into the residual stream
    int groups_per_wg = kw >= 4 ? 1 : 4 / kw;
    if (xl) {
        kw = kw < 4 ? kw : 4;
        groups_per_wg = kw == 4 ? 2 : 4;
    }
    KVA_REQUIRE(!xl || groups_per_wg >= 2, "gemm_skinny_qkv_rope: the shared-X form needs two tile groups per workgroup");
    a.k_waves = kw;
    const int waves = kw * groups_per_wg;
    size_t lds = kw > 1 ? (size_t)waves * 2 * 64 * 4 * sizeof(float) : 0;
    if (xl) {
        const size_t stage = (size_t)kw * 2 * ((M + 15) / 16 * 16) * 128;
        lds = lds > stage ? lds : stage;
    }
    KVA_REQUIRE(lds <= 64 * 1024, "gemm_skinny_qkv_rope: LDS buffer of %zu bytes does not fit", lds);
    dim3 grid((groups + groups_per_wg - 1) / groups_per_wg), block(64 * waves);
    if (xl) launch_xl<2, EPI_ROPE>(a, grid, block, lds, stream);
    else launch_mt<2, EPI_ROPE>(a, grid, block, lds, stream);
    KVA_CHECK_LAUNCH("gemm_skinny_qkv_rope");
    return KVA_OK;
}

// How many K ranges kva_gemm_skinny_partials cuts a product into (0: it does not take the shape).
// Two tiles of W per wavefront, two wavefronts per K range and two K ranges per workgroup share
// their rows of X through LDS; the ranges across workgroups are as many as fill the compute units
// while a range keeps at least 256 columns.
extern "C" int kva_gemm_skinny_partial_slices(int M, int N, int K) {
    if (M <= 16 || M > 64 || N < 32 || K % 128 != 0) return 0;
    const int n_tiles = (N + 15) / 16;
    const int groups = (n_tiles + 1) / 2;
    const int wgs = (groups + 1) / 2;
    int slices = 1;
    while (wgs * slices * 2 <= compute_units() && K % (slices * 2 * 128) == 0 && K / (slices * 2) >= 256) slices *= 2;
    return slices;
}

// P[s][M][N] (fp32) = X[:, range s of K] W[:, range s]^T for s in [0, slices): partial products for a
// kernel that adds them up and does what follows the product (residual and norm).  W: the tiled copy.
extern "C" int kva_gemm_skinny_partials(float *P, const void *X, const void *W, int M, int N, int K, int ldx,
                                        int slices, hipStream_t stream) {
    KVA_REQUIRE(slices >= 1 && slices == kva_gemm_skinny_partial_slices(M, N, K),
                "gemm_skinny_partials: M=%d N=%d K=%d is not taken in %d ranges", M, N, K, slices);
    KVA_REQUIRE(ldx >= K && ldx % 8 == 0, "gemm_skinny_partials: X row stride %d must be a multiple of 8 and >= K", ldx);
    SkinnyArgs a = {};
    a.X = (const bf16_t *)X; a.W = (const bf16_t *)W; a.Y = P;
    a.M = M; a.N = N; a.K = K; a.ldx = ldx; a.ldy = N; a.k_slices = slices;
    a.out_f32 = 1;
    const int n_tiles = (N + 15) / 16;
    const int groups = (n_tiles + 1) / 2;
    a.k_waves = 2;
    const int groups_per_wg = 2, waves = 4;
    const size_t stage = (size_t)a.k_waves * 2 * ((M + 15) / 16 * 16) * 128;
    const size_t sums = (size_t)waves * 2 * 64 * 4 * sizeof(float);
    const size_t lds = stage > sums ? stage : sums;
    dim3 grid((groups + groups_per_wg - 1) / groups_per_wg, slices), block(64 * waves);
    launch_xl<2, EPI_PLAIN>(a, grid, block, lds, stream);
    KVA_CHECK_LAUNCH("gemm_skinny_partials");
    return KVA_OK;
}
