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
// Both operands are read from memory directly in operand layout (16 bytes per lane).  A wave
// keeps one accumulator per 16-token tile (MT = ceil(M / 16) <= 4), so W is read once whatever M
// is.  K is split over `k_waves` wavefronts of a workgroup (partials summed through LDS in a
// fixed order) so that narrow matrices still put >= 2048 waves on the 256 compute units.
//
// A column of the result depends only on its own token's row of X: results do not change with
// the batch.  Epilogues: bf16 or fp32 output; or, for a joined [gate; up] matrix, the SwiGLU
// activation silu(gate) * up (reference siluKernel, base/src/kernels.cu:45-52) so the 2*I-wide
// intermediate never goes to memory.
#include "common.h"
#include <math.h>

typedef __bf16 gb16x8 __attribute__((ext_vector_type(8)));
typedef float gf32x4 __attribute__((ext_vector_type(4)));

union GFrag8 {
    gb16x8 v;
    uint4 u4;
};

template <int MT, bool SWIGLU>
__global__ void gemm_skinny_kernel(const bf16_t *__restrict__ X, const bf16_t *__restrict__ W,
                                   void *__restrict__ Y, int M, int N, int K, int ldx, int ldy,
                                   int k_waves, int out_f32, int inter) {
    extern __shared__ float red[];
    constexpr int NACC = SWIGLU ? 2 : 1;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int waves = blockDim.x >> 6;
    const int tiles_per_wg = waves / k_waves;
    const int tile = blockIdx.x * tiles_per_wg + wave / k_waves;
    const int kpart = wave % k_waves;
    const int r = lane & 15, g = lane >> 4;
    const int rows = SWIGLU ? inter : N;                 // rows of one operand block of W
    const int n_tiles = (rows + 15) / 16;
    const bool tile_ok = tile < n_tiles;
    const int kper = K / k_waves;
    const int kbeg = kpart * kper, kend = kbeg + kper;

    int row = tile * 16 + r;
    if (row > rows - 1) row = rows - 1;
    if (row < 0) row = 0;
    const bf16_t *wa = W + (size_t)row * K + 8 * g;
    const bf16_t *wb = SWIGLU ? W + (size_t)(inter + row) * K + 8 * g : nullptr;
    const bf16_t *xr[MT];
    bool xv[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = mt * 16 + r;
        xv[mt] = m < M;
        xr[mt] = X + (size_t)(xv[mt] ? m : 0) * ldx + 8 * g;
    }

    gf32x4 acc[NACC][MT];
#pragma unroll
    for (int a = 0; a < NACC; ++a)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[a][mt] = gf32x4{0.f, 0.f, 0.f, 0.f};

    if (tile_ok) {
#pragma unroll 4
        for (int k = kbeg; k < kend; k += 32) {
            GFrag8 a0, a1;
            a0.u4 = *reinterpret_cast<const uint4 *>(wa + k);
            if (SWIGLU) a1.u4 = *reinterpret_cast<const uint4 *>(wb + k);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                GFrag8 x;
                x.u4 = xv[mt] ? *reinterpret_cast<const uint4 *>(xr[mt] + k) : make_uint4(0, 0, 0, 0);
                acc[0][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0.v, x.v, acc[0][mt], 0, 0, 0);
                if (SWIGLU)
                    acc[1][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1.v, x.v, acc[1][mt], 0, 0, 0);
            }
        }
    }

    if (k_waves > 1) {
        // partial sums of the K slices, added by the first wave of each tile in slice order
        float *mine = red + (size_t)wave * (NACC * MT * 64 * 4);
        if (kpart != 0) {
#pragma unroll
            for (int a = 0; a < NACC; ++a)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    *reinterpret_cast<float4 *>(mine + ((a * MT + mt) * 64 + lane) * 4) =
                        make_float4(acc[a][mt][0], acc[a][mt][1], acc[a][mt][2], acc[a][mt][3]);
        }
        __syncthreads();
        if (kpart == 0) {
            for (int p = 1; p < k_waves; ++p) {
                const float *other = red + (size_t)(wave + p) * (NACC * MT * 64 * 4);
#pragma unroll
                for (int a = 0; a < NACC; ++a)
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt) {
                        const float4 v = *reinterpret_cast<const float4 *>(other + ((a * MT + mt) * 64 + lane) * 4);
                        acc[a][mt][0] += v.x; acc[a][mt][1] += v.y; acc[a][mt][2] += v.z; acc[a][mt][3] += v.w;
                    }
            }
        }
    }
    if (kpart != 0 || !tile_ok) return;

    const int n = tile * 16 + 4 * g;                       // first of this lane's 4 outputs
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = mt * 16 + r;
        if (m >= M) continue;
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if (SWIGLU) {
                const float gt = acc[0][mt][i];
                v[i] = gt * (1.f / (1.f + expf(-gt))) * acc[1][mt][i];
            } else {
                v[i] = acc[0][mt][i];
            }
        }
        if (out_f32) {
            float *dst = reinterpret_cast<float *>(Y) + (size_t)m * ldy + n;
            if (n + 3 < rows && (ldy % 4 == 0)) {
                *reinterpret_cast<float4 *>(dst) = make_float4(v[0], v[1], v[2], v[3]);
            } else {
                for (int i = 0; i < 4; ++i)
                    if (n + i < rows) dst[i] = v[i];
            }
        } else {
            bf16_t *dst = reinterpret_cast<bf16_t *>(Y) + (size_t)m * ldy + n;
            if (n + 3 < rows && (ldy % 4 == 0)) {
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

// k_waves: how many wavefronts share one n-tile's K range.  Depends on N and K only, never on M,
// so a token's result does not depend on the batch it is in.
static int choose_k_waves(int n_tiles, int K) {
    int kw = 1;
    while (kw < 16 && n_tiles * kw < 2048 && K % (32 * kw * 2) == 0 && K / (kw * 2) >= 128) kw *= 2;
    return kw;
}

extern "C" int kva_gemm_skinny_supported(int M, int N, int K) {
    return (M >= 1 && M <= 64 && N >= 1 && K >= 32 && K % 32 == 0) ? 1 : 0;
}

// mode 0: Y bf16 [M, N]; mode 1: Y fp32 [M, N]; mode 2: W is [2*inter, K] = [gate; up], Y bf16
// [M, inter] = silu(X gate^T) * (X up^T)
extern "C" int kva_gemm_skinny(void *Y, const void *X, const void *W, int M, int N, int K, int ldx,
                               int ldy, int mode, hipStream_t stream) {
    KVA_REQUIRE(kva_gemm_skinny_supported(M, N, K), "gemm_skinny: M=%d N=%d K=%d not supported "
                "(1 <= M <= 64, K a multiple of 32)", M, N, K);
    KVA_REQUIRE(mode >= 0 && mode <= 2, "gemm_skinny: unknown mode %d", mode);
    KVA_REQUIRE(ldx >= K && ldx % 8 == 0, "gemm_skinny: X row stride %d must be a multiple of 8 and >= K", ldx);
    KVA_REQUIRE(mode != 2 || N % 2 == 0, "gemm_skinny: a joined [gate; up] matrix needs an even row count");
    const int inter = mode == 2 ? N / 2 : 0;
    const int rows = mode == 2 ? inter : N;
    KVA_REQUIRE(ldy >= rows, "gemm_skinny: Y row stride %d is smaller than its %d columns", ldy, rows);
    const int n_tiles = (rows + 15) / 16;
    const int kw = choose_k_waves(n_tiles, K);
    const int tiles_per_wg = kw >= 4 ? 1 : 4 / kw;
    const int waves = kw * tiles_per_wg;
    const int mt = (M + 15) / 16;
    const int nacc = mode == 2 ? 2 : 1;
    const size_t lds = kw > 1 ? (size_t)waves * nacc * mt * 64 * 4 * sizeof(float) : 0;
    KVA_REQUIRE(lds <= 64 * 1024, "gemm_skinny: reduction buffer of %zu bytes does not fit", lds);
    dim3 grid((n_tiles + tiles_per_wg - 1) / tiles_per_wg), block(64 * waves);
    const int f32 = mode == 1 ? 1 : 0;
#define LAUNCH(MTV, SW)                                                                         \
    hipLaunchKernelGGL((gemm_skinny_kernel<MTV, SW>), grid, block, lds, stream, (const bf16_t *)X, \
                       (const bf16_t *)W, Y, M, N, K, ldx, ldy, kw, f32, inter)
    if (mode == 2) {
        switch (mt) {
        case 1: LAUNCH(1, true); break;
        case 2: LAUNCH(2, true); break;
        case 3: LAUNCH(3, true); break;
        default: LAUNCH(4, true); break;
        }
    } else {
        switch (mt) {
        case 1: LAUNCH(1, false); break;
        case 2: LAUNCH(2, false); break;
        case 3: LAUNCH(3, false); break;
        default: LAUNCH(4, false); break;
        }
    }
#undef LAUNCH
    KVA_CHECK_LAUNCH("gemm_skinny");
    return KVA_OK;
}
