// True fp32 matrix product for the 32-bit path: C[M,N] = A[M,K] * W[N,K]^T, everything
// row-major fp32, plain FMA (no matrix-core reduced-precision mode).
//
// It stands where the reference calls cublasGemmEx with the OP_T/OP_N trick for a row-major
// [out,in] weight (base/src/engine.cu:652-671).  Each output element is one accumulator that
// takes k = 0..K-1 in ascending order, so a row of C does not depend on M, on the tile it falls
// in or on the other rows: the fp32 path is bit-identical under any batching.
#include "common.h"

#define GF_BM 64
#define GF_BN 64
#define GF_BK 16

__global__ void __launch_bounds__(256)
gemm_nt_f32_kernel(float *__restrict__ C, const float *__restrict__ A, const float *__restrict__ W,
                   int M, int N, int K, int lda, int ldw, int ldc) {
    __shared__ float As[GF_BK][GF_BM + 4];
    __shared__ float Ws[GF_BK][GF_BN + 4];
    const int tid = threadIdx.x;
    const int tx = tid % 16, ty = tid / 16;
    const int m0 = blockIdx.y * GF_BM, n0 = blockIdx.x * GF_BN;
    const int lrow = tid / 4, lk = (tid % 4) * 4;
    const bool vec_ok = (K % 4 == 0) && (lda % 4 == 0) && (ldw % 4 == 0);

    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += GF_BK) {
        float a[4] = {0.f, 0.f, 0.f, 0.f}, w[4] = {0.f, 0.f, 0.f, 0.f};
        const int am = m0 + lrow, wn = n0 + lrow, kk = k0 + lk;
        if (am < M) {
            const float *p = A + (size_t)am * lda + kk;
            if (vec_ok && kk + 3 < K) {
                const float4 v = *reinterpret_cast<const float4 *>(p);
                a[0] = v.x; a[1] = v.y; a[2] = v.z; a[3] = v.w;
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (kk + e < K) a[e] = p[e];
            }
        }
        if (wn < N) {
            const float *p = W + (size_t)wn * ldw + kk;
            if (vec_ok && kk + 3 < K) {
                const float4 v = *reinterpret_cast<const float4 *>(p);
                w[0] = v.x; w[1] = v.y; w[2] = v.z; w[3] = v.w;
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (kk + e < K) w[e] = p[e];
            }
        }
        __syncthreads();
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            As[lk + e][lrow] = a[e];
            Ws[lk + e][lrow] = w[e];
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < GF_BK; ++k) {
            float av[4], wv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) av[i] = As[k][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) wv[j] = Ws[k][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n < N) C[(size_t)m * ldc + n] = acc[i][j];
        }
    }
}

extern "C" int kva_gemm_nt_f32(float *C, const float *A, const float *W, int M, int N, int K,
                               int lda, int ldw, int ldc, hipStream_t stream) {
    KVA_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_f32: bad sizes M=%d N=%d K=%d", M, N, K);
    KVA_REQUIRE(lda >= K && ldw >= K && ldc >= N, "gemm_f32: leading dimensions too small");
    if (M == 0) return KVA_OK;
    dim3 grid((N + GF_BN - 1) / GF_BN, (M + GF_BM - 1) / GF_BM), block(256);
    KVA_REQUIRE(grid.y <= 65535, "gemm_f32: M=%d is too large for one launch", M);
    hipLaunchKernelGGL(gemm_nt_f32_kernel, grid, block, 0, stream, C, A, W, M, N, K, lda, ldw, ldc);
    KVA_CHECK_LAUNCH("gemm_nt_f32");
    return KVA_OK;
}
