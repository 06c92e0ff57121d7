// Shared device helpers for the gfx950 kernels: bf16 storage type, 64-lane wavefront
// reductions, vector loads and the launch-error convention of the extern "C" entry points.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define KVA_WAVE 64

// Every entry point returns 0 on success or a negative code; the Python side turns the
// code into an exception with kva_last_error().
#define KVA_OK 0
#define KVA_ERR_ARG (-1)
#define KVA_ERR_LAUNCH (-2)

extern "C" const char *kva_last_error();
void kva_set_error(const char *fmt, ...);

#define KVA_REQUIRE(cond, ...)                                                             \
    do {                                                                                   \
        if (!(cond)) {                                                                     \
            kva_set_error(__VA_ARGS__);                                                    \
            return KVA_ERR_ARG;                                                            \
        }                                                                                  \
    } while (0)

#define KVA_CHECK_LAUNCH(name)                                                             \
    do {                                                                                   \
        hipError_t e_ = hipGetLastError();                                                 \
        if (e_ != hipSuccess) {                                                            \
            kva_set_error("%s: launch failed: %s", name, hipGetErrorString(e_));           \
            return KVA_ERR_LAUNCH;                                                         \
        }                                                                                  \
    } while (0)

// ---- bfloat16 as a storage type -------------------------------------------------------
// All arithmetic is done in float; bf16 is only ever loaded from and stored to memory.
struct bf16_t {
    uint16_t bits;
};

__host__ __device__ inline float bf16_bits_to_float(uint16_t b) {
    union { uint32_t u; float f; } c;
    c.u = ((uint32_t)b) << 16;
    return c.f;
}

// round to nearest, ties to even; NaN stays NaN
__host__ __device__ inline uint16_t float_to_bf16_bits(float f) {
    union { uint32_t u; float f; } c;
    c.f = f;
    uint32_t u = c.u;
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

__host__ __device__ inline float to_float(float v) { return v; }
__host__ __device__ inline float to_float(bf16_t v) { return bf16_bits_to_float(v.bits); }

template <typename T> __host__ __device__ inline T from_float(float f);
template <> __host__ __device__ inline float from_float<float>(float f) { return f; }
template <> __host__ __device__ inline bf16_t from_float<bf16_t>(float f) {
    bf16_t r;
    r.bits = float_to_bf16_bits(f);
    return r;
}

// ---- wavefront (64 lanes) reductions ---------------------------------------------------
__device__ inline float wave_sum(float v) {
#pragma unroll
    for (int off = KVA_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, KVA_WAVE);
    return v;
}

__device__ inline float wave_max(float v) {
#pragma unroll
    for (int off = KVA_WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, KVA_WAVE));
    return v;
}

// Loads with the non-temporal hint, for data that is read once per kernel and will have left the
// caches before it is wanted again (weights at decode time, the KV pages of decoded tokens): what
// else lives in L2 stays there.
typedef unsigned int kva_u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int kva_u32x2 __attribute__((ext_vector_type(2)));
__device__ inline uint4 load_streamed_u4(const void *p) {
    const kva_u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const kva_u32x4 *>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ inline uint2 load_streamed_u2(const void *p) {
    const kva_u32x2 v = __builtin_nontemporal_load(reinterpret_cast<const kva_u32x2 *>(p));
    return make_uint2(v.x, v.y);
}

// Reductions over the four lanes {r, r + 16, r + 32, r + 48} (r = lane % 16), every one of them
// getting the result.  v_permlane16_swap / v_permlane32_swap exchange 16- and 32-lane halves
// between two registers in the vector ALU (no trip through LDS as a wave shuffle takes): from two
// copies of x they leave (x of the lower half, x of the upper half) in every lane.
__device__ inline float quad_rows_sum(float x) {
    const unsigned u = __float_as_uint(x);
    auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    const float y = __uint_as_float(a[0]) + __uint_as_float(a[1]);
    const unsigned v = __float_as_uint(y);
    auto b = __builtin_amdgcn_permlane32_swap(v, v, false, false);
    return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

__device__ inline float quad_rows_max(float x) {
    const unsigned u = __float_as_uint(x);
    auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    const float y = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
    const unsigned v = __float_as_uint(y);
    auto b = __builtin_amdgcn_permlane32_swap(v, v, false, false);
    return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}

// Sum over the 16 lanes of a row (lanes 16 i .. 16 i + 15), every one of them getting it: four
// rotations within the row, done by the data-parallel-primitive path of the vector ALU.
template <int ROTATE>
__device__ inline float row16_rotated(float v) {
    return __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(v), 0x120 | ROTATE, 0xf, 0xf, false));
}
__device__ inline float row16_sum(float v) {
    v += row16_rotated<8>(v);
    v += row16_rotated<4>(v);
    v += row16_rotated<2>(v);
    v += row16_rotated<1>(v);
    return v;
}

// wave_sum without a trip through LDS: a chain of about a hundred cycles instead of six shuffles
// of about a hundred each, for kernels that are as short as that chain.  The additions are in
// another order than wave_sum's.
__device__ inline float wave_sum_valu(float v) { return quad_rows_sum(row16_sum(v)); }

// 8 neighbouring elements of the sum of `parts` fp32 partial products laid out [parts][rows][width]
// (row: the row's start in range 0, stride: rows * width), each rounded to bf16 as the whole product
// would have been.  Four ranges at a time, all eight loads asked for before the first is added (a
// plain loop over the ranges is a trip to memory per range); added in the order of the ranges.
__device__ inline void sum_ranges8(const float *row, int parts, size_t stride, int i, float (&f)[8]) {
    float4 lo = make_float4(0.f, 0.f, 0.f, 0.f), hi = lo;
    for (int s0 = 0; s0 < parts; s0 += 4) {
        float4 a[4], b[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int s = s0 + j < parts ? s0 + j : parts - 1;
            a[j] = *reinterpret_cast<const float4 *>(row + (size_t)s * stride + i);
            b[j] = *reinterpret_cast<const float4 *>(row + (size_t)s * stride + i + 4);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (s0 + j < parts) {
                lo.x += a[j].x; lo.y += a[j].y; lo.z += a[j].z; lo.w += a[j].w;
                hi.x += b[j].x; hi.y += b[j].y; hi.z += b[j].z; hi.w += b[j].w;
            }
        }
    }
    const float t[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
    for (int j = 0; j < 8; ++j) f[j] = bf16_bits_to_float(float_to_bf16_bits(t[j]));
}


// Sum over a whole workgroup of `nwaves` wavefronts; `scratch` holds at least nwaves floats.
// Every thread gets the result.  The order of the additions is fixed.
__device__ inline float block_sum(float v, float *scratch, int nwaves) {
    v = wave_sum(v);
    const int lane = threadIdx.x % KVA_WAVE, wave = threadIdx.x / KVA_WAVE;
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = 0.f;
    for (int w = 0; w < nwaves; ++w) total += scratch[w];
    return total;
}

enum KvaDtype { KVA_F32 = 0, KVA_BF16 = 1 };
