// Embedding gather, RMSNorm (optionally fused with the residual add before it and with a row
// gather), SwiGLU activation and dtype casts.  One workgroup handles one row; all arithmetic
// is fp32 whatever the storage type is.
//
// Formulas follow the reference's kernels: rmsNormKernel (base/src/kernels.cu:10-36),
// residualKernel (:38-43), siluKernel (:45-52), embeddingGatherKernel (:279-287) and
// gatherRowsKernel (:472-480).
#include "common.h"
#include <algorithm>
#include <stdarg.h>
#include <stdio.h>

static thread_local char g_error[512] = "";

extern "C" const char *kva_last_error() { return g_error; }

void kva_set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

// ---------------------------------------------------------------------------------------
// A negative id names a token that is still on the device: id = -1 - r stands for feedback[r]
// (the token a sampling kernel left in row r of its output), so a decode step can be launched
// before the host has seen the token it continues from.
template <typename TW, typename TO>
__global__ void embed_gather_kernel(TO *__restrict__ out, const TW *__restrict__ table,
                                    const int *__restrict__ ids, const int *__restrict__ feedback,
                                    int width, int table_rows) {
    const int row = blockIdx.x;
    int id = ids[row];
    if (id < 0) id = feedback[-1 - id];
    id = id < 0 ? 0 : (id >= table_rows ? table_rows - 1 : id);      // whatever a kernel left there: inside the table
    const TW *src = table + (size_t)id * width;
    TO *dst = out + (size_t)row * width;
    for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = from_float<TO>(to_float(src[i]));
}

// feedback may be null when no id is negative (the caller checks the ids it uploads).
extern "C" int kva_embed_gather(void *out, const void *table, const int *ids, const int *feedback,
                                int rows, int width, int table_rows, int table_dtype, int out_dtype,
                                hipStream_t stream) {
    KVA_REQUIRE(rows >= 0 && width > 0 && table_rows > 0, "embed_gather: bad sizes rows=%d width=%d table rows=%d",
                rows, width, table_rows);
    if (rows == 0) return KVA_OK;
    dim3 grid(rows), block(256);
#define LAUNCH(TW, TO)                                                                    \
    hipLaunchKernelGGL((embed_gather_kernel<TW, TO>), grid, block, 0, stream, (TO *)out, \
                       (const TW *)table, ids, feedback, width, table_rows)
    if (table_dtype == KVA_F32 && out_dtype == KVA_F32) LAUNCH(float, float);
    else if (table_dtype == KVA_BF16 && out_dtype == KVA_BF16) LAUNCH(bf16_t, bf16_t);
    else if (table_dtype == KVA_F32 && out_dtype == KVA_BF16) LAUNCH(float, bf16_t);
    else if (table_dtype == KVA_BF16 && out_dtype == KVA_F32) LAUNCH(bf16_t, float);
    else KVA_REQUIRE(false, "embed_gather: unsupported dtypes %d -> %d", table_dtype, out_dtype);
#undef LAUNCH
    KVA_CHECK_LAUNCH("embed_gather");
    return KVA_OK;
}

// ---------------------------------------------------------------------------------------
// y = (x / sqrt(mean(x^2) + eps)) * w.  The sum of squares is fp32, the sqrt runs in double
// as the reference's does.  With `delta`, the norm is taken of s = round(hidden + delta) (fp32
// add, rounded to the storage type), which is what a separate residual kernel followed by a norm
// kernel would see; s is written back to hidden unless rows are gathered.  With `row_idx`,
// output row i is the norm of input row row_idx[i] and hidden is left untouched (a row may be
// named twice).
template <typename T, typename TW>
__global__ void rmsnorm_kernel(T *__restrict__ out, T *__restrict__ hidden,
                               const T *__restrict__ delta, const TW *__restrict__ weight,
                               const int *__restrict__ row_idx, int width, float eps) {
    __shared__ float scratch[16];
    const int orow = blockIdx.x;
    const int irow = row_idx ? row_idx[orow] : orow;
    T *x = hidden + (size_t)irow * width;
    const T *dl = delta ? delta + (size_t)irow * width : nullptr;
    const bool write_back = dl && !row_idx;
    T *y = out + (size_t)orow * width;
    float ss = 0.f;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        float v = to_float(x[i]);
        if (dl) {
            const T r = from_float<T>(v + to_float(dl[i]));
            if (write_back) x[i] = r;
            v = to_float(r);
        }
        ss += v * v;
    }
    const float total = block_sum(ss, scratch, blockDim.x / KVA_WAVE);
    const float r = (float)sqrt((double)total / (double)width + (double)eps);
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        float v = to_float(x[i]);
        if (dl && !write_back) v = to_float(from_float<T>(v + to_float(dl[i])));
        y[i] = from_float<T>((v / r) * to_float(weight[i]));
    }
}

// The same for bf16 rows whose width is a multiple of 8: 16-byte loads and stores, the row (after
// the optional add) kept in registers between the two passes when it fits.
__device__ inline void unpack8(const uint4 &v, float (&f)[8]) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        f[2 * i] = bf16_bits_to_float((uint16_t)(w[i] & 0xffffu));
        f[2 * i + 1] = bf16_bits_to_float((uint16_t)(w[i] >> 16));
    }
}

__device__ inline uint4 pack8(const float (&f)[8]) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
        w[i] = (uint32_t)float_to_bf16_bits(f[2 * i]) | ((uint32_t)float_to_bf16_bits(f[2 * i + 1]) << 16);
    return make_uint4(w[0], w[1], w[2], w[3]);
}

template <typename TW> __device__ inline void load_weight8(const TW *w, float (&f)[8]);
template <> __device__ inline void load_weight8<bf16_t>(const bf16_t *w, float (&f)[8]) {
    unpack8(*reinterpret_cast<const uint4 *>(w), f);
}
template <> __device__ inline void load_weight8<float>(const float *w, float (&f)[8]) {
    const float4 a = *reinterpret_cast<const float4 *>(w), b = *reinterpret_cast<const float4 *>(w + 4);
    f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
}

// The gather for a few tokens of a bf16 model, with the first norm prepared in the same pass, as a
// product's residual epilogue prepares the norm after it: hidden[t, :] = table[id, :],
// scaled[t, :] = round(hidden * w_norm), sumsq[t] = sum hidden^2.  A decode step saves the
// norm kernel that would read back what this one has just written.
template <typename TW>
__global__ void __launch_bounds__(256)
embed_gather_prep_kernel(bf16_t *__restrict__ hidden, bf16_t *__restrict__ scaled, float *__restrict__ sumsq,
                         const bf16_t *__restrict__ table, const int *__restrict__ ids,
                         const int *__restrict__ feedback, const TW *__restrict__ norm_w, int width,
                         int table_rows) {
    __shared__ float scratch[4];
    const int row = blockIdx.x;
    int id = ids[row];
    if (id < 0) id = feedback[-1 - id];
    id = id < 0 ? 0 : (id >= table_rows ? table_rows - 1 : id);
    const bf16_t *src = table + (size_t)id * width;
    float ss = 0.f;
    for (int i = threadIdx.x * 8; i < width; i += blockDim.x * 8) {
        const uint4 raw = *reinterpret_cast<const uint4 *>(src + i);
        float v[8], w[8];
        unpack8(raw, v);
        load_weight8<TW>(norm_w + i, w);
        *reinterpret_cast<uint4 *>(hidden + (size_t)row * width + i) = raw;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            ss += v[j] * v[j];
            v[j] *= w[j];
        }
        *reinterpret_cast<uint4 *>(scaled + (size_t)row * width + i) = pack8(v);
    }
    const float total = block_sum(ss, scratch, blockDim.x / KVA_WAVE);
    if (threadIdx.x == 0) sumsq[row] = total;
}

// bf16 table and outputs, width a multiple of 8; norm_w [width] bf16 or fp32.
extern "C" int kva_embed_gather_prep(void *hidden, void *scaled, float *sumsq, const void *table, const int *ids,
                                     const int *feedback, const void *norm_w, int norm_w_f32, int rows, int width,
                                     int table_rows, hipStream_t stream) {
    KVA_REQUIRE(rows >= 0 && width > 0 && width % 8 == 0 && table_rows > 0,
                "embed_gather_prep: bad sizes rows=%d width=%d (a multiple of 8) table rows=%d", rows, width, table_rows);
    KVA_REQUIRE(hidden && scaled && sumsq && table && ids && norm_w, "embed_gather_prep: a pointer is missing");
    if (rows == 0) return KVA_OK;
    dim3 grid(rows), block(256);
    if (norm_w_f32)
        hipLaunchKernelGGL(embed_gather_prep_kernel<float>, grid, block, 0, stream, (bf16_t *)hidden, (bf16_t *)scaled,
                           sumsq, (const bf16_t *)table, ids, feedback, (const float *)norm_w, width, table_rows);
    else
        hipLaunchKernelGGL(embed_gather_prep_kernel<bf16_t>, grid, block, 0, stream, (bf16_t *)hidden, (bf16_t *)scaled,
                           sumsq, (const bf16_t *)table, ids, feedback, (const bf16_t *)norm_w, width, table_rows);
    KVA_CHECK_LAUNCH("embed_gather_prep");
    return KVA_OK;
}

#define RMS_VEC_CACHE 4   // vectors of 8 a thread keeps between the passes
// 8 elements of the branch output that is added to the stream: from the bf16 delta, or (parts > 0)
// the sum of `parts` fp32 partial products [parts][rows][width], rounded to bf16 as the product
// itself would have been
__device__ inline void load_delta8(const bf16_t *dl, const float *parts_row, int parts, size_t part_stride, int i,
                                   float (&d)[8]) {
    if (parts > 0) {
        sum_ranges8(parts_row, parts, part_stride, i, d);
    } else {
        unpack8(*reinterpret_cast<const uint4 *>(dl + i), d);
    }
}

template <typename TW>
__global__ void rmsnorm_vec_kernel(bf16_t *__restrict__ out, bf16_t *__restrict__ hidden,
                                   const bf16_t *__restrict__ delta, const float *__restrict__ delta_parts,
                                   int parts, size_t part_stride, const TW *__restrict__ weight,
                                   const int *__restrict__ row_idx, int width, float eps) {
    __shared__ float scratch[16];
    const int orow = blockIdx.x;
    const int irow = row_idx ? row_idx[orow] : orow;
    bf16_t *x = hidden + (size_t)irow * width;
    const bf16_t *dl = delta ? delta + (size_t)irow * width : nullptr;
    const float *pr = parts > 0 ? delta_parts + (size_t)irow * width : nullptr;
    const bool adds = dl != nullptr || parts > 0;
    const bool write_back = adds && !row_idx;
    bf16_t *y = out + (size_t)orow * width;
    float cache[RMS_VEC_CACHE][8];
    float ss = 0.f;
    int c = 0;
    for (int i = threadIdx.x * 8; i < width; i += blockDim.x * 8, ++c) {
        float v[8];
        unpack8(*reinterpret_cast<const uint4 *>(x + i), v);
        if (adds) {
            float d[8];
            load_delta8(dl, pr, parts, part_stride, i, d);
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = bf16_bits_to_float(float_to_bf16_bits(v[j] + d[j]));
            if (write_back) *reinterpret_cast<uint4 *>(x + i) = pack8(v);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) ss += v[j] * v[j];
        if (c < RMS_VEC_CACHE) {
#pragma unroll
            for (int j = 0; j < 8; ++j) cache[c][j] = v[j];
        }
    }
    const float total = block_sum(ss, scratch, blockDim.x / KVA_WAVE);
    const float r = (float)sqrt((double)total / (double)width + (double)eps);
    c = 0;
    for (int i = threadIdx.x * 8; i < width; i += blockDim.x * 8, ++c) {
        float v[8], w[8];
        if (c < RMS_VEC_CACHE) {
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = cache[c][j];
        } else {
            unpack8(*reinterpret_cast<const uint4 *>(x + i), v);
            if (adds && !write_back) {
                float d[8];
                load_delta8(dl, pr, parts, part_stride, i, d);
#pragma unroll
                for (int j = 0; j < 8; ++j) v[j] = bf16_bits_to_float(float_to_bf16_bits(v[j] + d[j]));
            }
        }
        load_weight8<TW>(weight + i, w);
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = (v[j] / r) * w[j];
        *reinterpret_cast<uint4 *>(y + i) = pack8(v);
    }
}

// delta_parts (bf16 rows of a width that is a multiple of 8 only): instead of delta, `parts` fp32
// partial products [parts][part_rows][width] whose sum, rounded to bf16, is what is added.
extern "C" int kva_rmsnorm(void *out, void *hidden, const void *delta, const void *weight,
                           const int *row_idx, int out_rows, int width, float eps, int dtype,
                           int weight_dtype, const float *delta_parts, int parts, int part_rows,
                           hipStream_t stream) {
    KVA_REQUIRE(out_rows >= 0 && width > 0, "rmsnorm: bad sizes rows=%d width=%d", out_rows, width);
    KVA_REQUIRE(parts == 0 || (delta_parts != nullptr && delta == nullptr && parts > 0 && part_rows > 0 &&
                               dtype == KVA_BF16 && width % 8 == 0),
                "rmsnorm: partial products stand in for a bf16 delta of a width that is a multiple of 8");
    if (out_rows == 0) return KVA_OK;
    if (dtype == KVA_BF16 && width % 8 == 0) {
        // Many rows (prompt portions): 256 threads walk a row of up to 8,184 columns in several turns and
        // the workgroups overlap each other's waits.  Few rows (decode steps): a thread per 8 columns
        // where a workgroup allows, every load of the row asked for at once (4,096 columns, 64 rows:
        // 5.3 -> 4.5 us, with partial products in 8 ranges 9.2 -> 7.0; 2,048 rows: 18.6 -> 20.9, so not there).
        int threads = width >= 8192 ? 1024 : (width >= 2048 ? 256 : (width >= 1024 ? 128 : 64));
        if (out_rows <= 256) threads = std::min(1024, std::max(64, (width / 8 + 63) / 64 * 64));
        dim3 vgrid(out_rows), vblock(threads);
        const size_t part_stride = (size_t)part_rows * width;
        if (weight_dtype == KVA_BF16)
            hipLaunchKernelGGL(rmsnorm_vec_kernel<bf16_t>, vgrid, vblock, 0, stream, (bf16_t *)out,
                               (bf16_t *)hidden, (const bf16_t *)delta, delta_parts, parts, part_stride,
                               (const bf16_t *)weight, row_idx, width, eps);
        else if (weight_dtype == KVA_F32)
            hipLaunchKernelGGL(rmsnorm_vec_kernel<float>, vgrid, vblock, 0, stream, (bf16_t *)out,
                               (bf16_t *)hidden, (const bf16_t *)delta, delta_parts, parts, part_stride,
                               (const float *)weight, row_idx, width, eps);
        else KVA_REQUIRE(false, "rmsnorm: unsupported weight dtype %d", weight_dtype);
        KVA_CHECK_LAUNCH("rmsnorm");
        return KVA_OK;
    }
    dim3 grid(out_rows), block(width >= 2048 ? 512 : 256);
#define LAUNCH(T, TW)                                                                      \
    hipLaunchKernelGGL((rmsnorm_kernel<T, TW>), grid, block, 0, stream, (T *)out, (T *)hidden, \
                       (const T *)delta, (const TW *)weight, row_idx, width, eps)
    if (dtype == KVA_F32 && weight_dtype == KVA_F32) LAUNCH(float, float);
    else if (dtype == KVA_BF16 && weight_dtype == KVA_BF16) LAUNCH(bf16_t, bf16_t);
    else if (dtype == KVA_BF16 && weight_dtype == KVA_F32) LAUNCH(bf16_t, float);
    else if (dtype == KVA_F32 && weight_dtype == KVA_BF16) LAUNCH(float, bf16_t);
    else KVA_REQUIRE(false, "rmsnorm: unsupported dtypes %d / %d", dtype, weight_dtype);
#undef LAUNCH
    KVA_CHECK_LAUNCH("rmsnorm");
    return KVA_OK;
}

// ---------------------------------------------------------------------------------------
// hidden <- hidden + delta, fp32 add, rounded to the storage type.
template <typename T>
__global__ void residual_add_kernel(T *__restrict__ hidden, const T *__restrict__ delta, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) hidden[i] = from_float<T>(to_float(hidden[i]) + to_float(delta[i]));
}

extern "C" int kva_residual_add(void *hidden, const void *delta, long long n, int dtype,
                                hipStream_t stream) {
    KVA_REQUIRE(n >= 0, "residual_add: bad size");
    if (n == 0) return KVA_OK;
    int blocks = (int)((n + 255) / 256);
    if (blocks > 8192) blocks = 8192;
    if (dtype == KVA_F32)
        hipLaunchKernelGGL(residual_add_kernel<float>, dim3(blocks), dim3(256), 0, stream,
                           (float *)hidden, (const float *)delta, (size_t)n);
    else if (dtype == KVA_BF16)
        hipLaunchKernelGGL(residual_add_kernel<bf16_t>, dim3(blocks), dim3(256), 0, stream,
                           (bf16_t *)hidden, (const bf16_t *)delta, (size_t)n);
    else KVA_REQUIRE(false, "residual_add: unsupported dtype %d", dtype);
    KVA_CHECK_LAUNCH("residual_add");
    return KVA_OK;
}

// ---------------------------------------------------------------------------------------
// A probe, not a part of the model: reads `count` 16-byte units once (non-temporal loads, four in
// flight per lane) and stores nothing.  Its time is the floor for any kernel that has to read as
// many bytes, and bytes / time the memory bandwidth this GPU gives a plain stream.
__global__ void __launch_bounds__(256) stream_read_kernel(const uint4 *__restrict__ p, size_t count,
                                                          unsigned *__restrict__ sink) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    unsigned acc = 0;
    for (; i + 3 * stride < count; i += 4 * stride) {
        const uint4 a = load_streamed_u4(p + i), b = load_streamed_u4(p + i + stride);
        const uint4 c = load_streamed_u4(p + i + 2 * stride), d = load_streamed_u4(p + i + 3 * stride);
        acc ^= a.x ^ b.y ^ c.z ^ d.w;
    }
    for (; i < count; i += stride) acc ^= load_streamed_u4(p + i).x;
    // practically never true; it keeps the loads from being dropped
    if (acc == 0x9E3779B9u && threadIdx.x == 255 && sink != nullptr) *sink = acc;
}

extern "C" int kva_stream_read(const void *p, long long bytes, int workgroups, void *sink, hipStream_t stream) {
    KVA_REQUIRE(workgroups >= 1 && workgroups <= 65535, "stream_read: 1..65535 workgroups");
    KVA_REQUIRE(bytes >= 0 && p != nullptr && ((uintptr_t)p % 16) == 0, "stream_read: a 16-byte aligned range is needed");
    if (bytes < 16) return KVA_OK;
    hipLaunchKernelGGL(stream_read_kernel, dim3(workgroups), dim3(256), 0, stream, (const uint4 *)p,
                       (size_t)(bytes / 16), (unsigned *)sink);
    KVA_CHECK_LAUNCH("stream_read");
    return KVA_OK;
}

// Another probe: EVERY workgroup reads all `count` 16-byte units, `repeats` times over, through the
// caches (plain loads, four in flight per lane).  With a range that fits the L2 of a die this is
// what a compute unit can take in from L2 - the rows of X that every workgroup of a few-rows
// product has to read beside its share of the weights.
__global__ void __launch_bounds__(256) stream_reread_kernel(const uint4 *__restrict__ p, size_t count, int repeats,
                                                            unsigned *__restrict__ sink) {
    unsigned acc = 0;
    for (int rep = 0; rep < repeats; ++rep) {
        size_t i = threadIdx.x;
        for (; i + 3 * 256 < count; i += 4 * 256) {
            const uint4 a = p[i], b = p[i + 256], c = p[i + 512], d = p[i + 768];
            acc ^= a.x ^ b.y ^ c.z ^ d.w;
        }
        for (; i < count; i += 256) acc ^= p[i].x;
        acc += rep;                                  // (the turns are not the same expression)
    }
    if (acc == 0x9E3779B9u && threadIdx.x == 255 && sink != nullptr) *sink = acc;
}

extern "C" int kva_stream_reread(const void *p, long long bytes, int workgroups, int repeats, void *sink,
                                 hipStream_t stream) {
    KVA_REQUIRE(workgroups >= 1 && workgroups <= 65535 && repeats >= 1, "stream_reread: 1..65535 workgroups, at least one turn");
    KVA_REQUIRE(bytes >= 16 && p != nullptr && ((uintptr_t)p % 16) == 0, "stream_reread: a 16-byte aligned range is needed");
    hipLaunchKernelGGL(stream_reread_kernel, dim3(workgroups), dim3(256), 0, stream, (const uint4 *)p,
                       (size_t)(bytes / 16), repeats, (unsigned *)sink);
    KVA_CHECK_LAUNCH("stream_reread");
    return KVA_OK;
}

// A probe of two streams into one compute unit at once.  Half of a workgroup's wavefronts read a
// range of the workgroup's own (from memory: streamed loads, every workgroup another range), the
// other half read a range that all workgroups share (from L2 after its first reader).  Either
// range may be empty.  Against the two alone this shows whether bytes that hit in L2 come for less
// than bytes from memory while a compute unit is also waiting for memory - the question behind
// the rows of X in a few-rows product.
__global__ void __launch_bounds__(512) stream_mixed_kernel(const uint4 *__restrict__ own, size_t own_count,
                                                           const uint4 *__restrict__ shared, size_t shared_count,
                                                           unsigned *__restrict__ sink) {
    unsigned acc = 0;
    const int t = threadIdx.x & 255;
    if (threadIdx.x < 256) {
        const uint4 *p = own + (size_t)blockIdx.x * own_count;
        size_t i = t;
        for (; i + 3 * 256 < own_count; i += 4 * 256) {
            const uint4 a = load_streamed_u4(p + i), b = load_streamed_u4(p + i + 256);
            const uint4 c = load_streamed_u4(p + i + 512), d = load_streamed_u4(p + i + 768);
            acc ^= a.x ^ b.y ^ c.z ^ d.w;
        }
        for (; i < own_count; i += 256) acc ^= load_streamed_u4(p + i).x;
    } else {
        size_t i = t;
        for (; i + 3 * 256 < shared_count; i += 4 * 256) {
            const uint4 a = shared[i], b = shared[i + 256], c = shared[i + 512], d = shared[i + 768];
            acc ^= a.x ^ b.y ^ c.z ^ d.w;
        }
        for (; i < shared_count; i += 256) acc ^= shared[i].x;
    }
    if (acc == 0x9E3779B9u && t == 255 && sink != nullptr) *sink = acc;
}

// own: workgroups x own_bytes; shared: shared_bytes (both may be 0 bytes, not both)
extern "C" int kva_stream_mixed(const void *own, long long own_bytes, const void *shared, long long shared_bytes,
                                int workgroups, void *sink, hipStream_t stream) {
    KVA_REQUIRE(workgroups >= 1 && workgroups <= 65535, "stream_mixed: 1..65535 workgroups");
    KVA_REQUIRE(own_bytes >= 0 && shared_bytes >= 0 && own_bytes + shared_bytes > 0 && own_bytes % 16 == 0 &&
                shared_bytes % 16 == 0, "stream_mixed: ranges in multiples of 16 bytes, one of them not empty");
    KVA_REQUIRE((own_bytes == 0 || (own && (uintptr_t)own % 16 == 0)) &&
                (shared_bytes == 0 || (shared && (uintptr_t)shared % 16 == 0)), "stream_mixed: 16-byte aligned ranges are needed");
    hipLaunchKernelGGL(stream_mixed_kernel, dim3(workgroups), dim3(512), 0, stream, (const uint4 *)own,
                       (size_t)(own_bytes / 16), (const uint4 *)shared, (size_t)(shared_bytes / 16), (unsigned *)sink);
    KVA_CHECK_LAUNCH("stream_mixed");
    return KVA_OK;
}

// ---------------------------------------------------------------------------------------
// x <- x * scale, and then, with cap > 0, x <- cap * tanh(x / cap): the constants a model may put
// on its embeddings and on its logits.  fp32 arithmetic, rounded to the storage type.
template <typename T>
__global__ void scale_softcap_kernel(T *__restrict__ x, size_t n, float scale, float cap) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    const float inv_cap = cap > 0.f ? 1.f / cap : 0.f;
    for (; i < n; i += stride) {
        float v = to_float(x[i]) * scale;
        if (cap > 0.f) v = cap * tanhf(v * inv_cap);
        x[i] = from_float<T>(v);
    }
}

extern "C" int kva_scale_softcap(void *x, long long n, float scale, float cap, int dtype, hipStream_t stream) {
    KVA_REQUIRE(n >= 0 && cap >= 0.f, "scale_softcap: bad size or a negative cap");
    if (n == 0) return KVA_OK;
    int blocks = (int)((n + 255) / 256);
    if (blocks > 8192) blocks = 8192;
    if (dtype == KVA_F32)
        hipLaunchKernelGGL(scale_softcap_kernel<float>, dim3(blocks), dim3(256), 0, stream, (float *)x, (size_t)n,
                           scale, cap);
    else if (dtype == KVA_BF16)
        hipLaunchKernelGGL(scale_softcap_kernel<bf16_t>, dim3(blocks), dim3(256), 0, stream, (bf16_t *)x,
                           (size_t)n, scale, cap);
    else KVA_REQUIRE(false, "scale_softcap: unsupported dtype %d", dtype);
    KVA_CHECK_LAUNCH("scale_softcap");
    return KVA_OK;
}

// ---------------------------------------------------------------------------------------
// out[t, i] = silu(gu[t, i]) * gu[t, inter + i]; silu(g) = g / (1 + exp(-g)) in fp32.
template <typename T>
__global__ void silu_mul_kernel(T *__restrict__ out, const T *__restrict__ gate_up, int inter) {
    const int row = blockIdx.y;
    const T *g = gate_up + (size_t)row * 2 * inter;
    const T *u = g + inter;
    T *o = out + (size_t)row * inter;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < inter; i += gridDim.x * blockDim.x) {
        const float gv = to_float(g[i]);
        o[i] = from_float<T>(gv * (1.f / (1.f + expf(-gv))) * to_float(u[i]));
    }
}

__global__ void silu_mul_vec_kernel(bf16_t *__restrict__ out, const bf16_t *__restrict__ gate_up, int inter) {
    const int row = blockIdx.y;
    const bf16_t *g = gate_up + (size_t)row * 2 * inter;
    const bf16_t *u = g + inter;
    bf16_t *o = out + (size_t)row * inter;
    for (int i = (blockIdx.x * blockDim.x + threadIdx.x) * 8; i < inter; i += gridDim.x * blockDim.x * 8) {
        float gv[8], uv[8];
        unpack8(*reinterpret_cast<const uint4 *>(g + i), gv);
        unpack8(*reinterpret_cast<const uint4 *>(u + i), uv);
#pragma unroll
        for (int j = 0; j < 8; ++j) gv[j] = gv[j] * (1.f / (1.f + expf(-gv[j]))) * uv[j];
        *reinterpret_cast<uint4 *>(o + i) = pack8(gv);
    }
}

extern "C" int kva_silu_mul(void *out, const void *gate_up, int rows, int inter, int dtype,
                            hipStream_t stream) {
    KVA_REQUIRE(rows >= 0 && inter > 0, "silu_mul: bad sizes");
    KVA_REQUIRE(rows <= 65535, "silu_mul: at most 65535 rows per call, got %d", rows);
    if (rows == 0) return KVA_OK;
    if (dtype == KVA_BF16 && inter % 8 == 0) {
        int vbx = (inter / 8 + 255) / 256;
        hipLaunchKernelGGL(silu_mul_vec_kernel, dim3(vbx, rows), dim3(256), 0, stream, (bf16_t *)out,
                           (const bf16_t *)gate_up, inter);
        KVA_CHECK_LAUNCH("silu_mul");
        return KVA_OK;
    }
    int bx = (inter + 255) / 256;
    if (bx > 64) bx = 64;
    dim3 grid(bx, rows), block(256);
    if (dtype == KVA_F32)
        hipLaunchKernelGGL(silu_mul_kernel<float>, grid, block, 0, stream, (float *)out,
                           (const float *)gate_up, inter);
    else if (dtype == KVA_BF16)
        hipLaunchKernelGGL(silu_mul_kernel<bf16_t>, grid, block, 0, stream, (bf16_t *)out,
                           (const bf16_t *)gate_up, inter);
    else KVA_REQUIRE(false, "silu_mul: unsupported dtype %d", dtype);
    KVA_CHECK_LAUNCH("silu_mul");
    return KVA_OK;
}

// ---------------------------------------------------------------------------------------
template <typename TI, typename TO>
__global__ void cast_kernel(TO *__restrict__ out, const TI *__restrict__ in, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) out[i] = from_float<TO>(to_float(in[i]));
}

extern "C" int kva_cast(void *out, const void *in, long long n, int in_dtype, int out_dtype,
                        hipStream_t stream) {
    KVA_REQUIRE(n >= 0, "cast: bad size");
    if (n == 0) return KVA_OK;
    int blocks = (int)((n + 255) / 256);
    if (blocks > 8192) blocks = 8192;
    if (in_dtype == KVA_BF16 && out_dtype == KVA_F32)
        hipLaunchKernelGGL((cast_kernel<bf16_t, float>), dim3(blocks), dim3(256), 0, stream,
                           (float *)out, (const bf16_t *)in, (size_t)n);
    else if (in_dtype == KVA_F32 && out_dtype == KVA_BF16)
        hipLaunchKernelGGL((cast_kernel<float, bf16_t>), dim3(blocks), dim3(256), 0, stream,
                           (bf16_t *)out, (const float *)in, (size_t)n);
    else KVA_REQUIRE(false, "cast: unsupported dtypes %d -> %d", in_dtype, out_dtype);
    KVA_CHECK_LAUNCH("cast");
    return KVA_OK;
}

// ---------------------------------------------------------------------------------------
// Finishes an RMSNorm that a matrix product's epilogue prepared: `scaled` holds
// round(hidden * w_norm), `sumsq` [T, parts] partial sums of hidden^2 per row;
// out[i, :] = scaled[row, :] * rsqrt(sum(sumsq[row]) / width + eps), row = row_idx[i] or i.
__global__ void normed_rows_finish_kernel(bf16_t *__restrict__ out, const bf16_t *__restrict__ scaled,
                                          const float *__restrict__ sumsq, int parts,
                                          const int *__restrict__ row_idx, int width, float eps) {
    __shared__ float scratch[16];
    const int orow = blockIdx.x;
    const int irow = row_idx ? row_idx[orow] : orow;
    float s = 0.f;
    for (int p = threadIdx.x; p < parts; p += blockDim.x) s += sumsq[(size_t)irow * parts + p];
    const float total = block_sum(s, scratch, blockDim.x / KVA_WAVE);
    const float rinv = 1.f / (float)sqrt((double)total / (double)width + (double)eps);
    const bf16_t *x = scaled + (size_t)irow * width;
    bf16_t *y = out + (size_t)orow * width;
    for (int i = threadIdx.x; i < width; i += blockDim.x) y[i] = from_float<bf16_t>(to_float(x[i]) * rinv);
}

extern "C" int kva_normed_rows_finish(void *out, const void *scaled, const float *sumsq, int parts,
                                      int out_rows, const int *row_idx, int width, float eps,
                                      hipStream_t stream) {
    KVA_REQUIRE(out_rows >= 0 && width > 0 && parts > 0, "normed_rows_finish: bad sizes");
    if (out_rows == 0) return KVA_OK;
    hipLaunchKernelGGL(normed_rows_finish_kernel, dim3(out_rows), dim3(256), 0, stream, (bf16_t *)out,
                       (const bf16_t *)scaled, sumsq, parts, row_idx, width, eps);
    KVA_CHECK_LAUNCH("normed_rows_finish");
    return KVA_OK;
}
