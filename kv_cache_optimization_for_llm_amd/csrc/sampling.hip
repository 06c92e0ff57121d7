// Token sampling on the device: greedy argmax (lowest id wins ties) and temperature sampling by
// inverse CDF with a counter-based uniform, both over optionally penalised fp32 logits.
//
// Same algorithm as the reference's sampling kernels (base/src/kernels.cu:489-835) and their
// numpy mirror (python/sampling_reference.py:26-89):
//   * a row is cut into `chunks` contiguous chunks of ceil(V / chunks) tokens;
//   * pass 1: per chunk, the best (value, index) - ties to the lower index;
//   * pass 2: per row, reduce the chunk results -> argmax token and row maximum;
//   * temperature rows only: per chunk sum of w_i = exp((l_i - max) / T); then a walk over the
//     chunk prefix sums picks the chunk holding target = u * sum(w), and a walk over 256
//     contiguous spans of that chunk picks the token: first i whose cumulative weight exceeds
//     the target, which is searchsorted(cdf, target, side="right") of the flat CDF.
//   * u = counter_uniform(seed, key, step): splitmix64 finaliser, top 24 bits, in [0, 1).
//   * repetition penalty on tokens marked in the request's mask row: l > 0 ? l / p : l * p.
#include "common.h"
#include <math.h>

#define SAMPLE_THREADS 256

__device__ inline void argmax_merge(float &bv, int &bi, float v, int i) {
    if (v > bv || (v == bv && i < bi)) {
        bv = v;
        bi = i;
    }
}

__device__ inline float penalised_logit(const float *row, const unsigned char *mask, int token,
                                        float penalty) {
    const float l = row[token];
    if (mask != nullptr && mask[token] != 0) return l > 0.f ? l / penalty : l * penalty;
    return l;
}

__host__ __device__ inline float counter_uniform(unsigned int seed, unsigned int key,
                                                 unsigned int step) {
    unsigned long long z = ((unsigned long long)key << 32) ^ (unsigned long long)step;
    z ^= (unsigned long long)seed * 0x9E3779B97F4A7C15ULL;
    z += 0x9E3779B97F4A7C15ULL;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
    z = z ^ (z >> 31);
    return (float)(z >> 40) * (1.0f / 16777216.0f);
}

__device__ inline const unsigned char *mask_row(const unsigned char *penalty_mask,
                                                const int *row_seat, int row, int vocab) {
    if (penalty_mask == nullptr || row_seat == nullptr) return nullptr;
    const int seat = row_seat[row];
    return seat < 0 ? nullptr : penalty_mask + (size_t)seat * vocab;
}

// grid (chunks, rows)
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_chunk_max_kernel(const float *__restrict__ logits, int vocab, int chunk_tokens,
                        const unsigned char *__restrict__ penalty_mask,
                        const int *__restrict__ row_seat, float penalty,
                        float *__restrict__ part_val, int *__restrict__ part_idx) {
    __shared__ float wv[SAMPLE_THREADS / KVA_WAVE];
    __shared__ int wi[SAMPLE_THREADS / KVA_WAVE];
    const int row = blockIdx.y, chunk = blockIdx.x, chunks = gridDim.x;
    const int begin = chunk * chunk_tokens;
    const int end = min(begin + chunk_tokens, vocab);
    const float *rl = logits + (size_t)row * vocab;
    const unsigned char *mk = mask_row(penalty_mask, row_seat, row, vocab);
    float bv = -INFINITY;
    int bi = vocab;
    for (int t = begin + threadIdx.x; t < end; t += SAMPLE_THREADS)
        argmax_merge(bv, bi, penalised_logit(rl, mk, t, penalty), t);
    for (int off = KVA_WAVE / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, KVA_WAVE);
        const int oi = __shfl_xor(bi, off, KVA_WAVE);
        argmax_merge(bv, bi, ov, oi);
    }
    const int lane = threadIdx.x % KVA_WAVE, wave = threadIdx.x / KVA_WAVE;
    if (lane == 0) {
        wv[wave] = bv;
        wi[wave] = bi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < SAMPLE_THREADS / KVA_WAVE; ++w) argmax_merge(wv[0], wi[0], wv[w], wi[w]);
        part_val[row * chunks + chunk] = wv[0];
        part_idx[row * chunks + chunk] = wi[0];
    }
}

// grid (rows), one wavefront
__global__ void __launch_bounds__(KVA_WAVE)
sample_row_max_kernel(const float *__restrict__ part_val, const int *__restrict__ part_idx,
                      int chunks, int vocab, float *__restrict__ row_max, int *__restrict__ out_tokens) {
    const int row = blockIdx.x;
    float bv = -INFINITY;
    int bi = vocab;
    for (int c = threadIdx.x; c < chunks; c += KVA_WAVE)
        argmax_merge(bv, bi, part_val[row * chunks + c], part_idx[row * chunks + c]);
    for (int off = KVA_WAVE / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, KVA_WAVE);
        const int oi = __shfl_xor(bi, off, KVA_WAVE);
        argmax_merge(bv, bi, ov, oi);
    }
    if (threadIdx.x == 0) {
        row_max[row] = bv;
        out_tokens[row] = bi;
    }
}

// grid (chunks, rows); rows with inv_temperature <= 0 are greedy and skipped
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_chunk_expsum_kernel(const float *__restrict__ logits, int vocab, int chunk_tokens,
                           const unsigned char *__restrict__ penalty_mask,
                           const int *__restrict__ row_seat, float penalty,
                           const float *__restrict__ row_max, const float *__restrict__ inv_temperature,
                           float *__restrict__ part_sum) {
    __shared__ float ws[SAMPLE_THREADS / KVA_WAVE];
    const int row = blockIdx.y, chunk = blockIdx.x, chunks = gridDim.x;
    const float inv_t = inv_temperature[row];
    if (!(inv_t > 0.f)) return;
    const int begin = chunk * chunk_tokens;
    const int end = min(begin + chunk_tokens, vocab);
    const float *rl = logits + (size_t)row * vocab;
    const unsigned char *mk = mask_row(penalty_mask, row_seat, row, vocab);
    const float m = row_max[row];
    float sum = 0.f;
    for (int t = begin + threadIdx.x; t < end; t += SAMPLE_THREADS)
        sum += expf((penalised_logit(rl, mk, t, penalty) - m) * inv_t);
    sum = wave_sum(sum);
    const int lane = threadIdx.x % KVA_WAVE, wave = threadIdx.x / KVA_WAVE;
    if (lane == 0) ws[wave] = sum;
    __syncthreads();
    if (threadIdx.x == 0) {
        float total = 0.f;
        for (int w = 0; w < SAMPLE_THREADS / KVA_WAVE; ++w) total += ws[w];
        part_sum[row * chunks + chunk] = total;
    }
}

// grid (rows)
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_finalize_kernel(const float *__restrict__ logits, int vocab, int chunk_tokens, int chunks,
                       const unsigned char *__restrict__ penalty_mask,
                       const int *__restrict__ row_seat, float penalty,
                       const float *__restrict__ row_max, const float *__restrict__ inv_temperature,
                       const float *__restrict__ part_sum, unsigned int seed,
                       const unsigned int *__restrict__ rng_key, const unsigned int *__restrict__ rng_step,
                       int *__restrict__ out_tokens) {
    __shared__ float thread_prefix[SAMPLE_THREADS];
    __shared__ int s_chunk;
    __shared__ float s_target;
    __shared__ int s_result;
    const int row = blockIdx.x;
    const float inv_t = inv_temperature[row];
    if (!(inv_t > 0.f)) return;  // greedy row: sample_row_max_kernel already wrote the argmax

    if (threadIdx.x == 0) {
        const float *ps = part_sum + (size_t)row * chunks;
        float total = 0.f;
        for (int c = 0; c < chunks; ++c) total += ps[c];
        const float u = counter_uniform(seed, rng_key[row], rng_step[row]);
        const float target = u * total;
        int chunk = chunks - 1;
        float before = 0.f, run = 0.f;
        bool found = false;
        for (int c = 0; c < chunks; ++c) {
            const float prev = run;
            run += ps[c];
            if (!found && target < run) {
                chunk = c;
                before = prev;
                found = true;
            }
        }
        if (!found) {
            // target landed on the total through rounding: take the last non-empty chunk
            float r2 = 0.f;
            for (int c = 0; c < chunks; ++c) {
                if (ps[c] > 0.f) {
                    chunk = c;
                    before = r2;
                }
                r2 += ps[c];
            }
        }
        s_chunk = chunk;
        s_target = target - before;
        s_result = min(chunk * chunk_tokens + chunk_tokens - 1, vocab - 1);
    }
    __syncthreads();

    const int begin_c = s_chunk * chunk_tokens;
    const int end_c = min(begin_c + chunk_tokens, vocab);
    const int span = (chunk_tokens + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
    const float *rl = logits + (size_t)row * vocab;
    const unsigned char *mk = mask_row(penalty_mask, row_seat, row, vocab);
    const float m = row_max[row];
    const int begin = begin_c + (int)threadIdx.x * span;
    float local = 0.f;
    for (int t = begin; t < min(begin + span, end_c); ++t)
        local += expf((penalised_logit(rl, mk, t, penalty) - m) * inv_t);
    thread_prefix[threadIdx.x] = local;
    __syncthreads();
    if (threadIdx.x == 0)
        for (int t = 1; t < SAMPLE_THREADS; ++t) thread_prefix[t] += thread_prefix[t - 1];
    __syncthreads();
    const float before = threadIdx.x == 0 ? 0.f : thread_prefix[threadIdx.x - 1];
    if (begin < end_c && s_target >= before && s_target < thread_prefix[threadIdx.x]) {
        float acc = before;
        for (int t = begin; t < min(begin + span, end_c); ++t) {
            acc += expf((penalised_logit(rl, mk, t, penalty) - m) * inv_t);
            if (s_target < acc) {
                s_result = t;
                break;
            }
        }
    }
    __syncthreads();
    if (threadIdx.x == 0) out_tokens[row] = s_result;
}

// workspace: rows * chunks * 3 + rows floats
extern "C" long long kva_sample_workspace_bytes(int rows, int chunks) {
    return ((long long)rows * chunks * 3 + rows) * 4;
}

extern "C" int kva_sample(int *out_tokens, const float *logits, int rows, int vocab, int chunks,
                          const unsigned char *penalty_mask, const int *row_seat, float penalty,
                          const float *inv_temperature, unsigned int seed,
                          const unsigned int *rng_key, const unsigned int *rng_step, int any_sampled,
                          void *workspace, hipStream_t stream) {
    KVA_REQUIRE(rows >= 0 && vocab > 0, "sample: bad sizes rows=%d vocab=%d", rows, vocab);
    KVA_REQUIRE(chunks >= 1 && chunks <= 1024, "sample: chunk count %d out of range", chunks);
    KVA_REQUIRE(rows <= 65535, "sample: at most 65535 rows per call");
    KVA_REQUIRE(penalty > 0.f, "sample: repetition penalty must be positive");
    KVA_REQUIRE(!any_sampled || (inv_temperature && rng_key && rng_step),
                "sample: temperature rows need inv_temperature, rng_key and rng_step");
    if (rows == 0) return KVA_OK;
    const int chunk_tokens = (vocab + chunks - 1) / chunks;
    float *part_val = (float *)workspace;
    int *part_idx = (int *)(part_val + (size_t)rows * chunks);
    float *part_sum = (float *)(part_idx + (size_t)rows * chunks);
    float *row_max = part_sum + (size_t)rows * chunks;
    hipLaunchKernelGGL(sample_chunk_max_kernel, dim3(chunks, rows), dim3(SAMPLE_THREADS), 0, stream,
                       logits, vocab, chunk_tokens, penalty_mask, row_seat, penalty, part_val, part_idx);
    hipLaunchKernelGGL(sample_row_max_kernel, dim3(rows), dim3(KVA_WAVE), 0, stream, part_val,
                       part_idx, chunks, vocab, row_max, out_tokens);
    if (any_sampled) {
        hipLaunchKernelGGL(sample_chunk_expsum_kernel, dim3(chunks, rows), dim3(SAMPLE_THREADS), 0,
                           stream, logits, vocab, chunk_tokens, penalty_mask, row_seat, penalty,
                           row_max, inv_temperature, part_sum);
        hipLaunchKernelGGL(sample_finalize_kernel, dim3(rows), dim3(SAMPLE_THREADS), 0, stream,
                           logits, vocab, chunk_tokens, chunks, penalty_mask, row_seat, penalty,
                           row_max, inv_temperature, part_sum, seed, rng_key, rng_step, out_tokens);
    }
    KVA_CHECK_LAUNCH("sample");
    return KVA_OK;
}

// mask[seat[i]][token[i]] = 1
__global__ void mark_tokens_kernel(unsigned char *__restrict__ mask, const int *__restrict__ seats,
                                   const int *__restrict__ tokens, int n, int vocab) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int seat = seats[i], tok = tokens[i];
    if (seat >= 0 && tok >= 0 && tok < vocab) mask[(size_t)seat * vocab + tok] = 1;
}

extern "C" int kva_mark_tokens(unsigned char *mask, const int *seats, const int *tokens, int n,
                               int vocab, hipStream_t stream) {
    KVA_REQUIRE(n >= 0 && vocab > 0, "mark_tokens: bad sizes");
    if (n == 0) return KVA_OK;
    hipLaunchKernelGGL(mark_tokens_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, mask, seats,
                       tokens, n, vocab);
    KVA_CHECK_LAUNCH("mark_tokens");
    return KVA_OK;
}
