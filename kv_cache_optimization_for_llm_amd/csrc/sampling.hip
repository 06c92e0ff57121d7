// Token sampling on the device: greedy argmax (lowest id wins ties) and temperature sampling by
// inverse CDF with a counter-based uniform, both over optionally penalised fp32 logits.
//
// What is computed is what the reference's sampling kernels compute (base/src/kernels.cu:489-835;
// numpy mirror python/sampling_reference.py:26-89): the token of a temperature row is the first i
// whose cumulative weight w_0 + ... + w_i, w_i = exp((l_i - max l) / T), exceeds u * sum(w) - the
// flat CDF's searchsorted(cdf, target, side="right") - with u = counter_uniform(seed, key, step);
// a greedy row takes the largest logit, the lowest id among equals; tokens marked in the request's
// mask row are penalised first (l > 0 ? l / p : l * p).
//
// How: two launches, and the logits are read once.
//   1. sample_scan_kernel, one workgroup per (chunk of a row, row): every thread keeps an online
//      (maximum, sum of exp((l - maximum) / T)) pair and its best (value, id) over the tokens it
//      reads; the workgroup joins them and leaves one record per chunk.
//   2. sample_pick_kernel, one wavefront per row: joins the chunk records (row maximum, argmax),
//      rescales the chunk sums to the row maximum, finds the chunk that holds the target by a
//      wavefront prefix scan, reads that one chunk again (a thousand tokens), scans the lanes'
//      spans the same way, and the lane that holds the target walks its few tokens.  The chosen
//      token is also marked in the request's mask row when there is one.
#include "common.h"
#include <math.h>

#define SAMPLE_THREADS 256
#define SCAN_IN_FLIGHT 8
#define SAMPLE_MAX_CHUNKS 1024
#define PICK_CHUNKS_PER_LANE (SAMPLE_MAX_CHUNKS / KVA_WAVE)
#define KVA_NO_TOKEN (-1)       // what a row gets whose logits name no token

namespace {

struct Best {
    float value;
    int index;
};

// the larger value; the lower index among equal values
__device__ inline Best better(Best a, Best b) {
    return (b.value > a.value || (b.value == a.value && b.index < a.index)) ? b : a;
}

__device__ inline Best wave_best(Best x) {
#pragma unroll
    for (int off = KVA_WAVE / 2; off > 0; off >>= 1) {
        Best o;
        o.value = __shfl_xor(x.value, off, KVA_WAVE);
        o.index = __shfl_xor(x.index, off, KVA_WAVE);
        x = better(x, o);
    }
    return x;
}

// Inclusive prefix sum over the 64 lanes, lane order (six shift-and-add steps in the vector ALU).
__device__ inline float wave_prefix_sum(float v) {
    const int lane = threadIdx.x % KVA_WAVE;
#pragma unroll
    for (int off = 1; off < KVA_WAVE; off <<= 1) {
        const float below = __shfl_up(v, off, KVA_WAVE);
        if (lane >= off) v += below;
    }
    return v;
}

// Index of the lowest lane whose flag is set, or -1.
__device__ inline int first_lane(bool flag) {
    const unsigned long long votes = __ballot(flag);
    return votes == 0 ? -1 : __ffsll((long long)votes) - 1;
}

__device__ inline float penalised(float l, const unsigned char *mask, int token, float penalty) {
    if (mask != nullptr && mask[token] != 0) return l > 0.f ? l / penalty : l * penalty;
    return l;
}

__device__ inline const unsigned char *mask_row(const unsigned char *penalty_mask, const int *row_seat,
                                                int row, int vocab) {
    if (penalty_mask == nullptr || row_seat == nullptr) return nullptr;
    const int seat = row_seat[row];
    return seat < 0 ? nullptr : penalty_mask + (size_t)seat * vocab;
}

// exp((l - top) / T); a logit that is -inf or NaN weighs nothing (as in Online::add)
__device__ inline float token_weight(float l, float top, float inv_t) {
    return l > -INFINITY ? expf((l - top) * inv_t) : 0.f;
}

// Running softmax denominator: sum of exp((l - m) * inv_t) over what has been added, m their maximum.
struct Online {
    float m, s;
    __device__ inline void add(float l, float inv_t) {
        if (!(l > -INFINITY)) return;        // -inf and NaN weigh nothing
        if (l > m) {
            s = s * expf((m - l) * inv_t) + 1.f;
            m = l;
        } else {
            s += expf((l - m) * inv_t);
        }
    }
    __device__ inline void join(Online o, float inv_t) {
        if (o.m == -INFINITY) return;
        if (m == -INFINITY) {
            *this = o;
            return;
        }
        const float top = fmaxf(m, o.m);
        s = s * expf((m - top) * inv_t) + o.s * expf((o.m - top) * inv_t);
        m = top;
    }
};

} // namespace

__host__ __device__ inline float counter_uniform(unsigned int seed, unsigned int key, unsigned int step) {
    unsigned long long z = ((unsigned long long)key << 32) ^ (unsigned long long)step;
    z ^= (unsigned long long)seed * 0x9E3779B97F4A7C15ULL;
    z += 0x9E3779B97F4A7C15ULL;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
    z = z ^ (z >> 31);
    return (float)(z >> 40) * (1.0f / 16777216.0f);
}

// One record per (row, chunk): the chunk's best (value, id), and for temperature rows the chunk's
// maximum and its sum of exp((l - maximum) / T).
struct ChunkRecord {
    float best_value;
    int best_index;
    float top;
    float sum;
};

// grid (chunks, rows)
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_scan_kernel(const float *__restrict__ logits, int vocab, int chunk_tokens,
                   const unsigned char *__restrict__ penalty_mask, const int *__restrict__ row_seat,
                   float penalty, const float *__restrict__ inv_temperature,
                   ChunkRecord *__restrict__ records) {
    __shared__ Best wave_b[SAMPLE_THREADS / KVA_WAVE];
    __shared__ Online wave_o[SAMPLE_THREADS / KVA_WAVE];
    const int row = blockIdx.y, chunk = blockIdx.x, chunks = gridDim.x;
    const int begin = chunk * chunk_tokens;
    const int end = min(begin + chunk_tokens, vocab);
    const float *rl = logits + (size_t)row * vocab;
    const unsigned char *mk = mask_row(penalty_mask, row_seat, row, vocab);
    const float inv_t = inv_temperature != nullptr ? inv_temperature[row] : 0.f;
    const bool sampled = inv_t > 0.f;
    Best b{-INFINITY, vocab};
    Online o{-INFINITY, 0.f};
    // A thread's tokens in turns of SCAN_IN_FLIGHT, every load of a turn asked for before the first
    // is used (a plain loop over a thread's four or eight tokens is a trip to memory each).
    for (int base = begin + threadIdx.x; base < end; base += SCAN_IN_FLIGHT * SAMPLE_THREADS) {
        float l[SCAN_IN_FLIGHT];
        unsigned char marked[SCAN_IN_FLIGHT];
#pragma unroll
        for (int j = 0; j < SCAN_IN_FLIGHT; ++j) {
            const int t = base + j * SAMPLE_THREADS;
            l[j] = rl[t < end ? t : end - 1];
            marked[j] = mk != nullptr ? mk[t < end ? t : end - 1] : (unsigned char)0;
        }
#pragma unroll
        for (int j = 0; j < SCAN_IN_FLIGHT; ++j) {
            const int t = base + j * SAMPLE_THREADS;
            if (t >= end) break;
            const float v = marked[j] != 0 ? (l[j] > 0.f ? l[j] / penalty : l[j] * penalty) : l[j];
            b = better(b, Best{v, t});
            if (sampled) o.add(v, inv_t);
        }
    }
    b = wave_best(b);
    if (sampled) {
#pragma unroll
        for (int off = KVA_WAVE / 2; off > 0; off >>= 1) {
            Online other;
            other.m = __shfl_xor(o.m, off, KVA_WAVE);
            other.s = __shfl_xor(o.s, off, KVA_WAVE);
            o.join(other, inv_t);
        }
    }
    const int lane = threadIdx.x % KVA_WAVE, wave = threadIdx.x / KVA_WAVE;
    if (lane == 0) {
        wave_b[wave] = b;
        wave_o[wave] = o;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
#pragma unroll
        for (int w = 1; w < SAMPLE_THREADS / KVA_WAVE; ++w) {
            b = better(b, wave_b[w]);
            if (sampled) o.join(wave_o[w], inv_t);
        }
        records[(size_t)row * chunks + chunk] = ChunkRecord{b.value, b.index, o.m, o.s};
    }
}

// grid (rows), one wavefront
__global__ void __launch_bounds__(KVA_WAVE)
sample_pick_kernel(const float *__restrict__ logits, int vocab, int chunk_tokens, int chunks,
                   const unsigned char *penalty_mask, const int *__restrict__ row_seat,
                   float penalty, const float *__restrict__ inv_temperature,
                   const ChunkRecord *__restrict__ records, unsigned int seed,
                   const unsigned int *__restrict__ rng_key, const unsigned int *__restrict__ rng_step,
                   unsigned char *mark_mask /* may be penalty_mask */, const int *__restrict__ mark_seat,
                   int *__restrict__ out_tokens, int *__restrict__ host_tokens) {
    const int row = blockIdx.x, lane = threadIdx.x;
    const ChunkRecord *rec = records + (size_t)row * chunks;
    // this lane's chunks: a contiguous run, so that lane order is chunk order
    const int per_lane = (chunks + KVA_WAVE - 1) / KVA_WAVE;
    const int c0 = lane * per_lane, c1 = min(c0 + per_lane, chunks);
    Best b{-INFINITY, vocab};
    for (int c = c0; c < c1; ++c) b = better(b, Best{rec[c].best_value, rec[c].best_index});
    b = wave_best(b);
    int token = b.index;                    // the greedy choice; the row maximum is b.value
    bool bad_row = !(b.value > -INFINITY);  // NaN compares false too
    const float inv_t = inv_temperature != nullptr ? inv_temperature[row] : 0.f;
    if (inv_t > 0.f && !bad_row) {
        const float top = b.value;
        // chunk sums brought to the row maximum, summed per lane, scanned over the lanes
        float weight[PICK_CHUNKS_PER_LANE];
        float mine = 0.f;
#pragma unroll
        for (int i = 0; i < PICK_CHUNKS_PER_LANE; ++i) {
            const int c = c0 + i;
            weight[i] = (i < per_lane && c < c1 && rec[c].sum > 0.f) ? rec[c].sum * expf((rec[c].top - top) * inv_t) : 0.f;
            mine += weight[i];
        }
        const float upto = wave_prefix_sum(mine);
        const float total = __shfl(upto, KVA_WAVE - 1, KVA_WAVE);
        bad_row = !(total > 0.f) || total == INFINITY;
        const float target = counter_uniform(seed, rng_key[row], rng_step[row]) * total;
        // the first lane whose chunks reach past the target holds the chunk
        int owner = first_lane(target < upto);
        int chunk = -1;
        float before = 0.f;
        if (lane == owner) {
            float run = upto - mine, last_before = run;
            int last_chunk = c0;
#pragma unroll
            for (int i = 0; i < PICK_CHUNKS_PER_LANE; ++i) {
                if (chunk < 0 && i < per_lane && c0 + i < c1) {
                    if (target < run + weight[i]) {
                        chunk = c0 + i;
                        before = run;
                    } else {
                        last_before = run;
                        last_chunk = c0 + i;
                        run += weight[i];
                    }
                }
            }
            if (chunk < 0) {                 // rounding between the lane's own sum and the scan's
                chunk = last_chunk;
                before = last_before;
            }
        }
        if (owner < 0) {
            // the target landed on the total through rounding: the last token of the last chunk
            // that weighs anything (before = -inf puts the target past every span below)
            int last = -1;
#pragma unroll
            for (int i = 0; i < PICK_CHUNKS_PER_LANE; ++i)
                if (i < per_lane && c0 + i < c1 && weight[i] > 0.f) last = c0 + i;
#pragma unroll
            for (int off = KVA_WAVE / 2; off > 0; off >>= 1) last = max(last, __shfl_xor(last, off, KVA_WAVE));
            chunk = last < 0 ? chunks - 1 : last;
            before = -INFINITY;
        } else {
            chunk = __shfl(chunk, owner, KVA_WAVE);
            before = __shfl(before, owner, KVA_WAVE);
        }
        // inside the chunk: lanes own contiguous spans; the same scan finds the lane, which walks
        const int begin = chunk * chunk_tokens, end = min(begin + chunk_tokens, vocab);
        const int span = (end - begin + KVA_WAVE - 1) / KVA_WAVE;
        const int t0 = min(begin + lane * span, end), t1 = min(t0 + span, end);
        const float *rl = logits + (size_t)row * vocab;
        const unsigned char *mk = mask_row(penalty_mask, row_seat, row, vocab);
        const float inner = target - before;
        float local = 0.f;
        for (int t = t0; t < t1; ++t) local += token_weight(penalised(rl[t], mk, t, penalty), top, inv_t);
        const float reach = wave_prefix_sum(local);
        owner = first_lane(t0 < t1 && inner < reach);
        int found = end - 1;                 // past every span's reach (rounding): the chunk's last token
        if (lane == owner) {
            float acc = reach - local;
            found = t1 - 1;
            for (int t = t0; t < t1; ++t) {
                acc += token_weight(penalised(rl[t], mk, t, penalty), top, inv_t);
                if (inner < acc) {
                    found = t;
                    break;
                }
            }
        }
        token = __shfl(found, owner < 0 ? 0 : owner, KVA_WAVE);
    }
    // A row without a finite best logit (all NaN, all -inf) has no token to name, greedy or sampled,
    // and neither has a temperature row whose weights do not add up to a positive finite total.
    // Such a row gets KVA_NO_TOKEN (-1): the host sees it and ends the request with an error, and
    // the next step's lookup of this buffer on the device, which may already be queued, takes
    // token 0 for any negative value it finds (a row past the table's end would be a memory fault).
    if (bad_row || token < 0 || token >= vocab) token = KVA_NO_TOKEN;
    if (lane == 0) {
        out_tokens[row] = token;
        if (host_tokens != nullptr) host_tokens[row] = token;      // pinned host memory, mapped for the device
        if (mark_mask != nullptr && mark_seat != nullptr) {
            const int seat = mark_seat[row];
            if (seat >= 0 && token >= 0 && token < vocab) mark_mask[(size_t)seat * vocab + token] = 1;
        }
    }
}

// workspace: one record per (row, chunk)
extern "C" long long kva_sample_workspace_bytes(int rows, int chunks) {
    return (long long)rows * chunks * (long long)sizeof(ChunkRecord);
}

// out_tokens[row] = the sampled (inv_temperature[row] > 0) or the best token of logits[row, :].
// penalty_mask [seats, vocab] with row_seat[row] (-1: none) says which logits are penalised;
// mark_mask / mark_seat (may be the same mask, -1: none) get the chosen token marked afterwards.
// Whether a kernel may write to this host memory: pinned and mapped for the current device.
extern "C" int kva_host_memory_is_mapped(void *host) {
    void *dev = nullptr;
    if (host == nullptr || hipHostGetDevicePointer(&dev, host, 0) != hipSuccess) {
        (void)hipGetLastError();                                    // the query's failure is an answer, not an error to keep
        return 0;
    }
    return dev != nullptr ? 1 : 0;
}

// host_tokens (optional): pinned host memory (hipHostMalloc, torch's pin_memory) with room for a token
// per row; the kernel that chooses the tokens writes them there as well, which saves the copy
// that would otherwise follow it on the stream.  Refused unless the runtime says the memory is
// mapped for the device.
extern "C" int kva_sample(int *out_tokens, const float *logits, int rows, int vocab, int chunks,
                          const unsigned char *penalty_mask, const int *row_seat, float penalty,
                          const float *inv_temperature, unsigned int seed,
                          const unsigned int *rng_key, const unsigned int *rng_step, int any_sampled,
                          void *workspace, unsigned char *mark_mask, const int *mark_seat,
                          int *host_tokens, hipStream_t stream) {
    int *host_mapped = nullptr;
    if (host_tokens != nullptr) {
        void *dev = nullptr;
        const hipError_t e = hipHostGetDevicePointer(&dev, host_tokens, 0);
        KVA_REQUIRE(e == hipSuccess && dev != nullptr, "sample: host_tokens is not pinned host memory mapped for the device (%s)",
                    hipGetErrorString(e));
        host_mapped = (int *)dev;
    }
    KVA_REQUIRE(rows >= 0 && vocab > 0, "sample: bad sizes rows=%d vocab=%d", rows, vocab);
    KVA_REQUIRE(chunks >= 1 && chunks <= SAMPLE_MAX_CHUNKS, "sample: chunk count %d is not in 1..%d", chunks,
                SAMPLE_MAX_CHUNKS);
    KVA_REQUIRE(rows <= 65535, "sample: at most 65535 rows per call");
    KVA_REQUIRE(penalty > 0.f, "sample: repetition penalty must be positive");
    KVA_REQUIRE(!any_sampled || (inv_temperature && rng_key && rng_step),
                "sample: temperature rows need inv_temperature, rng_key and rng_step");
    KVA_REQUIRE(workspace != nullptr || rows == 0, "sample: a workspace of kva_sample_workspace_bytes is needed");
    if (rows == 0) return KVA_OK;
    const int chunk_tokens = (vocab + chunks - 1) / chunks;
    ChunkRecord *records = (ChunkRecord *)workspace;
    const float *inv_t = any_sampled ? inv_temperature : nullptr;
    hipLaunchKernelGGL(sample_scan_kernel, dim3(chunks, rows), dim3(SAMPLE_THREADS), 0, stream, logits,
                       vocab, chunk_tokens, penalty_mask, row_seat, penalty, inv_t, records);
    hipLaunchKernelGGL(sample_pick_kernel, dim3(rows), dim3(KVA_WAVE), 0, stream, logits, vocab,
                       chunk_tokens, chunks, penalty_mask, row_seat, penalty, inv_t, records, seed, rng_key,
                       rng_step, mark_mask, mark_seat, out_tokens, host_mapped);
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
