// Y[M,N] = X[M,K] * W[N,K]^T for many rows (prompt portions, large decode batches): the vendor
// GEMM library, hipBLASLt, called directly.
//
// Stands where the reference calls cublasGemmEx (base/src/engine.cu:1040-1117).  bf16 operands,
// fp32 accumulation, bf16 or fp32 result.  What this file adds to calling the library through a
// tensor framework is only that everything that depends on the shape alone is looked up once:
// the descriptors, the layouts and the algorithm the library's heuristic picks are kept per
// (device, M, N, K, strides, result type), so a call costs a hash lookup and the launch, a few
// microseconds of host time instead of some 17.  Steps that are not replayed from a graph (every
// prompt portion) are bound by exactly that host time when they are short.
//
// Row-major Y = X W^T is, in the library's column-major terms, Y' [N x M] = op_T(W') op_N(X')
// with W' = [K x N] (ld K), X' = [K x M] (ld ldx), Y' = [N x M] (ld ldy).
//
// Tuning (kva_gemm_vendor_tune): the heuristic's choice is often not the library's fastest kernel
// for a shape.  The tuning call runs every algorithm the library has for the problem type that
// supports the shape on the caller's operands (weights of several layers in turn, so that they
// come from memory as in a real pass and not from a cache), times them with events and keeps the
// fastest for later calls of that shape.  It takes seconds per shape and waits for the device, so
// it belongs to start-up, outside any graph capture.
//
// One workspace of 32 MiB per device, allocated at the first call on it (kva_gemm_vendor_init
// does that call ahead of any graph capture) and never freed; products on different streams of
// one device would share it, the engine runs them on one stream.
#include "common.h"
#include <hipblaslt/hipblaslt.h>
#include <hipblaslt/hipblaslt-ext.hpp>
#include <algorithm>
#include <mutex>
#include <unordered_map>
#include <utility>
#include <vector>

namespace {

constexpr int kMaxDevices = 16;
constexpr size_t kWorkspaceBytes = 32u << 20;

struct Plan {
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t a = nullptr, b = nullptr, c = nullptr;
    hipblasLtMatmulAlgo_t algo;
    bool found = false;
};

struct Key {
    int dev, m, n, k, ldx, ldy, f32;
    bool operator==(const Key &o) const {
        return dev == o.dev && m == o.m && n == o.n && k == o.k && ldx == o.ldx && ldy == o.ldy && f32 == o.f32;
    }
};
struct KeyHash {
    size_t operator()(const Key &x) const {
        size_t h = 1469598103934665603ull;
        for (int v : {x.dev, x.m, x.n, x.k, x.ldx, x.ldy, x.f32}) h = (h ^ (size_t)(unsigned)v) * 1099511628211ull;
        return h;
    }
};

std::mutex g_mutex;
hipblasLtHandle_t g_handle[kMaxDevices];
void *g_workspace[kMaxDevices];
std::unordered_map<Key, Plan, KeyHash> g_plans;
// Algorithms that timing has kept, per (device, N, K, result type) with the row count they were
// timed at.  A row count that has not been timed itself takes the algorithm of the nearest timed
// one above it (at most twice as many rows) when the library says it supports the exact shape:
// decode batches of 33..64 requests then share what was found for 64.
struct TunedKey {
    int dev, n, k, f32;
    bool operator==(const TunedKey &o) const { return dev == o.dev && n == o.n && k == o.k && f32 == o.f32; }
};
struct TunedHash {
    size_t operator()(const TunedKey &x) const {
        size_t h = 1469598103934665603ull;
        for (int v : {x.dev, x.n, x.k, x.f32}) h = (h ^ (size_t)(unsigned)v) * 1099511628211ull;
        return h;
    }
};
std::unordered_map<TunedKey, std::vector<std::pair<int, hipblasLtMatmulAlgo_t>>, TunedHash> g_tuned;

// every algorithm of the library for bf16 x bf16 -> bf16 [0] / fp32 [1], asked for once per device
std::vector<hipblasLtMatmulHeuristicResult_t> g_all_algos[kMaxDevices][2];

// The handle and the workspace of a device; 0 on success.
int device_state(int dev) {
    if (g_handle[dev] != nullptr) return KVA_OK;
    if (hipblasLtCreate(&g_handle[dev]) != HIPBLAS_STATUS_SUCCESS) {
        g_handle[dev] = nullptr;
        kva_set_error("gemm_vendor: the GEMM library could not be initialised on device %d", dev);
        return KVA_ERR_LAUNCH;
    }
    if (hipMalloc(&g_workspace[dev], kWorkspaceBytes) != hipSuccess) {
        (void)hipGetLastError();
        hipblasLtDestroy(g_handle[dev]);
        g_handle[dev] = nullptr;
        kva_set_error("gemm_vendor: no memory for the library's workspace (%zu bytes)", kWorkspaceBytes);
        return KVA_ERR_LAUNCH;
    }
    return KVA_OK;
}

bool make_plan(int dev, const Key &key, Plan &p) {
    const hipblasOperation_t op_t = HIPBLAS_OP_T, op_n = HIPBLAS_OP_N;
    const hipDataType out_type = key.f32 ? HIP_R_32F : HIP_R_16BF;
    bool ok = hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &op_t, sizeof(op_t)) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &op_n, sizeof(op_n)) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && hipblasLtMatrixLayoutCreate(&p.a, HIP_R_16BF, key.k, key.n, key.k) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && hipblasLtMatrixLayoutCreate(&p.b, HIP_R_16BF, key.k, key.m, key.ldx) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && hipblasLtMatrixLayoutCreate(&p.c, out_type, key.n, key.m, key.ldy) == HIPBLAS_STATUS_SUCCESS;
    if (ok) {
        auto it = g_tuned.find(TunedKey{dev, key.n, key.k, key.f32});
        if (it != g_tuned.end()) {
            int best_rows = 0;
            const hipblasLtMatmulAlgo_t *best = nullptr;
            for (const auto &entry : it->second)
                if (entry.first >= key.m && entry.first <= 2 * key.m && (best == nullptr || entry.first < best_rows)) {
                    best_rows = entry.first;
                    best = &entry.second;
                }
            if (best != nullptr) {
                const float alpha = 1.f, beta = 0.f;
                size_t need = 0;
                hipblasLtMatmulAlgo_t algo = *best;
                if (hipblaslt_ext::matmulIsAlgoSupported(g_handle[dev], p.desc, &alpha, p.a, p.b, &beta, p.c, p.c, algo,
                                                         need) == HIPBLAS_STATUS_SUCCESS && need <= kWorkspaceBytes) {
                    p.algo = algo;
                    p.found = true;
                    return true;
                }
            }
        }
    }
    hipblasLtMatmulPreference_t pref = nullptr;
    ok = ok && hipblasLtMatmulPreferenceCreate(&pref) == HIPBLAS_STATUS_SUCCESS;
    if (ok) {
        const uint64_t ws = kWorkspaceBytes;
        ok = hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ws, sizeof(ws)) ==
             HIPBLAS_STATUS_SUCCESS;
    }
    if (ok) {
        // the first of the heuristic's choices that is usable with this workspace
        constexpr int kAsk = 8;
        hipblasLtMatmulHeuristicResult_t result[kAsk];
        int returned = 0;
        const hipblasStatus_t st = hipblasLtMatmulAlgoGetHeuristic(g_handle[dev], p.desc, p.a, p.b, p.c, p.c, pref, kAsk,
                                                                   result, &returned);
        for (int i = 0; st == HIPBLAS_STATUS_SUCCESS && i < returned && i < kAsk && !p.found; ++i) {
            if (result[i].state == HIPBLAS_STATUS_SUCCESS && result[i].workspaceSize <= kWorkspaceBytes) {
                p.algo = result[i].algo;
                p.found = true;
            }
        }
    }
    if (pref) hipblasLtMatmulPreferenceDestroy(pref);
    return ok;
}

// Mean time of one product in microseconds over `reps` runs after one untimed run, the weights
// taken in turn from `Ws`; negative when the library refuses the algorithm or a call fails.
float time_algo(const Plan &p, hipblasLtMatmulAlgo_t &algo, hipblasLtHandle_t handle, void *workspace, void *Y,
                const void *X, const void *const *Ws, int n_w, int reps, hipEvent_t t0, hipEvent_t t1,
                hipStream_t stream) {
    const float alpha = 1.f, beta = 0.f;
    bool ok = true;
    for (int run = -1; run < reps && ok; ++run) {
        if (run == 0) ok = hipEventRecord(t0, stream) == hipSuccess;
        const void *W = Ws[(run + 1) % n_w];
        ok = ok && hipblasLtMatmul(handle, p.desc, &alpha, W, p.a, X, p.b, &beta, Y, p.c, Y, p.c, &algo, workspace,
                                   kWorkspaceBytes, stream) == HIPBLAS_STATUS_SUCCESS;
    }
    float ms = 0.f;
    ok = ok && hipEventRecord(t1, stream) == hipSuccess && hipEventSynchronize(t1) == hipSuccess &&
         hipEventElapsedTime(&ms, t0, t1) == hipSuccess;
    if (!ok) {
        (void)hipGetLastError();
        return -1.f;
    }
    return ms * 1000.f / (float)reps;
}

}  // namespace

// Finds the library's fastest algorithm for Y[M,N] = X[M,K] W[N,K]^T by running all that support
// the shape, and keeps it for later kva_gemm_vendor calls of the same shape, strides and result
// type.  `Ws` are n_w weight matrices of that shape (host array of device pointers) used in turn.
// first_us / best_us: time of the heuristic's choice and of the one kept; tried: algorithms run.
// Y is overwritten with products of the last weights used.  Waits for the device.
extern "C" int kva_gemm_vendor_tune(void *Y, const void *X, const void *const *Ws, int n_w, int M, int N, int K,
                                    int ldx, int ldy, int out_f32, hipStream_t stream, float *first_us,
                                    float *best_us, int *tried) {
    KVA_REQUIRE(M >= 1 && N >= 1 && K >= 1 && ldx >= K && ldy >= N && n_w >= 1 && Ws != nullptr,
                "gemm_vendor_tune: bad sizes M=%d N=%d K=%d ldx=%d ldy=%d weights=%d", M, N, K, ldx, ldy, n_w);
    int dev = 0;
    KVA_REQUIRE(hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < kMaxDevices, "gemm_vendor_tune: no current device");
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    KVA_REQUIRE(hipStreamIsCapturing(stream, &capturing) == hipSuccess && capturing == hipStreamCaptureStatusNone,
                "gemm_vendor_tune: the stream is being captured into a graph; tuning waits for the device");
    std::lock_guard<std::mutex> lock(g_mutex);
    const int st = device_state(dev);
    if (st != KVA_OK) return st;
    const Key key{dev, M, N, K, ldx, ldy, out_f32 ? 1 : 0};
    auto it = g_plans.find(key);
    if (it == g_plans.end()) {
        Plan fresh;
        if (!make_plan(dev, key, fresh)) {
            kva_set_error("gemm_vendor_tune: the library refused the description of M=%d N=%d K=%d", M, N, K);
            return KVA_ERR_LAUNCH;
        }
        it = g_plans.emplace(key, fresh).first;
    }
    Plan &p = it->second;
    auto &all = g_all_algos[dev][key.f32];
    if (all.empty()) {
        const hipDataType out_type = key.f32 ? HIP_R_32F : HIP_R_16BF;
        if (hipblaslt_ext::getAllAlgos(g_handle[dev], hipblaslt_ext::GemmType::HIPBLASLT_GEMM, HIPBLAS_OP_T, HIPBLAS_OP_N,
                                       HIP_R_16BF, HIP_R_16BF, out_type, out_type, HIPBLAS_COMPUTE_32F,
                                       all) != HIPBLAS_STATUS_SUCCESS)
            all.clear();
    }
    hipEvent_t t0 = nullptr, t1 = nullptr;
    if (hipEventCreate(&t0) != hipSuccess || hipEventCreate(&t1) != hipSuccess) {
        (void)hipGetLastError();
        if (t0) (void)hipEventDestroy(t0);
        kva_set_error("gemm_vendor_tune: no events");
        return KVA_ERR_LAUNCH;
    }
    constexpr int kQuickReps = 3, kFinalReps = 24, kFinalists = 6;
    constexpr float kMargin = 0.97f;            // what timing noise alone gives is not worth another rounding
    const float alpha = 1.f, beta = 0.f;
    std::vector<std::pair<float, int>> timed;
    for (size_t i = 0; i < all.size(); ++i) {
        size_t need = 0;
        if (hipblaslt_ext::matmulIsAlgoSupported(g_handle[dev], p.desc, &alpha, p.a, p.b, &beta, p.c, p.c, all[i].algo,
                                                 need) != HIPBLAS_STATUS_SUCCESS || need > kWorkspaceBytes)
            continue;
        const float us = time_algo(p, all[i].algo, g_handle[dev], g_workspace[dev], Y, X, Ws, n_w, kQuickReps, t0, t1, stream);
        if (us > 0.f) timed.emplace_back(us, (int)i);
    }
    std::sort(timed.begin(), timed.end());
    float first = -1.f, best = -1.f;
    if (p.found) first = best = time_algo(p, p.algo, g_handle[dev], g_workspace[dev], Y, X, Ws, n_w, kFinalReps, t0, t1, stream);
    for (int j = 0; j < kFinalists && j < (int)timed.size(); ++j) {
        hipblasLtMatmulAlgo_t &algo = all[timed[j].second].algo;
        const float us = time_algo(p, algo, g_handle[dev], g_workspace[dev], Y, X, Ws, n_w, kFinalReps, t0, t1, stream);
        if (us > 0.f && (best < 0.f || us < best * kMargin)) {
            best = us;
            p.algo = algo;
            p.found = true;
        }
    }
    (void)hipEventDestroy(t0);
    (void)hipEventDestroy(t1);
    if (p.found) {
        auto &list = g_tuned[TunedKey{dev, N, K, key.f32}];
        bool replaced = false;
        for (auto &entry : list)
            if (entry.first == M) {
                entry.second = p.algo;
                replaced = true;
            }
        if (!replaced) list.emplace_back(M, p.algo);
    }
    if (first_us) *first_us = first;
    if (best_us) *best_us = best;
    if (tried) *tried = (int)timed.size();
    return KVA_OK;
}

// Forgets what is kept for a shape: its next call asks the library's heuristic again.
extern "C" int kva_gemm_vendor_forget(int M, int N, int K, int ldx, int ldy, int out_f32) {
    int dev = 0;
    KVA_REQUIRE(hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < kMaxDevices, "gemm_vendor_forget: no current device");
    std::lock_guard<std::mutex> lock(g_mutex);
    auto tuned = g_tuned.find(TunedKey{dev, N, K, out_f32 ? 1 : 0});
    if (tuned != g_tuned.end()) {
        auto &list = tuned->second;
        list.erase(std::remove_if(list.begin(), list.end(),
                                  [M](const std::pair<int, hipblasLtMatmulAlgo_t> &e) { return e.first == M; }),
                   list.end());
    }
    auto it = g_plans.find(Key{dev, M, N, K, ldx, ldy, out_f32 ? 1 : 0});
    if (it != g_plans.end()) {
        Plan &p = it->second;
        if (p.a) hipblasLtMatrixLayoutDestroy(p.a);
        if (p.b) hipblasLtMatrixLayoutDestroy(p.b);
        if (p.c) hipblasLtMatrixLayoutDestroy(p.c);
        if (p.desc) hipblasLtMatmulDescDestroy(p.desc);
        g_plans.erase(it);
    }
    return KVA_OK;
}

// Makes the library handle and the workspace of the current device (no effect when they exist).
extern "C" int kva_gemm_vendor_init() {
    int dev = 0;
    KVA_REQUIRE(hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < kMaxDevices, "gemm_vendor: no current device");
    std::lock_guard<std::mutex> lock(g_mutex);
    return device_state(dev);
}

// Returns KVA_OK, an error, or 1 when the library offers no algorithm for the shape (nothing was
// launched then and the caller takes another path).
extern "C" int kva_gemm_vendor(void *Y, const void *X, const void *W, int M, int N, int K, int ldx, int ldy,
                               int out_f32, hipStream_t stream) {
    KVA_REQUIRE(M >= 1 && N >= 1 && K >= 1 && ldx >= K && ldy >= N, "gemm_vendor: bad sizes M=%d N=%d K=%d ldx=%d ldy=%d",
                M, N, K, ldx, ldy);
    int dev = 0;
    KVA_REQUIRE(hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < kMaxDevices, "gemm_vendor: no current device");
    Plan plan;
    hipblasLtHandle_t handle;
    void *workspace;
    {
        std::lock_guard<std::mutex> lock(g_mutex);
        const int st = device_state(dev);
        if (st != KVA_OK) return st;
        const Key key{dev, M, N, K, ldx, ldy, out_f32 ? 1 : 0};
        auto it = g_plans.find(key);
        if (it == g_plans.end()) {
            Plan fresh;
            if (!make_plan(dev, key, fresh)) {
                kva_set_error("gemm_vendor: the library refused the description of M=%d N=%d K=%d", M, N, K);
                return KVA_ERR_LAUNCH;
            }
            it = g_plans.emplace(key, fresh).first;
        }
        plan = it->second;
        handle = g_handle[dev];
        workspace = g_workspace[dev];
    }
    if (!plan.found) return 1;
    const float alpha = 1.f, beta = 0.f;
    const hipblasStatus_t st = hipblasLtMatmul(handle, plan.desc, &alpha, W, plan.a, X, plan.b, &beta, Y, plan.c, Y,
                                               plan.c, &plan.algo, workspace, kWorkspaceBytes, stream);
    if (st != HIPBLAS_STATUS_SUCCESS) {
        kva_set_error("gemm_vendor: the library failed on M=%d N=%d K=%d (status %d)", M, N, K, (int)st);
        return KVA_ERR_LAUNCH;
    }
    return KVA_OK;
}
