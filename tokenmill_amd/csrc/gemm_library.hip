// C[M, N] = A[M, K] * W[N, K]^T (+ bias) through hipBLASLt, for the large products of a prompt
// step, where the reference also calls a library (F.linear, reference src/infer/model/layers.py:144-164).
//
// What this file adds to the library call is a cache: the descriptors and the algorithm the
// library's heuristic picks for a (shape, strides, types, epilogue) are made once and kept, so that
// a call after the first costs one hipblasLtMatmul launch. A prompt step makes about a hundred of
// these calls; setting each of them up again costs more host time than the step's kernels take.
//
// hipBLASLt is column-major. Row-major C = A W^T is the column-major product C^T = W A^T:
// first operand W as [K, N] with leading dimension ldw, transposed; second A as [K, M] with
// leading dimension lda; result [N, M] with leading dimension ldc. The bias has one entry per row
// of that result, i.e. per output feature, and is added to the 32-bit sum before rounding.
#include <hipblaslt/hipblaslt.h>
#include <hipblaslt/hipblaslt-ext.hpp>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <unordered_map>
#include <utility>
#include <vector>

#include "common.h"
#include "api.h"

namespace {

struct PlanKey {
    int M, N, K, lda, ldw, ldc, bias_dtype, out_f32, device;
    int tuned;      // 1: the plan of callers that ask for timed algorithms; the others never see what timing chose
    bool operator==(const PlanKey& o) const {
        return M == o.M && N == o.N && K == o.K && lda == o.lda && ldw == o.ldw && ldc == o.ldc &&
               bias_dtype == o.bias_dtype && out_f32 == o.out_f32 && device == o.device && tuned == o.tuned;
    }
};

struct PlanKeyHash {
    size_t operator()(const PlanKey& k) const {
        size_t h = 1469598103934665603ull;
        for (int v : {k.M, k.N, k.K, k.lda, k.ldw, k.ldc, k.bias_dtype, k.out_f32, k.device, k.tuned})
            h = (h ^ (size_t)(uint32_t)v) * 1099511628211ull;
        return h;
    }
};

struct Plan {
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t w = nullptr, a = nullptr, c = nullptr;
    hipblasLtMatmulAlgo_t algo;
    size_t workspace = 0;
    bool ok = false;
    int calls = 0;          // eager calls of this shape with the matrix of its first call so far
    const void* first_w = nullptr;
    bool timed = false;     // its candidates have been timed (or timing was tried)
    // The candidates the heuristic gave when the plan was made, kept until they are timed. They are
    // asked for once: a second, longer query for a product the library has already answered a short
    // one for gave the same first choice followed by far slower candidates than the one long query.
    hipblasLtMatmulHeuristicResult_t* found = nullptr;
    int n_found = 0;
};

struct Library {
    std::mutex lock;
    std::unordered_map<int, hipblasLtHandle_t> handles;          // one per device
    std::unordered_map<PlanKey, Plan, PlanKeyHash> plans;
};

Library& lib() {
    static Library* l = new Library();      // never destroyed: the runtime may be gone at exit
    return *l;
}

// Timing is the caller's choice, call by call (TmTune, api.h): how many of the heuristic's candidates are
// timed for a shape before the fastest is kept (0 or 1: keep the heuristic's first choice untimed), and
// at which call of a shape that happens. Steps of a serving run come in hundreds of different numbers
// of rows, most of them once: timing costs tens of milliseconds per shape, so only a shape that comes
// back is timed (or one whose caller says that it will be replayed, by asking for the first call).
// Beyond the heuristic's candidates, a shape that is timed at its first call (its caller is about to
// replay it from a graph) can also have every algorithm the library holds for the operand types tried:
// one quick run each, the fastest few timed like the heuristic's candidates. About a second a shape.
// Plans made for callers that time live beside the plans of callers that do not (PlanKey::tuned): an
// engine that keeps the library's first choice gets the same algorithm whoever else runs in the process.
// With TOKENMILL_TUNE_LOG set in the environment every timing is printed to stderr.
constexpr int SHORT_LIST = 12;

struct Operands {
    const void *A, *W, *bias;
    void *C, *workspace;
    size_t workspace_bytes;
    hipStream_t stream;
};

// What the timed runs evict the caches with: larger than the last-level cache, so that every timed
// product finds its matrix in HBM, as it does inside a step (a decode step reads about a gigabyte of
// other matrices between two uses of this one). Made when the first shape is timed, never freed.
constexpr size_t FLUSH_BYTES = (size_t)768 << 20;
std::unordered_map<int, void*> g_flush;                      // per device; nullptr: could not be allocated

void* flush_buffer(int device) {
    auto it = g_flush.find(device);
    if (it != g_flush.end()) return it->second;
    void* buf = nullptr;
    if (hipMalloc(&buf, FLUSH_BYTES) != hipSuccess) {
        (void)hipGetLastError();
        buf = nullptr;
    }
    g_flush[device] = buf;
    return buf;
}

// Mean time of a few runs of one algorithm on the caller's own operands (the result is the same
// whichever algorithm wrote it last, up to rounding); with `flush` each run follows a flush of the
// caches. Negative if it fails.
float time_algo(hipblasLtHandle_t handle, const Plan& p, const hipblasLtMatmulAlgo_t& algo, const Operands& op,
                void* flush, bool quick = false) {
    const float one = 1.f, zero = 0.f;
    hipEvent_t t0, t1;
    if (hipEventCreate(&t0) != hipSuccess) return -1.f;
    if (hipEventCreate(&t1) != hipSuccess) {
        hipEventDestroy(t0);
        return -1.f;
    }
    const int WARM = quick ? 1 : 2, TIMED = quick ? (flush ? 1 : 3) : (flush ? 5 : 20);
    float total = 0.f;
    bool ok = true;
    if (!flush) {       // operands in cache: the runs follow each other without a gap, one time for all of them
        for (int i = 0; i < WARM + TIMED && ok; ++i) {
            if (i == WARM) hipEventRecord(t0, op.stream);
            ok = hipblasLtMatmul(handle, p.desc, &one, op.W, p.w, op.A, p.a, &zero, op.C, p.c, op.C, p.c, &algo,
                                 op.workspace, op.workspace_bytes, op.stream) == HIPBLAS_STATUS_SUCCESS;
        }
        hipEventRecord(t1, op.stream);
        ok = ok && hipEventSynchronize(t1) == hipSuccess && hipEventElapsedTime(&total, t0, t1) == hipSuccess;
    } else {            // each run after a flush, timed alone
        for (int i = 0; i < WARM + TIMED && ok; ++i) {
            ok = hipMemsetAsync(flush, i, FLUSH_BYTES, op.stream) == hipSuccess;
            hipEventRecord(t0, op.stream);
            ok = ok && hipblasLtMatmul(handle, p.desc, &one, op.W, p.w, op.A, p.a, &zero, op.C, p.c, op.C, p.c, &algo,
                                       op.workspace, op.workspace_bytes, op.stream) == HIPBLAS_STATUS_SUCCESS;
            hipEventRecord(t1, op.stream);
            float ms = 0.f;
            ok = ok && hipEventSynchronize(t1) == hipSuccess && hipEventElapsedTime(&ms, t0, t1) == hipSuccess;
            if (i >= WARM) total += ms;
        }
    }
    hipEventDestroy(t0);
    hipEventDestroy(t1);
    return ok ? total / TIMED : -1.f;
}

constexpr int MAX_CANDIDATES = 32;

// The library's candidates for a plan's product, best first by its own heuristic.
int candidates(hipblasLtHandle_t handle, const Plan& p, size_t workspace_bytes, int want,
               hipblasLtMatmulHeuristicResult_t (&found)[MAX_CANDIDATES]) {
    hipblasLtMatmulPreference_t pref = nullptr;
    if (hipblasLtMatmulPreferenceCreate(&pref) != HIPBLAS_STATUS_SUCCESS) return 0;
    const uint64_t max_ws = workspace_bytes;
    hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &max_ws, sizeof(max_ws));
    if (want > MAX_CANDIDATES) want = MAX_CANDIDATES;
    int n_found = 0;
    const hipblasStatus_t st =
        hipblasLtMatmulAlgoGetHeuristic(handle, p.desc, p.w, p.a, p.c, p.c, pref, want, found, &n_found);
    hipblasLtMatmulPreferenceDestroy(pref);
    return st == HIPBLAS_STATUS_SUCCESS ? n_found : 0;
}

// Descriptors, layouts and the heuristic's first valid choice: no run, no wait.
bool make_plan(hipblasLtHandle_t handle, const PlanKey& k, size_t workspace_bytes, const TmTune& tune, Plan& p) {
    const hipDataType in_t = HIP_R_16BF, out_t = k.out_f32 ? HIP_R_32F : HIP_R_16BF;
    if (hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) != HIPBLAS_STATUS_SUCCESS) return false;
    const hipblasOperation_t tr = HIPBLAS_OP_T, no = HIPBLAS_OP_N;
    hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &tr, sizeof(tr));
    hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &no, sizeof(no));
    if (k.bias_dtype != TM_NONE) {
        const hipblasLtEpilogue_t epi = HIPBLASLT_EPILOGUE_BIAS;
        const hipDataType bias_t = k.bias_dtype == TM_F32 ? HIP_R_32F : HIP_R_16BF;
        hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_EPILOGUE, &epi, sizeof(epi));
        hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, &bias_t, sizeof(bias_t));
    }
    if (hipblasLtMatrixLayoutCreate(&p.w, in_t, k.K, k.N, k.ldw) != HIPBLAS_STATUS_SUCCESS ||
        hipblasLtMatrixLayoutCreate(&p.a, in_t, k.K, k.M, k.lda) != HIPBLAS_STATUS_SUCCESS ||
        hipblasLtMatrixLayoutCreate(&p.c, out_t, k.N, k.M, k.ldc) != HIPBLAS_STATUS_SUCCESS)
        return false;
    // Several candidates also when none will be timed: the heuristic's first choice can ask for more
    // workspace than the preference allows (a split of K with one partial result per split, seen at
    // 8,192 and 16,384 rows), and the first that fits is taken.
    constexpr int UNTIMED_CANDIDATES = 8;
    hipblasLtMatmulHeuristicResult_t found[MAX_CANDIDATES];
    const int n_found = candidates(handle, p, workspace_bytes,
                                   tune.candidates > UNTIMED_CANDIDATES ? tune.candidates : UNTIMED_CANDIDATES, found);
    for (int i = 0; i < n_found && !p.ok; ++i)
        if (found[i].state == HIPBLAS_STATUS_SUCCESS && found[i].workspaceSize <= workspace_bytes) {
            p.algo = found[i].algo;
            p.workspace = found[i].workspaceSize;
            p.ok = true;
        }
    if (p.ok && n_found > 1 && tune.candidates > 1) {
        p.found = new hipblasLtMatmulHeuristicResult_t[n_found];
        for (int i = 0; i < n_found; ++i) p.found[i] = found[i];
        p.n_found = n_found;
    }
    return p.ok;
}

// Every algorithm the library holds for the plan's types that takes this product, short-listed by one
// quick run each: the fastest SHORT_LIST are appended to `pool`.
void add_every(hipblasLtHandle_t handle, const PlanKey& k, const Plan& p, const Operands& op, void* flush,
               std::vector<hipblasLtMatmulHeuristicResult_t>& pool) {
    const hipDataType in_t = HIP_R_16BF, out_t = k.out_f32 ? HIP_R_32F : HIP_R_16BF;
    std::vector<hipblasLtMatmulHeuristicResult_t> all;
    if (hipblaslt_ext::getAllAlgos(handle, hipblaslt_ext::GemmType::HIPBLASLT_GEMM, HIPBLAS_OP_T, HIPBLAS_OP_N, in_t, in_t,
                                   out_t, out_t, HIPBLAS_COMPUTE_32F, all) != HIPBLAS_STATUS_SUCCESS)
        return;
    const float one = 1.f, zero = 0.f;
    std::vector<std::pair<float, size_t>> quick;
    for (size_t i = 0; i < all.size(); ++i) {
        size_t need = 0;
        if (hipblaslt_ext::matmulIsAlgoSupported(handle, p.desc, &one, p.w, p.a, &zero, p.c, p.c, all[i].algo, need) !=
                HIPBLAS_STATUS_SUCCESS || need > op.workspace_bytes)
            continue;
        all[i].workspaceSize = need;
        all[i].state = HIPBLAS_STATUS_SUCCESS;
        const float ms = time_algo(handle, p, all[i].algo, op, flush, true);
        if (ms > 0.f) quick.push_back({ms, i});
    }
    std::sort(quick.begin(), quick.end());
    for (size_t i = 0; i < quick.size() && i < (size_t)SHORT_LIST; ++i) pool.push_back(all[quick[i].second]);
    if (getenv("TOKENMILL_TUNE_LOG"))
        fprintf(stderr, "[tokenmill_amd] M=%d N=%d K=%d: %zu algorithms, %zu take the product\n", k.M, k.N, k.K, all.size(),
                quick.size());
}

// max |x - y| and max |x| over n values, as the bits of non-negative floats (which order like integers).
template <typename T>
__global__ void max_difference_kernel(const T* __restrict__ x, const T* __restrict__ y, size_t n, unsigned* __restrict__ out) {
    float diff = 0.f, top = 0.f;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        const float a = Elem<T>::load(x + i), b = Elem<T>::load(y + i);
        const float d = fabsf(a - b);
        diff = (d == d) ? fmaxf(diff, d) : INFINITY;       // a NaN on either side counts as a difference
        top = fmaxf(top, fabsf(a));
    }
    for (int o = TM_WAVE / 2; o > 0; o >>= 1) {
        diff = fmaxf(diff, __shfl_xor(diff, o, TM_WAVE));
        top = fmaxf(top, __shfl_xor(top, o, TM_WAVE));
    }
    if (threadIdx.x % TM_WAVE == 0) {
        atomicMax(out, __float_as_uint(diff));
        atomicMax(out + 1, __float_as_uint(top));
    }
}

// Does `algo` give what the heuristic's first choice `first` gives, up to the rounding of the sums?
// An algorithm that the heuristic did not name is only kept if it does. Needs a dense result (ldc == N).
bool same_result(hipblasLtHandle_t handle, const PlanKey& k, const Plan& p, const Operands& op,
                 const hipblasLtMatmulAlgo_t& first, const hipblasLtMatmulAlgo_t& algo) {
    if (k.ldc != k.N) return false;
    const size_t n = (size_t)k.M * k.N, bytes = n * (k.out_f32 ? 4 : 2);
    void* other = nullptr;
    unsigned* found = nullptr;
    if (hipMalloc(&other, bytes) != hipSuccess || hipMalloc((void**)&found, 2 * sizeof(unsigned)) != hipSuccess) {
        (void)hipGetLastError();
        if (other) hipFree(other);
        return false;
    }
    const float one = 1.f, zero = 0.f;
    bool ok = hipMemsetAsync(found, 0, 2 * sizeof(unsigned), op.stream) == hipSuccess;
    ok = ok && hipblasLtMatmul(handle, p.desc, &one, op.W, p.w, op.A, p.a, &zero, other, p.c, other, p.c, &first,
                               op.workspace, op.workspace_bytes, op.stream) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && hipblasLtMatmul(handle, p.desc, &one, op.W, p.w, op.A, p.a, &zero, op.C, p.c, op.C, p.c, &algo,
                               op.workspace, op.workspace_bytes, op.stream) == HIPBLAS_STATUS_SUCCESS;
    if (ok) {
        if (k.out_f32)
            max_difference_kernel<float><<<256, 256, 0, op.stream>>>((const float*)other, (const float*)op.C, n, found);
        else
            max_difference_kernel<bf16_t><<<256, 256, 0, op.stream>>>((const bf16_t*)other, (const bf16_t*)op.C, n, found);
    }
    unsigned host[2] = {0, 0};
    ok = ok && hipMemcpyAsync(host, found, sizeof(host), hipMemcpyDeviceToHost, op.stream) == hipSuccess &&
         hipStreamSynchronize(op.stream) == hipSuccess;
    hipFree(other);
    hipFree(found);
    if (!ok) return false;
    float diff, top;
    memcpy(&diff, &host[0], 4);
    memcpy(&top, &host[1], 4);
    // two orders of a 32-bit sum, rounded once to the output type: a few units of the largest value's last place
    const float allowed = top * (k.out_f32 ? 1.f / 4096 : 1.f / 32);
    return diff <= allowed;
}

// Times up to tune.candidates of the library's candidates on the caller's own operands and keeps
// the fastest. Needs the stream to run now: never called while it is being captured into a graph.
void time_plan(hipblasLtHandle_t handle, const PlanKey& k, const Operands& op, const TmTune& tune, Plan& p) {
    std::vector<hipblasLtMatmulHeuristicResult_t> pool;
    if (p.found) {
        const int n = p.n_found < tune.candidates ? p.n_found : tune.candidates;
        pool.assign(p.found, p.found + n);
        delete[] p.found;
        p.found = nullptr;
        p.n_found = 0;
    } else {                                // the plan was made before timing was switched on
        hipblasLtMatmulHeuristicResult_t found[MAX_CANDIDATES];
        const int n = candidates(handle, p, op.workspace_bytes, tune.candidates, found);
        pool.assign(found, found + n);
    }
    const size_t named = pool.size();       // the candidates before this index are the heuristic's
    if (k.bias_dtype != TM_NONE)
        hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &op.bias, sizeof(op.bias));
    // Flushed where the matrix is the larger part of what the product reads and writes (few
    // rows: the matrix comes from HBM in a real step); with many rows the activations, which the
    // kernel before has just written, are the larger part, and those are in cache in a step too.
    const size_t out_size = k.out_f32 ? 4 : 2;
    const bool cold = (size_t)k.N * k.K * 2 > (size_t)k.M * k.K * 2 + (size_t)k.M * k.N * out_size;
    void* flush = cold ? flush_buffer(k.device) : nullptr;
    if (tune.every && tune.after <= 1) add_every(handle, k, p, op, flush, pool);
    if (pool.size() < 2) return;
    // The heuristic's first choice stays unless another candidate beats it clearly (timings of a
    // few runs scatter by some percent).
    std::vector<std::pair<float, size_t>> timed;
    float first_ms = -1.f;
    int first = -1;
    for (size_t i = 0; i < pool.size(); ++i) {
        if (pool[i].state != HIPBLAS_STATUS_SUCCESS || pool[i].workspaceSize > op.workspace_bytes) continue;
        const float ms = time_algo(handle, p, pool[i].algo, op, flush);
        if (getenv("TOKENMILL_TUNE_LOG")) fprintf(stderr, " %.4f", ms);
        if (ms < 0.f) continue;
        if (first < 0) {
            first = (int)i;
            first_ms = ms;
        }
        timed.push_back({ms, i});
    }
    if (first < 0) return;                  // nothing could be timed: the plan stays as it is
    std::stable_sort(timed.begin(), timed.end());
    int best = first;
    float best_ms = first_ms;
    for (const auto& cand : timed) {
        if (cand.first > 0.93f * first_ms) break;
        // an algorithm the heuristic did not name must give the first choice's result
        if (cand.second >= named && !same_result(handle, k, p, op, pool[first].algo, pool[cand.second].algo)) {
            fprintf(stderr, "[tokenmill_amd] M=%d N=%d K=%d: a faster algorithm gave another result and is left out\n",
                    k.M, k.N, k.K);
            continue;
        }
        best = (int)cand.second;
        best_ms = cand.first;
        break;
    }
    if (getenv("TOKENMILL_TUNE_LOG"))
        fprintf(stderr, "[tokenmill_amd] timed M=%d N=%d K=%d %s: %zu candidates (%zu the heuristic's), first %.4f ms, best %.4f ms, kept #%d\n",
                k.M, k.N, k.K, cold ? "cold" : "warm", pool.size(), named, first_ms, best_ms, best);
    p.algo = pool[best].algo;
    p.workspace = pool[best].workspaceSize;
}

}  // namespace

// bias_dtype: TM_NONE (no bias), TM_BF16 or TM_F32. out_f32: C is float32 (else bfloat16).
// workspace: device memory the library may use, the same for every call on a stream.
// tune: null or candidates < 2 keeps the library's first choice. Else up to `candidates` of the library's
// candidates are timed on this call's own operands when the shape is called the `after`-th time with the
// matrix of its first call outside a graph capture, and the fastest is kept (after = 1: at its first call,
// for a caller that is about to capture the step into a graph and replay it); every != 0: a shape timed at
// its first call also tries every algorithm the library holds for the operand types (about a second a shape).
// Returns TM_ERR_ARG for arguments it does not take, TM_ERR_UNSUPPORTED when the library has no
// algorithm for the product (the caller then uses another path), TM_ERR_LAUNCH when the call fails.
extern "C" int tm_gemm_library(const void* A, int lda, const void* W, int ldw, const void* bias, int bias_dtype,
                               void* C, int ldc, int out_f32, int M, int N, int K, void* workspace,
                               size_t workspace_bytes, const TmTune* tune_or_null, hipStream_t stream) {
    if (M <= 0 || N <= 0 || K <= 0 || lda < K || ldw < K || ldc < N || !A || !W || !C ||
        (bias_dtype != TM_NONE && bias_dtype != TM_BF16 && bias_dtype != TM_F32) || ((bias_dtype != TM_NONE) != (bias != nullptr)))
        return TM_ERR_ARG;
    TmTune tune{0, 3, 0};
    if (tune_or_null) tune = *tune_or_null;
    if (tune.candidates < 0 || tune.candidates > MAX_CANDIDATES || (tune.every && tune.candidates < 2)) return TM_ERR_ARG;
    if (tune.after < 1) tune.after = 1;
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess) return TM_ERR_LAUNCH;
    const PlanKey key{M, N, K, lda, ldw, ldc, bias_dtype, out_f32 ? 1 : 0, device, tune.candidates > 1 ? 1 : 0};
    Library& l = lib();
    hipblasLtHandle_t handle;
    Plan plan;
    {
        std::lock_guard<std::mutex> guard(l.lock);
        auto h = l.handles.find(device);
        if (h == l.handles.end()) {
            hipblasLtHandle_t made;
            if (hipblasLtCreate(&made) != HIPBLAS_STATUS_SUCCESS) return TM_ERR_LAUNCH;
            h = l.handles.emplace(device, made).first;
        }
        handle = h->second;
        auto it = l.plans.find(key);
        if (it == l.plans.end()) {
            Plan made;
            make_plan(handle, key, workspace_bytes, tune, made);           // a failed plan is kept too: asked once
            it = l.plans.emplace(key, made).first;
        }
        Plan& kept = it->second;
        if (kept.ok && !kept.timed && tune.candidates > 1) {
            hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
            hipStreamIsCapturing(stream, &capturing);
            // calls with the matrix of the first call are counted: every layer of a step brings the
            // shape once with its own matrix, and a step is not a shape that came back
            if (!kept.first_w) kept.first_w = W;
            if (capturing == hipStreamCaptureStatusNone && W == kept.first_w && ++kept.calls >= tune.after) {
                kept.timed = true;
                const Operands op{A, W, bias, C, workspace, workspace_bytes, stream};
                time_plan(handle, key, op, tune, kept);
            }
        }
        plan = kept;
    }
    if (!plan.ok || plan.workspace > workspace_bytes) return TM_ERR_UNSUPPORTED;
    if (bias_dtype != TM_NONE)          // the descriptor is shared by every call of this shape: calls on one device are serial
        hipblasLtMatmulDescSetAttribute(plan.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bias, sizeof(bias));
    const float one = 1.f, zero = 0.f;
    const hipblasStatus_t st = hipblasLtMatmul(handle, plan.desc, &one, W, plan.w, A, plan.a, &zero, C, plan.c, C, plan.c,
                                               &plan.algo, workspace, workspace_bytes, stream);
    return st == HIPBLAS_STATUS_SUCCESS ? TM_OK : TM_ERR_LAUNCH;
}
