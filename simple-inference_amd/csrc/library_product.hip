// Y[M, N] = X[M, K] * W[N, K]^T in bfloat16 with float accumulation by the vendor's BLAS library (hipBLASLt),
// called directly: the products of steps of many tokens, where the reference's go to its vendor's library
// (``ops/attention.py:128-130``, ``ops/mlp.py:117,128``).  Called through a tensor library the same product
// costs the host some 18 microseconds a call, most of it a search for the algorithm; here the descriptors and the
// algorithm of a shape are looked up once and kept, and a call costs a few.
//
// Row-major Y = X W^T is, in the library's column-major terms, Y^T[N, M] = A^T B with A = W seen as [K, N]
// (leading dimension K, transposed) and B = X seen as [K, M].
#include <hip/hip_runtime.h>
#include <hipblaslt/hipblaslt.h>
#include <stdint.h>

#include <unordered_map>

#define SIA_EXPORT extern "C" __attribute__((visibility("default")))

namespace {

constexpr size_t WORKSPACE_BYTES = 32u << 20;
constexpr int TRIED = 24;        // candidates of the library that are timed for a shape of few rows
constexpr int TIMED_RUNS = 8;
constexpr float CLEARLY = 0.96f;
constexpr size_t SWEEP_BYTES = 512u << 20;  // twice the memory-side cache
constexpr int TRY_OUT_ROWS = 256;  // up to here a product streams its weights once and the candidates differ widely

struct Plan {
    hipblasLtMatmulDesc_t op = nullptr;
    hipblasLtMatrixLayout_t a = nullptr, b = nullptr, c = nullptr;
    hipblasLtMatmulAlgo_t algo;
    size_t workspace = 0;
    bool ok = false;
    bool tried_out = false;  // the algorithm was chosen by timing the candidates
};

struct State {
    bool try_out = false;  // shapes met now will recur: time the candidates
    void* sweep = nullptr;  // while try_out: memory whose filling sweeps the caches between timed runs
    hipblasLtHandle_t handle = nullptr;
    void* workspace = nullptr;
    std::unordered_map<uint64_t, Plan> plans;
};

State* g_state[16] = {};

State* state_of_current_device() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) return nullptr;
    return g_state[dev];
}

// With `try_out` the library's candidates for the shape are run on the operands of the call that asks (whose
// result the call itself then overwrites) and the fastest is kept; else its first candidate is taken.
void release(Plan& p) {
    if (p.a) hipblasLtMatrixLayoutDestroy(p.a);
    if (p.b) hipblasLtMatrixLayoutDestroy(p.b);
    if (p.c) hipblasLtMatrixLayoutDestroy(p.c);
    if (p.op) hipblasLtMatmulDescDestroy(p.op);
    p = Plan{};
}

bool make_plan(State& st, Plan& p, int M, int N, int K, bool out_float, bool try_out, const void* X, const void* W,
               void* Y, hipStream_t stream) {
    const hipDataType out_type = out_float ? HIP_R_32F : HIP_R_16BF;
    if (hipblasLtMatmulDescCreate(&p.op, HIPBLAS_COMPUTE_32F, HIP_R_32F) != HIPBLAS_STATUS_SUCCESS) return false;
    const hipblasOperation_t trans = HIPBLAS_OP_T, none = HIPBLAS_OP_N;
    if (hipblasLtMatmulDescSetAttribute(p.op, HIPBLASLT_MATMUL_DESC_TRANSA, &trans, sizeof(trans)) != HIPBLAS_STATUS_SUCCESS ||
        hipblasLtMatmulDescSetAttribute(p.op, HIPBLASLT_MATMUL_DESC_TRANSB, &none, sizeof(none)) != HIPBLAS_STATUS_SUCCESS)
        return false;
    if (hipblasLtMatrixLayoutCreate(&p.a, HIP_R_16BF, K, N, K) != HIPBLAS_STATUS_SUCCESS ||
        hipblasLtMatrixLayoutCreate(&p.b, HIP_R_16BF, K, M, K) != HIPBLAS_STATUS_SUCCESS ||
        hipblasLtMatrixLayoutCreate(&p.c, out_type, N, M, N) != HIPBLAS_STATUS_SUCCESS)
        return false;
    hipblasLtMatmulPreference_t pref = nullptr;
    if (hipblasLtMatmulPreferenceCreate(&pref) != HIPBLAS_STATUS_SUCCESS) return false;
    const size_t limit = WORKSPACE_BYTES;
    hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &limit, sizeof(limit));
    hipblasLtMatmulHeuristicResult_t found[TRIED];
    int n_found = 0;
    const int wanted = try_out ? TRIED : 1;
    const hipblasStatus_t status =
        hipblasLtMatmulAlgoGetHeuristic(st.handle, p.op, p.a, p.b, p.c, p.c, pref, wanted, found, &n_found);
    hipblasLtMatmulPreferenceDestroy(pref);
    if (status != HIPBLAS_STATUS_SUCCESS || n_found < 1) return false;
    int best = -1;
    float best_ms = 0.f;
    hipEvent_t t0 = nullptr, t1 = nullptr;
    const bool timed = try_out && n_found > 1 && hipEventCreate(&t0) == hipSuccess && hipEventCreate(&t1) == hipSuccess;
    const float one = 1.f, zero = 0.f;
    for (int i = 0; i < n_found; ++i) {
        if (found[i].state != HIPBLAS_STATUS_SUCCESS || found[i].workspaceSize > WORKSPACE_BYTES) continue;
        if (!timed) {
            best = i;
            break;
        }
        // The real operands, the real stream: one run to load the code, then TIMED_RUNS runs, each after the caches
        // have been swept (a product of few rows streams its weights from memory in the model, where other layers'
        // weights pass through the caches between two uses; timed with its weights in the caches, candidates that
        // are slower from memory can win).
        float ms = 0.f;
        bool ran = hipblasLtMatmul(st.handle, p.op, &one, W, p.a, X, p.b, &zero, Y, p.c, Y, p.c, &found[i].algo,
                                   st.workspace, WORKSPACE_BYTES, stream) == HIPBLAS_STATUS_SUCCESS;
        for (int run = 0; run < TIMED_RUNS && ran; ++run) {
            float one_ms = 0.f;
            if (st.sweep) hipMemsetAsync(st.sweep, run, SWEEP_BYTES, stream);
            hipEventRecord(t0, stream);
            ran = hipblasLtMatmul(st.handle, p.op, &one, W, p.a, X, p.b, &zero, Y, p.c, Y, p.c, &found[i].algo,
                                  st.workspace, WORKSPACE_BYTES, stream) == HIPBLAS_STATUS_SUCCESS &&
                  hipEventRecord(t1, stream) == hipSuccess && hipEventSynchronize(t1) == hipSuccess &&
                  hipEventElapsedTime(&one_ms, t0, t1) == hipSuccess;
            ms += one_ms;
        }
        if (!ran) continue;
        // the library's first candidate stays unless another is clearly faster, so that noise cannot choose
        if (best < 0 || ms < best_ms * (best == 0 ? CLEARLY : 1.f)) {
            best = i;
            best_ms = ms;
        }
    }
    if (t0) hipEventDestroy(t0);
    if (t1) hipEventDestroy(t1);
    if (best < 0) return false;
    p.algo = found[best].algo;
    p.workspace = found[best].workspaceSize;
    p.ok = true;
    p.tried_out = timed;
    return true;
}

}  // namespace

// Once per device, with that device current, outside any stream capture: creates the library handle and the
// workspace that its algorithms may use.  0 on success.
SIA_EXPORT int sia_blas_init() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) return 1;
    if (g_state[dev]) return 0;
    State* st = new State();
    if (hipblasLtCreate(&st->handle) != HIPBLAS_STATUS_SUCCESS) {
        delete st;
        return 2;
    }
    if (hipMalloc(&st->workspace, WORKSPACE_BYTES) != hipSuccess) {
        hipblasLtDestroy(st->handle);
        delete st;
        return 3;
    }
    g_state[dev] = st;
    return 0;
}

// While on, every product of up to TRY_OUT_ROWS rows whose shape has not been tried out yet runs the library's
// candidates on its own operands first (some tens of milliseconds, once per shape) and keeps the fastest; half a
// gigabyte of device memory is held meanwhile.  Not to be switched inside a stream capture.  For callers who
// know that the shapes they are running will recur many times, such as the runs before a graph is captured.
SIA_EXPORT int sia_blas_try_out(int on) {
    State* st = state_of_current_device();
    if (!st) return 1;
    st->try_out = on != 0;
    if (on && !st->sweep) {
        if (hipMalloc(&st->sweep, SWEEP_BYTES) != hipSuccess) st->sweep = nullptr;  // then the runs are timed warm
    } else if (!on && st->sweep) {
        hipFree(st->sweep);  // waits for the device: nothing that fills it is still running
        st->sweep = nullptr;
    }
    return 0;
}

// 0 if the library has an algorithm for the shape (found now, if the shape is new, and kept: nothing is launched or
// timed), else as sia_blas_mm.  For callers that cannot take another way once they have begun.
SIA_EXPORT int sia_blas_can(int M, int N, int K, int out_float) {
    State* st = state_of_current_device();
    if (!st) return 1;
    if (M <= 0 || N <= 0 || K <= 0) return 2;
    const uint64_t key = ((uint64_t)(uint32_t)M << 42) ^ ((uint64_t)(uint32_t)N << 21) ^ (uint64_t)(uint32_t)K ^
                         ((uint64_t)(out_float ? 1 : 0) << 63);
    auto it = st->plans.find(key);
    if (it == st->plans.end()) {
        Plan p;
        make_plan(*st, p, M, N, K, out_float != 0, false, nullptr, nullptr, nullptr, nullptr);
        it = st->plans.emplace(key, p).first;
    }
    return it->second.ok ? 0 : 3;
}

// 0: launched.  Anything else: nothing was launched (not initialised, or the library has no algorithm for the
// shape), and the caller takes another way.
SIA_EXPORT int sia_blas_mm(const void* X, const void* W, void* Y, int M, int N, int K, int out_float,
                           hipStream_t stream) {
    State* st = state_of_current_device();
    if (!st) return 1;
    if (M <= 0 || N <= 0 || K <= 0) return 2;
    // Plans chosen by timing are kept apart from the library's first choices (bit 62 of the key) and are used only
    // while the caller says that the shapes it runs will recur: the runs before a graph is captured and the capture
    // itself.  Every other call takes the first choice, so a product outside a graph never changes its algorithm
    // (and with it the last bits of its result) because some graph was captured in between.  Candidates are never
    // timed while the stream is being captured (a graph's shapes are met in the eager runs before its capture).
    const bool tuned = st->try_out && M <= TRY_OUT_ROWS;
    uint64_t key = ((uint64_t)(uint32_t)M << 42) ^ ((uint64_t)(uint32_t)N << 21) ^ (uint64_t)(uint32_t)K ^
                   ((uint64_t)(out_float ? 1 : 0) << 63) ^ ((uint64_t)(tuned ? 1 : 0) << 62);
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    const bool may_time = tuned && hipStreamIsCapturing(stream, &capturing) == hipSuccess &&
                          capturing == hipStreamCaptureStatusNone;
    auto it = st->plans.find(key);
    if (it == st->plans.end() && tuned && !may_time) {   // captured without a timed run before it: the first choice
        key ^= (uint64_t)1 << 62;
        it = st->plans.find(key);
    }
    if (it == st->plans.end()) {
        Plan p;
        make_plan(*st, p, M, N, K, out_float != 0, may_time, X, W, Y, stream);
        it = st->plans.emplace(key, p).first;
    }
    const Plan& p = it->second;
    if (!p.ok) return 3;
    const float one = 1.f, zero = 0.f;
    const hipblasStatus_t status = hipblasLtMatmul(st->handle, p.op, &one, W, p.a, X, p.b, &zero, Y, p.c, Y, p.c,
                                                   &p.algo, st->workspace, WORKSPACE_BYTES, stream);
    return status == HIPBLAS_STATUS_SUCCESS ? 0 : 4;
}
