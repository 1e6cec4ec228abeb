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

struct Plan {
    hipblasLtMatmulDesc_t op = nullptr;
    hipblasLtMatrixLayout_t a = nullptr, b = nullptr, c = nullptr;
    hipblasLtMatmulAlgo_t algo;
    size_t workspace = 0;
    bool ok = false;
};

struct State {
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

bool make_plan(State& st, Plan& p, int M, int N, int K, bool out_float) {
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
    hipblasLtMatmulHeuristicResult_t found[1];
    int n_found = 0;
    const hipblasStatus_t status =
        hipblasLtMatmulAlgoGetHeuristic(st.handle, p.op, p.a, p.b, p.c, p.c, pref, 1, found, &n_found);
    hipblasLtMatmulPreferenceDestroy(pref);
    if (status != HIPBLAS_STATUS_SUCCESS || n_found < 1 || found[0].workspaceSize > WORKSPACE_BYTES) return false;
    p.algo = found[0].algo;
    p.workspace = found[0].workspaceSize;
    p.ok = true;
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

// 0: launched.  Anything else: nothing was launched (not initialised, or the library has no algorithm for the
// shape), and the caller takes another way.
SIA_EXPORT int sia_blas_mm(const void* X, const void* W, void* Y, int M, int N, int K, int out_float,
                           hipStream_t stream) {
    State* st = state_of_current_device();
    if (!st) return 1;
    if (M <= 0 || N <= 0 || K <= 0) return 2;
    const uint64_t key = ((uint64_t)(uint32_t)M << 42) ^ ((uint64_t)(uint32_t)N << 21) ^ (uint64_t)(uint32_t)K ^
                         ((uint64_t)(out_float ? 1 : 0) << 63);
    auto it = st->plans.find(key);
    if (it == st->plans.end()) {
        Plan p;
        make_plan(*st, p, M, N, K, out_float != 0);
        it = st->plans.emplace(key, p).first;
    }
    const Plan& p = it->second;
    if (!p.ok) return 3;
    const float one = 1.f, zero = 0.f;
    const hipblasStatus_t status = hipblasLtMatmul(st->handle, p.op, &one, W, p.a, X, p.b, &zero, Y, p.c, Y, p.c,
                                                   &p.algo, st->workspace, WORKSPACE_BYTES, stream);
    return status == HIPBLAS_STATUS_SUCCESS ? 0 : 4;
}
